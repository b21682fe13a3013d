// MNIST-shaped binarized MLP 784 -> 1024 -> 1024 -> 1024 -> 10: the layer wiring of the
// reference's mnist_mlp.cu:111-124 as a host loop over layer->forward(stream).
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "mnist_mlp [--batch N] [--seed S] [--reps R] [--weights mlp_mnist.csv] [--input x.f32] [--out logits.f32] [--labels y.u32] "
        "[--variant popc|mfma_i8|mfma_f4]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 8192;
    const unsigned output_size = o.classes ? o.classes : 10;
    const unsigned n_hidden = 1024;
    const unsigned image_size = o.image ? o.image * o.image : 28 * 28;

    std::vector<float> images = o.input.empty() ? driver::synthetic_input(o.seed, (size_t)batch * image_size, true)
                                                : driver::read_floats(o.input, (size_t)batch * image_size);
    driver::Synthetic syn(o.seed);
    FILE* config_file = NULL;
    const float* cursor = NULL;
    if (!o.weights.empty()) {
        config_file = fopen(o.weights.c_str(), "r");
        CHECK_NULL_POINTER(config_file);
    } else {
        syn.binary_layer(image_size, n_hidden);
        syn.binary_layer(n_hidden, n_hidden);
        syn.binary_layer(n_hidden, n_hidden);
        syn.output_layer(n_hidden, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    In128LayerParam* bin = new In128LayerParam("Fin", batch, image_size);
    bin->initialize(images.data());
    Fc128LayerParam* bfc1 = new Fc128LayerParam("Fc1", batch, image_size, n_hidden);
    bfc1->initialize(cfg(), bin->get_output_gpu());
    Fc128LayerParam* bfc2 = new Fc128LayerParam("Fc2", batch, n_hidden, n_hidden);
    bfc2->initialize(cfg(), bfc1->get_output_gpu());
    Fc128LayerParam* bfc3 = new Fc128LayerParam("Fc3", batch, n_hidden, n_hidden);
    bfc3->initialize(cfg(), bfc2->get_output_gpu());
    Out128LayerParam* bout = new Out128LayerParam("Fout", batch, n_hidden, output_size);
    bout->initialize(cfg(), bfc3->get_output_gpu());

    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    auto forward = [&]() {
        bin->forward(stream);
        bfc1->forward(stream);
        bfc2->forward(stream);
        bfc3->forward(stream);
        bout->forward(stream);
    };
    const double ms = driver::time_forward(forward, stream, o.warmup, o.reps);
    float* output = bout->download_output();
    const double ops = 2.0 * batch * ((double)image_size * n_hidden + 2.0 * n_hidden * n_hidden + n_hidden * output_size);
    driver::report("mnist_mlp", batch, ms, ops, output, output_size, o);

    delete bin;
    delete bfc1;
    delete bfc2;
    delete bfc3;
    delete bout;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
