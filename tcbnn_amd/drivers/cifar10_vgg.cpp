// CIFAR-10-shaped VGG-small BNN: the layer wiring of the reference's cifar10_vgg.cu:162-199
// as a host loop over layer->forward(stream).
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "cifar10_vgg [--batch N] [--seed S] [--reps R] [--weights vgg_cifar10.csv] [--input x.f32] "
        "[--out logits.f32] [--labels y.u32] [--variant popc|mfma_i8|mfma_f4]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 256;
    const unsigned output_size = o.classes ? o.classes : 10;
    const unsigned image_height = o.image ? o.image : 32, image_width = image_height, image_channel = 3;
    const unsigned filter_height = 3, filter_width = 3, n_hidden = 1024;
    const size_t in_size = (size_t)batch * image_channel * image_height * image_width;

    std::vector<float> images = o.input.empty() ? driver::synthetic_input(o.seed, in_size, false)
                                                : driver::read_floats(o.input, in_size);
    driver::Synthetic syn(o.seed);
    FILE* config_file = NULL;
    const float* cursor = NULL;
    if (!o.weights.empty()) {
        config_file = fopen(o.weights.c_str(), "r");
        CHECK_NULL_POINTER(config_file);
    } else {
        const unsigned hw = image_height / 8;
        syn.binary_layer(9 * 3, 128);
        syn.binary_layer(9 * 128, 128);
        syn.binary_layer(9 * 128, 256);
        syn.binary_layer(9 * 256, 256);
        syn.binary_layer(9 * 256, 512);
        syn.binary_layer(9 * 512, 512);
        syn.binary_layer((size_t)hw * hw * 512, n_hidden);
        syn.binary_layer(n_hidden, n_hidden);
        syn.output_layer(n_hidden, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    InConv128LayerParam* bconv1 = new InConv128LayerParam("Conv1", image_height, image_width, filter_height,
                                                          filter_width, 3, 128, batch);
    bconv1->initialize(images.data(), cfg());
    Conv128LayerParam* bconv2 = new Conv128LayerParam("Conv2", bconv1->output_height, bconv1->output_width,
                                                      filter_height, filter_width, 128, 128, batch, 1, 1, true, 2, 2, false);
    bconv2->initialize(cfg(), bconv1->get_output_gpu());
    Conv128LayerParam* bconv3 = new Conv128LayerParam("Conv3", bconv2->output_height, bconv2->output_width,
                                                      filter_height, filter_width, 128, 256, batch);
    bconv3->initialize(cfg(), bconv2->get_output_gpu());
    Conv128LayerParam* bconv4 = new Conv128LayerParam("Conv4", bconv3->output_height, bconv3->output_width,
                                                      filter_height, filter_width, 256, 256, batch, 1, 1, true, 2, 2, false);
    bconv4->initialize(cfg(), bconv3->get_output_gpu());
    Conv128LayerParam* bconv5 = new Conv128LayerParam("Conv5", bconv4->output_height, bconv4->output_width,
                                                      filter_height, filter_width, 256, 512, batch);
    bconv5->initialize(cfg(), bconv4->get_output_gpu());
    Conv128LayerParam* bconv6 = new Conv128LayerParam("Conv6", bconv5->output_height, bconv5->output_width,
                                                      filter_height, filter_width, 512, 512, batch, 1, 1, true, 2, 2, true);
    bconv6->initialize(cfg(), bconv5->get_output_gpu());
    Fc128LayerParam* bfc1 = new Fc128LayerParam("Fc1", batch, (bconv6->output_height) * (bconv6->output_width) * 512, n_hidden);
    bfc1->initialize(cfg(), bconv6->get_output_gpu());
    Fc128LayerParam* bfc2 = new Fc128LayerParam("Fc2", batch, n_hidden, n_hidden);
    bfc2->initialize(cfg(), bfc1->get_output_gpu());
    Out128LayerParam* bout = new Out128LayerParam("Fout", batch, n_hidden, output_size);
    bout->initialize(cfg(), bfc2->get_output_gpu());

    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    auto forward = [&]() {
        bconv1->forward(stream);
        bconv2->forward(stream);
        bconv3->forward(stream);
        bconv4->forward(stream);
        bconv5->forward(stream);
        bconv6->forward(stream);
        bfc1->forward(stream);
        bfc2->forward(stream);
        bout->forward(stream);
    };
    const double ms = driver::time_forward(forward, stream, o.warmup, o.reps);
    float* output = bout->download_output();
    double ops = 0;
    Conv128LayerParam* convs[] = {bconv2, bconv3, bconv4, bconv5, bconv6};
    for (Conv128LayerParam* c : convs)
        ops += 2.0 * batch * c->buf_height * c->buf_width * c->output_channels * c->input_channels * 9;
    ops += 2.0 * batch * ((double)bfc1->input_width * n_hidden + (double)n_hidden * n_hidden + n_hidden * output_size);
    driver::report("cifar10_vgg", batch, ms, ops, output, output_size, o);

    delete bconv1; delete bconv2; delete bconv3; delete bconv4; delete bconv5; delete bconv6;
    delete bfc1; delete bfc2; delete bout;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
