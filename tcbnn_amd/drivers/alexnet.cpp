// ImageNet-shaped AlexNet BNN: the layer wiring of the reference's alexnet.cu:143-177 (11x11
// stride-4 first layer with 2x2 pooling, a 5x5 layer, 192 / 384 channels, three FC layers) as a host
// loop over layer->forward(stream).
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "alexnet [--batch N] [--image 224] [--classes 1000] [--seed S] [--reps R] [--weights alexnet_imagenet.csv] "
        "[--input x.f32] [--out logits.f32] [--labels y.u32] [--variant popc|mfma_i8|mfma_f4]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 256;
    const unsigned output_size = o.classes ? o.classes : 1000;
    const unsigned image_height = o.image ? o.image : 224, image_width = image_height, image_channel = 3;
    const unsigned n_hidden = 4096;
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
        const int h1 = tcbnn_conv_out(image_height, 11, 4, 1, 2), h2 = tcbnn_conv_out(h1, 5, 1, 1, 2),
                  h5 = tcbnn_conv_out(h2, 3, 1, 1, 2);
        syn.binary_layer(121 * 3, 64);
        syn.binary_layer(25 * 64, 192);
        syn.binary_layer(9 * 192, 384);
        syn.binary_layer(9 * 384, 256);
        syn.binary_layer(9 * 256, 256);
        syn.binary_layer((size_t)h5 * h5 * 256, n_hidden);
        syn.binary_layer(n_hidden, n_hidden);
        syn.output_layer(n_hidden, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    InConv128LayerParam* bconv1 = new InConv128LayerParam("Conv1", image_height, image_width, 11, 11, 3, 64, batch, 4, 4, true, 2, 2);
    bconv1->initialize(images.data(), cfg());
    Conv128LayerParam* bconv2 = new Conv128LayerParam("Conv2", bconv1->output_height, bconv1->output_width, 5, 5, 64, 192, batch, 1, 1, true, 2, 2);
    bconv2->initialize(cfg(), bconv1->get_output_gpu());
    Conv128LayerParam* bconv3 = new Conv128LayerParam("Conv3", bconv2->output_height, bconv2->output_width, 3, 3, 192, 384, batch);
    bconv3->initialize(cfg(), bconv2->get_output_gpu());
    Conv128LayerParam* bconv4 = new Conv128LayerParam("Conv4", bconv3->output_height, bconv3->output_width, 3, 3, 384, 256, batch);
    bconv4->initialize(cfg(), bconv3->get_output_gpu());
    Conv128LayerParam* bconv5 = new Conv128LayerParam("Conv5", bconv4->output_height, bconv4->output_width, 3, 3, 256, 256, batch, 1, 1, true, 2, 2, true);
    bconv5->initialize(cfg(), bconv4->get_output_gpu());
    Fc128LayerParam* bfc1 = new Fc128LayerParam("Fc1", batch, (bconv5->output_height) * (bconv5->output_width) * 256, n_hidden);
    bfc1->initialize(cfg(), bconv5->get_output_gpu());
    Fc128LayerParam* bfc2 = new Fc128LayerParam("Fc2", batch, n_hidden, n_hidden);
    bfc2->initialize(cfg(), bfc1->get_output_gpu());
    Out128LayerParam* bout = new Out128LayerParam("Fout", batch, n_hidden, output_size);
    bout->initialize(cfg(), bfc2->get_output_gpu());

    Conv128LayerParam* convs[4] = {bconv2, bconv3, bconv4, bconv5};
    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    auto forward = [&]() {
        bconv1->forward(stream);
        for (Conv128LayerParam* c : convs) c->forward(stream);
        bfc1->forward(stream);
        bfc2->forward(stream);
        bout->forward(stream);
    };
    const double ms = driver::time_forward(forward, stream, o.warmup, o.reps);
    float* output = bout->download_output();
    double ops = 0;
    for (Conv128LayerParam* c : convs)
        ops += 2.0 * batch * c->buf_height * c->buf_width * c->output_channels * c->input_channels * c->filter_height * c->filter_width;
    ops += 2.0 * batch * ((double)bfc1->input_width * n_hidden + (double)n_hidden * n_hidden + (double)n_hidden * output_size);
    driver::report("alexnet", batch, ms, ops, output, output_size, o);

    delete bconv1;
    for (Conv128LayerParam* c : convs) delete c;
    delete bfc1; delete bfc2; delete bout;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
