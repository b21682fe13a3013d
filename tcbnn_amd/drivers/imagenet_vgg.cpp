// ImageNet-shaped VGG-16 BNN: the layer wiring of the reference's imagenet_vgg.cu:217-286 (13
// 3x3 convolution layers, 2x2 pooling after layers 2, 4, 7, 10 and 13, three FC layers) as a host
// loop over layer->forward(stream).
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "imagenet_vgg [--batch N] [--image 224] [--classes 1000] [--seed S] [--reps R] [--weights vgg_imagenet.csv] "
        "[--input x.f32] [--out logits.f32] [--labels y.u32] [--variant popc|mfma_i8|mfma_f4]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 256;
    const unsigned output_size = o.classes ? o.classes : 1000;
    const unsigned image_height = o.image ? o.image : 224, image_width = image_height, image_channel = 3;
    const unsigned filter_height = 3, filter_width = 3, n_hidden = 4096;
    const size_t in_size = (size_t)batch * image_channel * image_height * image_width;

    std::vector<float> images = o.input.empty() ? driver::synthetic_input(o.seed, in_size, false)
                                                : driver::read_floats(o.input, in_size);
    // output channels and pooling of convolution layers 2..13
    const int n_conv = 12;
    const int cout[n_conv] = {64, 128, 128, 256, 256, 256, 512, 512, 512, 512, 512, 512};
    const int pool[n_conv] = {2, 1, 2, 1, 1, 2, 1, 1, 2, 1, 1, 2};
    driver::Synthetic syn(o.seed);
    FILE* config_file = NULL;
    const float* cursor = NULL;
    if (!o.weights.empty()) {
        config_file = fopen(o.weights.c_str(), "r");
        CHECK_NULL_POINTER(config_file);
    } else {
        syn.binary_layer(9 * 3, 64);
        int cin = 64, h = image_height;
        for (int i = 0; i < n_conv; ++i) {
            syn.binary_layer(9 * cin, cout[i]);
            cin = cout[i];
            h = tcbnn_conv_out(h, 3, 1, 1, pool[i]);
        }
        syn.binary_layer((size_t)h * h * 512, n_hidden);
        syn.binary_layer(n_hidden, n_hidden);
        syn.output_layer(n_hidden, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    InConv128LayerParam* bconv1 = new InConv128LayerParam("Conv1", image_height, image_width, filter_height, filter_width, 3, 64, batch);
    bconv1->initialize(images.data(), cfg());
    Conv128LayerParam* convs[n_conv];
    {
        char name[16];
        unsigned h = bconv1->output_height, w = bconv1->output_width;
        int cin = 64;
        uint32_t* prev = bconv1->get_output_gpu();
        for (int i = 0; i < n_conv; ++i) {
            snprintf(name, sizeof(name), "Conv%d", i + 2);
            // the last convolution layer writes the FC-ready layout (imagenet_vgg.cu:274-277)
            convs[i] = new Conv128LayerParam(name, h, w, filter_height, filter_width, cin, cout[i], batch, 1, 1, true,
                                             pool[i], pool[i], i == n_conv - 1);
            convs[i]->initialize(cfg(), prev);
            prev = convs[i]->get_output_gpu();
            h = convs[i]->output_height;
            w = convs[i]->output_width;
            cin = cout[i];
        }
    }
    Conv128LayerParam* bconv13 = convs[n_conv - 1];
    Fc128LayerParam* bfc1 = new Fc128LayerParam("Fc1", batch, (bconv13->output_height) * (bconv13->output_width) * 512, n_hidden);
    bfc1->initialize(cfg(), bconv13->get_output_gpu());
    Fc128LayerParam* bfc2 = new Fc128LayerParam("Fc2", batch, n_hidden, n_hidden);
    bfc2->initialize(cfg(), bfc1->get_output_gpu());
    Out128LayerParam* bout = new Out128LayerParam("Fout", batch, n_hidden, output_size);
    bout->initialize(cfg(), bfc2->get_output_gpu());

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
        ops += 2.0 * batch * c->buf_height * c->buf_width * c->output_channels * c->input_channels * 9;
    ops += 2.0 * batch * ((double)bfc1->input_width * n_hidden + (double)n_hidden * n_hidden + (double)n_hidden * output_size);
    driver::report("imagenet_vgg", batch, ms, ops, output, output_size, o);

    delete bconv1;
    for (Conv128LayerParam* c : convs) delete c;
    delete bfc1; delete bfc2; delete bout;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
