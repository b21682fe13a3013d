// ImageNet-shaped ResNet-18 BNN in the textbook wiring: 7x7 stride-2 first layer + 3x3 stride-2
// max-pool, a 1x1 stride-2 binarized convolution as the shortcut at every stage entry (its
// pre-threshold sums are the injected residual), global average pool of the last residual + fp32 FC.
// The reference has no driver for this wiring (imagenet_resnet.cu:223-325 uses a stride-4 first layer,
// max-pooled residuals as shortcuts and a binarized FC head); the layers are the reference's
// InConv128 / Conv128 classes plus Pool128 and AvgPoolFc.
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "imagenet_resnet_textbook [--batch N] [--image 224] [--classes 1000] [--seed S] [--reps R] "
        "[--weights FILE] [--input x.f32] [--out logits.f32] [--labels y.u32] [--variant popc|mfma_i8|mfma_f4]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 256;
    const unsigned output_size = o.classes ? o.classes : 1000;
    const unsigned image_height = o.image ? o.image : 224, image_width = image_height, image_channel = 3;
    const size_t in_size = (size_t)batch * image_channel * image_height * image_width;

    std::vector<float> images = o.input.empty() ? driver::synthetic_input(o.seed, in_size, false)
                                                : driver::read_floats(o.input, in_size);
    const int ch[5] = {64, 64, 128, 256, 512};
    driver::Synthetic syn(o.seed);
    FILE* config_file = NULL;
    const float* cursor = NULL;
    if (!o.weights.empty()) {
        config_file = fopen(o.weights.c_str(), "r");
        CHECK_NULL_POINTER(config_file);
    } else {  // the order the layers are initialized in
        syn.binary_layer(49 * 3, 64);
        for (int k = 0; k < 4; ++k) syn.binary_layer(9 * 64, 64);
        for (int s = 2; s <= 4; ++s) {
            syn.binary_layer(ch[s - 1], ch[s]);      // shortcut 1x1
            syn.binary_layer(9 * ch[s - 1], ch[s]);  // block 1 conv 1
            for (int k = 0; k < 3; ++k) syn.binary_layer(9 * ch[s], ch[s]);
        }
        syn.fp32_layer(512, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    InConv128LayerParam* bconv1 = new InConv128LayerParam("Conv1", image_height, image_width, 7, 7, 3, 64, batch, 2, 2,
                                                          true, 1, 1, true);  // save residual
    bconv1->initialize(images.data(), cfg());
    Pool128LayerParam* pool1 = new Pool128LayerParam("Pool1", bconv1->output_height, bconv1->output_width, 64, batch,
                                                     3, 2, 1, true);
    pool1->initialize(bconv1->get_output_gpu(), bconv1->get_output_residual_gpu());

    std::vector<Conv128LayerParam*> convs;
    auto add = [&](Conv128LayerParam* c, uin32* in, int* res = NULL) {
        c->initialize(cfg(), in, res);
        convs.push_back(c);
        return c;
    };
    unsigned h = pool1->output_height, w = pool1->output_width;
    // stage 1: two blocks on the pooled first-layer output
    Conv128LayerParam* b1c1 = add(new Conv128LayerParam("L1B1C1", h, w, 3, 3, 64, 64, batch), pool1->get_output_gpu());
    Conv128LayerParam* b1c2 = add(new Conv128LayerParam("L1B1C2", h, w, 3, 3, 64, 64, batch, 1, 1, true, 1, 1, false, true, true, 64),
                                  b1c1->get_output_gpu(), pool1->get_output_residual_gpu());
    Conv128LayerParam* b2c1 = add(new Conv128LayerParam("L1B2C1", h, w, 3, 3, 64, 64, batch), b1c2->get_output_gpu());
    Conv128LayerParam* prev = add(new Conv128LayerParam("L1B2C2", h, w, 3, 3, 64, 64, batch, 1, 1, true, 1, 1, false, true, true, 64),
                                  b2c1->get_output_gpu(), b1c2->get_output_residual_gpu());
    char name[16];
    for (int s = 2; s <= 4; ++s) {
        const int cin = ch[s - 1], cout = ch[s];
        snprintf(name, sizeof(name), "L%dDS", s);  // shortcut: 1x1 stride 2, only its residual is used
        Conv128LayerParam* ds = add(new Conv128LayerParam(name, h, w, 1, 1, cin, cout, batch, 2, 2, true, 1, 1, false, true),
                                    prev->get_output_gpu());
        snprintf(name, sizeof(name), "L%dB1C1", s);
        Conv128LayerParam* c1 = add(new Conv128LayerParam(name, h, w, 3, 3, cin, cout, batch, 2, 2), prev->get_output_gpu());
        h = c1->output_height;
        w = c1->output_width;
        snprintf(name, sizeof(name), "L%dB1C2", s);
        Conv128LayerParam* c2 = add(new Conv128LayerParam(name, h, w, 3, 3, cout, cout, batch, 1, 1, true, 1, 1, false, true, true, cout),
                                    c1->get_output_gpu(), ds->get_output_residual_gpu());
        snprintf(name, sizeof(name), "L%dB2C1", s);
        Conv128LayerParam* c3 = add(new Conv128LayerParam(name, h, w, 3, 3, cout, cout, batch), c2->get_output_gpu());
        snprintf(name, sizeof(name), "L%dB2C2", s);
        prev = add(new Conv128LayerParam(name, h, w, 3, 3, cout, cout, batch, 1, 1, true, 1, 1, false, true, true, cout),
                   c3->get_output_gpu(), c2->get_output_residual_gpu());
    }
    AvgPoolFcLayerParam* head = new AvgPoolFcLayerParam("Fout", h, w, 512, batch, output_size);
    head->initialize(cfg(), prev->get_output_residual_gpu());

    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    auto forward = [&]() {
        bconv1->forward(stream);
        pool1->forward(stream);
        for (Conv128LayerParam* c : convs) c->forward(stream);
        head->forward(stream);
    };
    const double ms = driver::time_forward(forward, stream, o.warmup, o.reps);
    float* output = head->download_output();
    double ops = 0;
    for (Conv128LayerParam* c : convs)
        ops += 2.0 * batch * c->buf_height * c->buf_width * c->output_channels * c->input_channels * c->filter_height *
               c->filter_width;
    driver::report("imagenet_resnet_textbook", batch, ms, ops, output, output_size, o);

    delete bconv1;
    delete pool1;
    for (Conv128LayerParam* c : convs) delete c;
    delete head;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
