// ImageNet-shaped ResNet-18 BNN: the 19 layer objects and residual wiring of the reference's
// imagenet_resnet.cu:223-325 (7x7 stride-4 stem with saved residual; the int32 pre-threshold
// residual carried between blocks, 2x2-max-pooled at stage entry and injected into the first
// residual_channels output channels; binarized FC 25088->512; fp32 output layer), run as a host
// loop over layer->forward(stream) instead of one cooperative kernel.
#include "driver_common.hpp"

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv,
        "imagenet_resnet [--batch N] [--image 224] [--classes 1000] [--seed S] [--reps R] "
        "[--weights resnet_imagenet.csv] [--input x.f32] [--out logits.f32] [--labels y.u32] [--variant popc|mfma_i8|mfma_f4] "
        "[--packed-input]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 256;
    const unsigned output_size = o.classes ? o.classes : 1000;
    const unsigned image_height = o.image ? o.image : 224, image_width = image_height, image_channel = 3;
    const size_t in_size = (size_t)batch * image_channel * image_height * image_width;

    std::vector<float> images = o.input.empty() ? driver::synthetic_input(o.seed, in_size, false)
                                                : driver::read_floats(o.input, in_size);

    // channel plan of the four stages
    const int ch[5] = {64, 64, 128, 256, 512};
    driver::Synthetic syn(o.seed);
    FILE* config_file = NULL;
    const float* cursor = NULL;
    if (!o.weights.empty()) {
        config_file = fopen(o.weights.c_str(), "r");
        CHECK_NULL_POINTER(config_file);
    } else {
        syn.binary_layer(49 * 3, 64);
        for (int s = 1; s <= 4; ++s) {
            syn.binary_layer(9 * ch[s - 1], ch[s]);
            for (int k = 0; k < 3; ++k) syn.binary_layer(9 * ch[s], ch[s]);
        }
        const int h7 = tcbnn_conv_out(tcbnn_conv_out(tcbnn_conv_out(tcbnn_conv_out(image_height, 7, 4, 1, 1), 3, 2, 1, 1), 3, 2, 1, 1), 3, 2, 1, 1);
        syn.binary_layer((size_t)h7 * h7 * 512, 512);
        syn.output_layer(512, output_size);
        cursor = syn.values.data();
    }
    auto cfg = [&]() {
        return config_file ? tcbnn_host::ConfigSource(config_file)
                           : tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size());
    };

    //Layer-0
    InConv128LayerParam* bconv1 = new InConv128LayerParam("Conv1", image_height, image_width,
            7, 7, 3, 64, batch, 4, 4, true, 1, 1, true);  // save residual
    if (o.packed_input) bconv1->use_packed_input();
    bconv1->initialize(images.data(), cfg());
    //Layer-1
    Conv128LayerParam* l1b1c1 = new Conv128LayerParam("L1B1C1", bconv1->output_height, bconv1->output_width, 3, 3, 64, 64, batch);
    l1b1c1->initialize(cfg(), bconv1->get_output_gpu());
    Conv128LayerParam* l1b1c2 = new Conv128LayerParam("L1B1C2", l1b1c1->output_height, l1b1c1->output_width, 3, 3, 64, 64, batch, 1, 1, true, 1, 1, false, true, true, 64);
    l1b1c2->initialize(cfg(), l1b1c1->get_output_gpu(), bconv1->get_output_residual_gpu());
    Conv128LayerParam* l1b2c1 = new Conv128LayerParam("L1B2C1", l1b1c2->output_height, l1b1c2->output_width, 3, 3, 64, 64, batch);
    l1b2c1->initialize(cfg(), l1b1c2->get_output_gpu());
    Conv128LayerParam* l1b2c2 = new Conv128LayerParam("L1B2C2", l1b2c1->output_height, l1b2c1->output_width, 3, 3, 64, 64, batch, 1, 1, true, 1, 1, false, true, true, 128);
    l1b2c2->initialize(cfg(), l1b2c1->get_output_gpu(), l1b1c2->get_output_residual_gpu());
    //Layer-2
    Conv128LayerParam* l2b1c1 = new Conv128LayerParam("L2B1C1", l1b2c2->output_height, l1b2c2->output_width, 3, 3, 64, 128, batch, 2, 2);
    l2b1c1->initialize(cfg(), l1b2c2->get_output_gpu());
    Conv128LayerParam* l2b1c2 = new Conv128LayerParam("L2B1C2", l2b1c1->output_height, l2b1c1->output_width, 3, 3, 128, 128, batch, 1, 1, true, 1, 1, false, true, true, 128, true);
    l2b1c2->initialize(cfg(), l2b1c1->get_output_gpu(), l1b2c2->get_output_residual_gpu());
    Conv128LayerParam* l2b2c1 = new Conv128LayerParam("L2B2C1", l2b1c2->output_height, l2b1c2->output_width, 3, 3, 128, 128, batch, 1, 1);
    l2b2c1->initialize(cfg(), l2b1c2->get_output_gpu());
    Conv128LayerParam* l2b2c2 = new Conv128LayerParam("L2B2C2", l2b2c1->output_height, l2b2c1->output_width, 3, 3, 128, 128, batch, 1, 1, true, 1, 1, false, true, true, 128);
    l2b2c2->initialize(cfg(), l2b2c1->get_output_gpu(), l2b1c2->get_output_residual_gpu());
    //Layer-3
    Conv128LayerParam* l3b1c1 = new Conv128LayerParam("L3B1C1", l2b2c2->output_height, l2b2c2->output_width, 3, 3, 128, 256, batch, 2, 2);
    l3b1c1->initialize(cfg(), l2b2c2->get_output_gpu());
    Conv128LayerParam* l3b1c2 = new Conv128LayerParam("L3B1C2", l3b1c1->output_height, l3b1c1->output_width, 3, 3, 256, 256, batch, 1, 1, true, 1, 1, false, true, true, 128, true);
    l3b1c2->initialize(cfg(), l3b1c1->get_output_gpu(), l2b2c2->get_output_residual_gpu());
    Conv128LayerParam* l3b2c1 = new Conv128LayerParam("L3B2C1", l3b1c2->output_height, l3b1c2->output_width, 3, 3, 256, 256, batch, 1, 1);
    l3b2c1->initialize(cfg(), l3b1c2->get_output_gpu());
    Conv128LayerParam* l3b2c2 = new Conv128LayerParam("L3B2C2", l3b2c1->output_height, l3b2c1->output_width, 3, 3, 256, 256, batch, 1, 1, true, 1, 1, false, true, true, 256);
    l3b2c2->initialize(cfg(), l3b2c1->get_output_gpu(), l3b1c2->get_output_residual_gpu());
    //Layer-4
    Conv128LayerParam* l4b1c1 = new Conv128LayerParam("L4B1C1", l3b2c2->output_height, l3b2c2->output_width, 3, 3, 256, 512, batch, 2, 2);
    l4b1c1->initialize(cfg(), l3b2c2->get_output_gpu());
    Conv128LayerParam* l4b1c2 = new Conv128LayerParam("L4B1C2", l4b1c1->output_height, l4b1c1->output_width, 3, 3, 512, 512, batch, 1, 1, true, 1, 1, false, true, true, 256, true);
    l4b1c2->initialize(cfg(), l4b1c1->get_output_gpu(), l3b2c2->get_output_residual_gpu());
    Conv128LayerParam* l4b2c1 = new Conv128LayerParam("L4B2C1", l4b1c2->output_height, l4b1c2->output_width, 3, 3, 512, 512, batch, 1, 1);
    l4b2c1->initialize(cfg(), l4b1c2->get_output_gpu());
    Conv128LayerParam* l4b2c2 = new Conv128LayerParam("L4B2C2", l4b2c1->output_height, l4b2c1->output_width, 3, 3, 512, 512, batch, 1, 1, true, 1, 1, true, false, true, 512);
    l4b2c2->initialize(cfg(), l4b2c1->get_output_gpu(), l4b1c2->get_output_residual_gpu());
    //Layer-5
    Fc128LayerParam* bfc1 = new Fc128LayerParam("Fc1", batch, (l4b2c2->output_height) * (l4b2c2->output_width) * 512, 512);
    bfc1->initialize(cfg(), l4b2c2->get_output_gpu());
    Out128LayerParam* bout = new Out128LayerParam("Fout", batch, 512, output_size);
    bout->initialize(cfg(), bfc1->get_output_gpu());

    Conv128LayerParam* convs[16] = {l1b1c1, l1b1c2, l1b2c1, l1b2c2, l2b1c1, l2b1c2, l2b2c1, l2b2c2,
                                    l3b1c1, l3b1c2, l3b2c1, l3b2c2, l4b1c1, l4b1c2, l4b2c1, l4b2c2};
    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    auto forward = [&]() {
        bconv1->forward(stream);
        for (Conv128LayerParam* c : convs) c->forward(stream);
        bfc1->forward(stream);
        bout->forward(stream);
    };
    const double ms = driver::time_forward(forward, stream, o.warmup, o.reps);
    float* output = bout->download_output();
    double ops = 0;
    for (Conv128LayerParam* c : convs)
        ops += 2.0 * batch * c->buf_height * c->buf_width * c->output_channels * c->input_channels * 9;
    ops += 2.0 * batch * ((double)bfc1->input_width * 512 + 512.0 * output_size);
    driver::report("imagenet_resnet", batch, ms, ops, output, output_size, o);

    delete bconv1;
    for (Conv128LayerParam* c : convs) delete c;
    delete bfc1;
    delete bout;
    if (config_file) fclose(config_file);
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
