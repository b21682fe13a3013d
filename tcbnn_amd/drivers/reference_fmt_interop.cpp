// Self-check of the reference-layout accessors of the layer classes: a small residual network is run
// twice on the same synthetic parameters, once with engine-layout buffers between the layers and once
// with EVERY hand-over (activation bits and residuals) going through device buffers in the reference's
// own tile layouts, as if each neighbour were a layer of the reference (kernel.cuh:170, 222-223,
// 650-668, 811-824).  Logits, exported tiles and residuals must agree exactly; prints one JSON line
// and exits 0, or says what differs and exits 1.
#include "driver_common.hpp"

template <class T>
static std::vector<T> to_host(const T* dev, size_t n) {
    std::vector<T> v(n);
    HIP_SAFE_CALL(hipDeviceSynchronize());
    HIP_SAFE_CALL(hipMemcpy(v.data(), dev, n * sizeof(T), hipMemcpyDeviceToHost));
    return v;
}

int main(int argc, char** argv) {
    driver::Options o = driver::parse(argc, argv, "reference_fmt_interop [--batch N] [--seed S] [--variant V] [--oversize-input]");
    HIP_SAFE_CALL(hipSetDevice(0));
    const unsigned batch = o.batch ? o.batch : 12, image = 16, ch = 64, n_hidden = 256, classes = 10;

    std::vector<float> images = driver::synthetic_input(o.seed, (size_t)batch * 3 * image * image, false);
    driver::Synthetic syn(o.seed);
    syn.binary_layer(3 * 3 * 3, ch);       // stem, saves its residual
    syn.binary_layer(3 * 3 * ch, ch);      // c1
    syn.binary_layer(3 * 3 * ch, ch);      // c2: injects the stem's residual, saves its own
    syn.binary_layer(3 * 3 * ch, 2 * ch);  // c3: stride 2
    syn.binary_layer(3 * 3 * 2 * ch, 2 * ch);  // c4: injects c2's residual through the 2x2 max, FC-ready output
    const unsigned feats = (image / 2) * (image / 2) * 2 * ch;
    syn.binary_layer(feats, n_hidden);
    syn.output_layer(n_hidden, classes);

    hipStream_t stream;
    HIP_SAFE_CALL(hipStreamCreate(&stream));
    std::vector<float> logits[2];
    std::vector<uin32> tiles[2];
    std::vector<int> resid[2];
    for (int pass = 0; pass < 2; ++pass) {
        const bool via_ref = pass == 1;
        const float* cursor = syn.values.data();
        auto cfg = [&]() { return tcbnn_host::ConfigSource(&cursor, syn.values.data() + syn.values.size()); };
        InConv128LayerParam stem("Conv1", image, image, 3, 3, 3, ch, batch, 1, 1, true, 1, 1, true);
        stem.initialize(images.data(), cfg());
        stem.forward(stream);
        uin32* stem_out = via_ref ? stem.get_output_gpu_reference_fmt(stream) : stem.get_output_gpu();
        int* stem_res = via_ref ? stem.get_output_residual_gpu_reference(stream) : stem.get_output_residual_gpu();

        Conv128LayerParam c1("C1", image, image, 3, 3, ch, ch, batch);
        c1.initialize(cfg(), stem_out);
        if (via_ref) c1.set_input_gpu_reference_fmt(stem_out, stream);
        c1.forward(stream);
        uin32* c1_out = via_ref ? c1.get_output_gpu_reference_fmt(stream) : c1.get_output_gpu();

        Conv128LayerParam c2("C2", image, image, 3, 3, ch, ch, batch, 1, 1, true, 1, 1, false, true, true, ch);
        c2.initialize(cfg(), c1_out, stem_res);
        if (via_ref) {
            c2.set_input_gpu_reference_fmt(c1_out, stream);
            c2.set_input_residual_gpu_reference(stem_res, stream);
        }
        c2.forward(stream);
        uin32* c2_out = via_ref ? c2.get_output_gpu_reference_fmt(stream) : c2.get_output_gpu();
        int* c2_res = via_ref ? c2.get_output_residual_gpu_reference(stream) : c2.get_output_residual_gpu();

        Conv128LayerParam c3("C3", image, image, 3, 3, ch, 2 * ch, batch, 2, 2);
        c3.initialize(cfg(), c2_out);
        if (via_ref) c3.set_input_gpu_reference_fmt(c2_out, stream);
        c3.forward(stream);
        uin32* c3_out = via_ref ? c3.get_output_gpu_reference_fmt(stream) : c3.get_output_gpu();

        Conv128LayerParam c4("C4", image / 2, image / 2, 3, 3, 2 * ch, 2 * ch, batch, 1, 1, true, 1, 1, true, false,
                             true, ch, true);
        c4.initialize(cfg(), c3_out, c2_res);
        if (via_ref) {
            c4.set_input_gpu_reference_fmt(c3_out, stream);
            c4.set_input_residual_gpu_reference(c2_res, stream);
        }
        c4.forward(stream);
        uin32* c4_out = via_ref ? c4.get_output_gpu_reference_fmt(stream) : c4.get_output_gpu();

        Fc128LayerParam fc("Fc1", batch, feats, n_hidden);
        fc.initialize(cfg(), c4_out);
        if (via_ref) fc.set_input_gpu_reference_fmt(c4_out, stream);
        fc.forward(stream);
        uin32* fc_out = via_ref ? fc.get_output_gpu_reference_fmt(stream) : fc.get_output_gpu();

        Out128LayerParam out("Fout", batch, n_hidden, classes);
        out.initialize(cfg(), fc_out);
        if (via_ref) out.set_input_gpu_reference_fmt(fc_out, stream);
        out.forward(stream);
        HIP_SAFE_CALL(hipStreamSynchronize(stream));

        float* l = out.download_output();
        logits[pass].assign(l, l + (size_t)batch * classes);
        // the exported tiles against the download path of the same layer, and the two passes against each other
        uin32* t = c2.download_output();
        tiles[pass].assign(t, t + (size_t)c2.output_bit_size() * 4);
        const size_t rn = (size_t)image * image * PAD8(batch) * PAD128(ch);
        resid[pass] = to_host(c2.get_output_residual_gpu_reference(stream), rn);
        if (via_ref) {
            if (to_host(c2_out, tiles[1].size()) != tiles[1]) {
                fprintf(stderr, "C2: get_output_gpu_reference_fmt() differs from download_output()\n");
                return 1;
            }
            if (to_host(c2_res, rn) != resid[1]) {
                fprintf(stderr, "C2: reference-layout residual changed between two exports\n");
                return 1;
            }
        }
    }
    if (logits[0] != logits[1] || tiles[0] != tiles[1] || resid[0] != resid[1]) {
        fprintf(stderr, "reference-layout hand-over changed the result: logits %s, C2 tiles %s, C2 residual %s\n",
                logits[0] == logits[1] ? "same" : "DIFFER", tiles[0] == tiles[1] ? "same" : "DIFFER",
                resid[0] == resid[1] ? "same" : "DIFFER");
        return 1;
    }
    // A second batch through the same first-layer object: set_input() must give what a freshly initialized layer
    // gives on that batch, and must refuse (print + exit(-1)) a batch beyond the bound the 16-bit residual format
    // was chosen for at initialize().
    {
        const float* cursor = syn.values.data();
        tcbnn_host::ConfigSource cfg(&cursor, syn.values.data() + syn.values.size());
        InConv128LayerParam stem("Conv1", image, image, 3, 3, 3, ch, batch, 1, 1, true, 1, 1, true);
        stem.use_packed_input();  // (set_input() must also renew the packed copy; `fresh` below reads the plain one)
        stem.initialize(images.data(), cfg);
        std::vector<float> half(images);
        for (float& v : half) v *= 0.5f;
        stem.set_input(half.data());
        stem.forward(stream);
        uin32* t = stem.download_output();
        std::vector<uin32> got(t, t + (size_t)stem.output_bit_size() * 4);
        const float* cursor2 = syn.values.data();
        tcbnn_host::ConfigSource cfg2(&cursor2, syn.values.data() + syn.values.size());
        InConv128LayerParam fresh("Conv1", image, image, 3, 3, 3, ch, batch, 1, 1, true, 1, 1, true);
        fresh.initialize(half.data(), cfg2);
        fresh.forward(stream);
        uin32* t2 = fresh.download_output();
        if (got != std::vector<uin32>(t2, t2 + (size_t)fresh.output_bit_size() * 4)) {
            fprintf(stderr, "Conv1: set_input() and a fresh initialize() disagree on the same batch\n");
            return 1;
        }
        // a batch LARGER than the one the layer was initialized with, but within what the chosen residual format
        // holds: accepted (the recorded bound is raised), and again what a fresh layer gives
        {
            std::vector<float> twice(images);
            for (float& v : twice) v *= 2.0f;
            stem.set_input(twice.data());
            stem.forward(stream);
            int* r1 = stem.get_output_residual_gpu_reference(stream);
            const size_t rn1 = (size_t)stem.buf_height * stem.buf_width * PAD8(batch) * PAD128(ch);
            const std::vector<int> got_res = to_host(r1, rn1);
            const float* cursor3 = syn.values.data();
            tcbnn_host::ConfigSource cfg3(&cursor3, syn.values.data() + syn.values.size());
            InConv128LayerParam fresh2("Conv1", image, image, 3, 3, 3, ch, batch, 1, 1, true, 1, 1, true);
            fresh2.initialize(twice.data(), cfg3);
            fresh2.forward(stream);
            if (fresh2.residual_info.format != stem.residual_info.format) {
                fprintf(stderr, "Conv1: the doubled batch was meant to keep the residual format\n");
                return 1;
            }
            if (got_res != to_host(fresh2.get_output_residual_gpu_reference(stream), rn1)) {
                fprintf(stderr, "Conv1: set_input() of a larger batch and a fresh initialize() disagree\n");
                return 1;
            }
        }
        if (o.oversize_input) {
            std::vector<float> big(images);
            for (float& v : big) v *= 1000.0f;
            stem.set_input(big.data());  // must not return
            fprintf(stderr, "Conv1: set_input() accepted a batch beyond the residual bound\n");
            return 1;
        }
    }
    long long nz = 0;
    for (int v : resid[0]) nz += v != 0;
    printf("{\"check\": \"reference_fmt_interop\", \"batch\": %u, \"logits0\": [%.6g, %.6g, %.6g], "
           "\"c2_residual_nonzero\": %lld, \"ok\": true}\n",
           batch, logits[0][0], logits[0][1], logits[0][2], nz);
    if (!o.out.empty()) {
        FILE* f = fopen(o.out.c_str(), "wb");
        if (f == NULL || fwrite(logits[1].data(), sizeof(float), logits[1].size(), f) != logits[1].size()) return 1;
        fclose(f);
    }
    HIP_SAFE_CALL(hipStreamDestroy(stream));
    return 0;
}
