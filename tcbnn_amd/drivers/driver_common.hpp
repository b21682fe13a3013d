// Shared pieces of the network drivers: a small argv parser (the reference hard-codes batch,
// device and file paths in each main), seeded synthetic parameters / inputs (the reference's
// trained weight files are not distributed), hipEvent timing and result output.
#pragma once

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

#include "../host/tcbnn_data.hpp"
#include "../host/tcbnn_layers.hpp"

namespace driver {

struct Options {
    int batch = 0;          // 0 = the driver's default
    uint64_t seed = 0;
    int reps = 10;          // timed repetitions (the reference benches use TEST_TIMES 10)
    int warmup = 3;
    int image = 0;          // image side (0 = default)
    int classes = 0;        // output classes (0 = default)
    std::string weights;    // text weight file in the reference's format; empty = synthetic
    std::string input;      // raw float32 input file; empty = synthetic
    std::string out;        // raw float32 logits are written here if set
    std::string labels;     // raw uint32 labels (read_dataset writes them): scores the logits against them
    std::string variant;    // popc | mfma_i8 | mfma_f4
    bool oversize_input = false;  // reference_fmt_interop: end by giving the first layer a batch beyond its bound
    bool packed_input = false;    // the first convolution reads a packed copy of the input that the upload makes
};

inline Options parse(int argc, char** argv, const char* usage) {
    Options o;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        auto next = [&]() -> const char* {
            if (i + 1 >= argc) {
                fprintf(stderr, "missing value for %s\n%s\n", a.c_str(), usage);
                exit(1);
            }
            return argv[++i];
        };
        if (a == "--batch") o.batch = atoi(next());
        else if (a == "--seed") o.seed = strtoull(next(), NULL, 10);
        else if (a == "--reps") o.reps = atoi(next());
        else if (a == "--warmup") o.warmup = atoi(next());
        else if (a == "--image") o.image = atoi(next());
        else if (a == "--classes") o.classes = atoi(next());
        else if (a == "--weights") o.weights = next();
        else if (a == "--input") o.input = next();
        else if (a == "--out") o.out = next();
        else if (a == "--labels") o.labels = next();
        else if (a == "--variant") o.variant = next();
        else if (a == "--oversize-input") o.oversize_input = true;
        else if (a == "--packed-input") o.packed_input = true;
        else {
            fprintf(stderr, "unknown argument %s\n%s\n", a.c_str(), usage);
            exit(1);
        }
    }
    if (!o.variant.empty()) {
        int v = o.variant == "popc" ? TCBNN_VARIANT_POPC
                : o.variant == "mfma_i8" ? TCBNN_VARIANT_MFMA_I8
                : o.variant == "mfma_f4" ? TCBNN_VARIANT_MFMA_F4 : -1;
        TCBNN_SAFE_CALL(tcbnn_set_default_variant(v));
    }
    return o;
}

// splitmix64: one independent stream per tensor (seed xor tensor id)
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    double uniform() { return (next() >> 11) * (1.0 / 9007199254740992.0); }
    double normal() {
        double u1 = uniform(), u2 = uniform();
        if (u1 < 1e-300) u1 = 1e-300;
        return sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2);
    }
};

// Synthetic parameters in weight-file order.
struct Synthetic {
    std::vector<float> values;
    uint64_t seed;
    int tensor = 0;
    explicit Synthetic(uint64_t s) : seed(s) {}
    // +-1 weights [fan_in][nout] (fan_in slowest) and N(0, sqrt(fan_in)) thresholds, with a random
    // BN sign folded into the column and its threshold
    void binary_layer(size_t fan_in, size_t nout) {
        Rng r(seed ^ (0x1000ull + tensor++));
        const size_t base = values.size();
        values.resize(base + fan_in * nout + nout);
        float* w = &values[base];
        float* thr = w + fan_in * nout;
        for (size_t i = 0; i < fan_in * nout; ++i) w[i] = (r.next() >> 63) ? 1.0f : -1.0f;
        for (size_t j = 0; j < nout; ++j) thr[j] = (float)(r.normal() * sqrt((double)fan_in));
        for (size_t j = 0; j < nout; ++j)
            if (r.next() >> 63) {
                for (size_t k = 0; k < fan_in; ++k) w[k * nout + j] = -w[k * nout + j];
                thr[j] = -thr[j];
            }
    }
    // fp32 head: weights N(0, 1/sqrt(fan_in)) [fan_in][nout], bias N(0, 1)
    void fp32_layer(size_t fan_in, size_t nout) {
        Rng r(seed ^ (0x1000ull + tensor++));
        const size_t base = values.size();
        values.resize(base + fan_in * nout + nout);
        for (size_t i = 0; i < fan_in * nout; ++i) values[base + i] = (float)(r.normal() / sqrt((double)fan_in));
        for (size_t j = 0; j < nout; ++j) values[base + fan_in * nout + j] = (float)r.normal();
    }
    // output layer: +-1 weights, scale N(1, 0.1), bias N(0, 1)
    void output_layer(size_t fan_in, size_t nout) {
        Rng r(seed ^ (0x1000ull + tensor++));
        const size_t base = values.size();
        values.resize(base + fan_in * nout + 2 * nout);
        float* w = &values[base];
        for (size_t i = 0; i < fan_in * nout; ++i) w[i] = (r.next() >> 63) ? 1.0f : -1.0f;
        for (size_t j = 0; j < nout; ++j) w[fan_in * nout + j] = (float)(1.0 + 0.1 * r.normal());
        for (size_t j = 0; j < nout; ++j) w[fan_in * nout + nout + j] = (float)r.normal();
    }
};

inline std::vector<float> read_floats(const std::string& path, size_t n) {
    std::vector<float> v(n);
    FILE* f = fopen(path.c_str(), "rb");
    if (f == NULL || fread(v.data(), sizeof(float), n, f) != n) {
        fprintf(stderr, "cannot read %zu floats from %s\n", n, path.c_str());
        exit(1);
    }
    fclose(f);
    return v;
}

inline std::vector<float> synthetic_input(uint64_t seed, size_t n, bool centred_uniform) {
    std::vector<float> v(n);
    Rng r(seed ^ 0xabcdefull);
    for (size_t i = 0; i < n; ++i) v[i] = centred_uniform ? (float)(r.uniform() - 0.5) : (float)r.normal();
    return v;
}

// Times `reps` forward passes between two hipEvents on `stream` (START_TIMER / STOP_TIMER of the
// reference, utility.h:161-173 — which computes the time but never prints it).
template <class F>
double time_forward(F&& forward, hipStream_t stream, int warmup, int reps) {
    for (int i = 0; i < warmup; ++i) forward();
    hipEvent_t start, stop;
    HIP_SAFE_CALL(hipEventCreate(&start));
    HIP_SAFE_CALL(hipEventCreate(&stop));
    HIP_SAFE_CALL(hipEventRecord(start, stream));
    for (int i = 0; i < reps; ++i) forward();
    HIP_SAFE_CALL(hipEventRecord(stop, stream));
    HIP_SAFE_CALL(hipEventSynchronize(stop));
    float ms = 0;
    HIP_SAFE_CALL(hipEventElapsedTime(&ms, start, stop));
    HIP_SAFE_CALL(hipEventDestroy(start));
    HIP_SAFE_CALL(hipEventDestroy(stop));
    return ms / reps;
}

inline void report(const char* net, int batch, double ms, double binary_ops, const float* logits, int classes,
                   const Options& o) {
    printf("{\"net\": \"%s\", \"batch\": %d, \"ms_per_batch\": %.4f, \"images_per_s\": %.1f, "
           "\"binary_tops\": %.2f, \"logits0\": [%.6g, %.6g, %.6g]}\n",
           net, batch, ms, batch / (ms * 1e-3), binary_ops / (ms * 1e-3) / 1e12, logits[0],
           logits[classes > 1 ? 1 : 0], logits[classes > 2 ? 2 : 0]);
    if (!o.labels.empty()) {  // the call every reference main carries, commented out (e.g. mnist_mlp.cu:156)
        std::vector<unsigned> labels(batch);
        FILE* f = tcbnn_data::open_or_die(o.labels, "label");
        tcbnn_data::read_or_die(f, labels.data(), labels.size() * sizeof(unsigned), o.labels);
        fclose(f);
        validate_prediction(const_cast<float*>(logits), labels.data(), (unsigned)classes, (unsigned)batch);
    }
    if (!o.out.empty()) {
        FILE* f = fopen(o.out.c_str(), "wb");
        if (f == NULL || fwrite(logits, sizeof(float), (size_t)batch * classes, f) != (size_t)batch * classes) {
            fprintf(stderr, "cannot write %s\n", o.out.c_str());
            exit(1);
        }
        fclose(f);
    }
}

}  // namespace driver
