// C++ host mirror of the reference's layer objects (param.h:115-1065) over the C ABI of
// libtcbnn_hip.so.  Same class names, constructor signatures, public fields and method
// names, so a driver written against the reference's param.h keeps compiling:
//
//     Conv128LayerParam* c = new Conv128LayerParam("L1B1C2", h, w, 3, 3, 64, 64, batch,
//                                                  1, 1, true, 1, 1, false, true, true, 64);
//     c->initialize(config_file, prev->get_output_gpu(), stem->get_output_residual_gpu());
//
// What differs, by design:
//   * initialize() returns `this` (the reference returns the device shadow that its
//     cooperative network kernel dereferences); each layer is run with forward(stream),
//     one stream-ordered launch, in place of the call inside the network kernel
//     (imagenet_resnet.cu:34-125).  forward() is idempotent: outputs are plainly stored,
//     not OR-accumulated into a once-zeroed buffer (param.h:973-974).
//   * device buffers use the engine's batch-innermost layouts; download_output() converts
//     to the reference's tile-contiguous layout, so it returns what the reference returns.
//   * errors follow the reference convention: message on stderr and exit(-1)
//     (utility.h:57-92); the C ABI underneath returns codes instead.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <math.h>

#include <algorithm>
#include <map>
#include <vector>

#include "../../include/tcbnn_hip.h"

// ---- utility.h:25-52 ---------------------------------------------------------------
typedef unsigned char uin8;
typedef unsigned short uin16;
typedef unsigned int uin32;
typedef unsigned long long uin64;

#define STEP8(X) (((X) + 7) >> 3)
#define STEP32(X) (((X) + 31) >> 5)
#define STEP128(X) (((X) + 127) >> 7)
#define PAD8(X) (STEP8(X) << 3)
#define PAD32(X) (STEP32(X) << 5)
#define PAD128(X) (STEP128(X) << 7)

// ---- error convention, utility.h:57-92 ------------------------------------------------
#define HIP_SAFE_CALL(err) tcbnn_host::hip_safe_call((err), __FILE__, __LINE__)
#define TCBNN_SAFE_CALL(rc) tcbnn_host::tcbnn_safe_call((rc), __FILE__, __LINE__)
#define CHECK_NULL_POINTER(X) tcbnn_host::check_null((const void*)(X), __FILE__, __LINE__)
#define SAFE_ALOC_GPU(X, Y) HIP_SAFE_CALL(hipMalloc((void**)&(X), (Y) > 0 ? (size_t)(Y) : 4))
#define SAFE_ALOC_HOST(X, Y) HIP_SAFE_CALL(hipHostMalloc((void**)&(X), (Y) > 0 ? (size_t)(Y) : 4))
#define SAFE_FREE_GPU(X)               \
    if ((X) != NULL) {                 \
        HIP_SAFE_CALL(hipFree((X)));   \
        (X) = NULL;                    \
    }
#define SAFE_FREE_HOST(X)                \
    if ((X) != NULL) {                   \
        HIP_SAFE_CALL(hipHostFree((X))); \
        (X) = NULL;                      \
    }

namespace tcbnn_host {

inline void hip_safe_call(hipError_t err, const char* file, int line) {
    if (err != hipSuccess) {
        fprintf(stderr, "hipSafeCall() failed at %s:%i : %s\n", file, line, hipGetErrorString(err));
        exit(-1);
    }
}
inline void tcbnn_safe_call(int rc, const char* file, int line) {
    if (rc != TCBNN_OK) {
        fprintf(stderr, "tcbnn call failed at %s:%i : %s\n", file, line, tcbnn_last_error());
        exit(-1);
    }
}
inline void check_null(const void* p, const char* file, int line) {
    if (p == NULL) {
        fprintf(stderr, "Error: NULL pointer at %s:%i.\n", file, line);
        exit(-1);
    }
}

// load weights from file, utility.h:188-196
inline void launch_array(FILE* cf, float* array, unsigned array_size) {
    if (cf == NULL) {
        fprintf(stderr, "NULL pointer to the network configuration file.\n");
        exit(1);
    }
    for (unsigned i = 0; i < array_size; i++) {
        int c;
        while ((c = fgetc(cf)) == ',') {  // the reference's files are white-space separated; tolerate commas
        }
        if (c != EOF) ungetc(c, cf);
        if (fscanf(cf, "%f", &array[i]) != 1) {
            fprintf(stderr, "network configuration file ended after %u of %u values.\n", i, array_size);
            exit(1);
        }
    }
}

// Where a layer's parameters come from: the reference's text weight file, or an in-memory
// float array consumed in the same order.  Converts implicitly from FILE*, so
// initialize(config_file, ...) reads exactly like the reference.
class ConfigSource {
   public:
    ConfigSource(FILE* f) : file_(f), cursor_(NULL), end_(NULL) {}
    ConfigSource(const float** cursor, const float* end) : file_(NULL), cursor_(cursor), end_(end) {}
    void read(float* dst, unsigned n) {
        if (cursor_ != NULL) {
            if (*cursor_ + n > end_) {
                fprintf(stderr, "in-memory network configuration ended early.\n");
                exit(1);
            }
            memcpy(dst, *cursor_, (size_t)n * sizeof(float));
            *cursor_ += n;
        } else {
            launch_array(file_, dst, n);
        }
    }

   private:
    FILE* file_;
    const float** cursor_;
    const float* end_;
};

// What a consumer has to know about a saved residual, recorded by its producer and keyed by the
// device pointer that get_output_residual_gpu() hands out:
//   channels: the reference infers the channel stride of an injected residual from PAD128 of the
//             consumer's residual_channels (kernel.cuh:778-791); the engine stores the true count;
//   bound:    upper bound of |value| (first layer: from the actual input; each bit convolution
//             adds Cin*R*S), INT32_MAX when unknown;
//   format:   TCBNN_RES_I16 when the bound proves that 16 bits hold every value, else int32.
// The registry's copy also records who reads the tensor, which decides whether its producer may store only the
// maximum over 2x2 windows of pixels (a quarter of the bytes written and read; tcbnn_conv128_desc's
// output_residual_pool): how often get_output_residual_gpu() handed the pointer out, how many Conv128 consumers
// registered with residual_pool, how many other consumers of this library, whether the full tensor was ever asked
// for, and what the buffer holds since the producer's last forward().  The maximum alone is stored when every
// hand-out went to a pooling consumer (so that nobody else can be reading the tensor), nobody asked for the full
// tensor, and the producer's kernel can do it (will_pool).
// A reader whose own saved residual depends on the tensor's bound: that tensor's pointer variable (NULL while it
// saves nothing) and what the reader adds to the bound (Cin*R*S for a bit convolution, 0 for a pooling layer).
struct ResidualReader {
    const void* who;
    int* const* out_gpu;
    int add;
};
struct ResidualInfo {
    int channels, bound, format;
    int handed_out, pool_consumers, other_consumers;
    bool observed, pooled, written;
    bool (*will_pool)(void*);  // the producer's decision for its next forward(); NULL: never
    void* producer;
    std::vector<ResidualReader> readers;
};
inline std::map<const void*, ResidualInfo>& residual_registry() {
    static std::map<const void*, ResidualInfo> reg;
    return reg;
}
// (the narrowest format that is exact for the bound: 12 bits up to 2047 for even batches, 16 bits up to 32767)
inline ResidualInfo make_residual_info(int channels, int bound, int batch) {
    ResidualInfo info;
    info.channels = channels;
    info.bound = bound;
    info.format = tcbnn_residual_format_narrowest(bound, batch);
    info.handed_out = info.pool_consumers = info.other_consumers = 0;
    info.observed = info.pooled = info.written = false;
    info.will_pool = NULL;
    info.producer = NULL;
    return info;
}
inline ResidualInfo* find_residual(const void* gpu) {
    std::map<const void*, ResidualInfo>::iterator it = residual_registry().find(gpu);
    return it != residual_registry().end() ? &it->second : NULL;
}
// a layer of this library starts (sign = +1) or stops (-1) reading the saved residual at `gpu`
inline void register_residual_consumer(const void* gpu, bool pools, int sign, const void* who = NULL,
                                       int* const* out_gpu = NULL, int add = 0) {
    ResidualInfo* u = find_residual(gpu);
    if (u == NULL) return;
    (pools ? u->pool_consumers : u->other_consumers) += sign;
    if (who == NULL) return;
    if (sign > 0) {
        const ResidualReader r = {who, out_gpu, add};
        u->readers.push_back(r);
    } else {
        for (size_t i = 0; i < u->readers.size(); ++i)
            if (u->readers[i].who == who) {
                u->readers.erase(u->readers.begin() + i);
                break;
            }
    }
}
// The largest bound of |value| the saved residual at `gpu` can take with every tensor that depends on it staying in
// the format it was allocated in: its own format's range, and for every reader that saves a residual of its own,
// that tensor's limit less what the reader adds.
inline int residual_bound_limit(const void* gpu) {
    const ResidualInfo* u = find_residual(gpu);
    if (u == NULL) return INT32_MAX / 4;
    int lim = u->format == TCBNN_RES_I12 ? 2047 : (u->format == TCBNN_RES_I16 ? 32767 : INT32_MAX / 4);
    for (size_t i = 0; i < u->readers.size(); ++i) {
        const ResidualReader& r = u->readers[i];
        if (r.out_gpu != NULL && *r.out_gpu != NULL) lim = std::min(lim, residual_bound_limit(*r.out_gpu) - r.add);
    }
    return lim;
}
// records a larger bound (within residual_bound_limit) for the tensor and for everything that depends on it
inline void raise_residual_bound(const void* gpu, int bound) {
    ResidualInfo* u = find_residual(gpu);
    if (u == NULL || bound <= u->bound) return;
    u->bound = bound;
    for (size_t i = 0; i < u->readers.size(); ++i) {
        const ResidualReader& r = u->readers[i];
        if (r.out_gpu != NULL && *r.out_gpu != NULL) raise_residual_bound(*r.out_gpu, bound + r.add);
    }
}
inline int* hand_out_residual(int* gpu) {
    ResidualInfo* u = find_residual(gpu);
    if (u != NULL) u->handed_out += 1;
    return gpu;
}
// does the buffer hold (after its producer's forward) the maximum over 2x2 windows instead of the full tensor?
inline bool residual_holds_window_maximum(const void* gpu) {
    const ResidualInfo* u = find_residual(gpu);
    if (u == NULL) return false;
    return u->written ? u->pooled : (u->will_pool != NULL && u->will_pool(u->producer));
}

}  // namespace tcbnn_host

using tcbnn_host::launch_array;

// ======================================================================================
class In128LayerParam {  // param.h:115-222
   public:
    In128LayerParam(const char* _name, int _input_height, int _input_width)
        : input(NULL), input_gpu(NULL), output(NULL), output_gpu(NULL), input_width(_input_width),
          input_height(_input_height), output_width(_input_width), output_height(_input_height), gpu(this) {
        strncpy(name, _name, 8);
    }
    int input_size() { return input_height * input_width; }
    int input_bytes() { return input_size() * sizeof(float); }
    int output_size() { return output_height * output_width; }
    int output_bytes() { return output_size() * sizeof(float); }
    int output_bit_size() { return PAD8(output_height) * STEP128(output_width); }
    int output_bit_bytes() { return output_bit_size() * 16; }

    In128LayerParam* initialize(float* input) {
        CHECK_NULL_POINTER(input);
        this->input = input;
        SAFE_ALOC_GPU(input_gpu, input_bytes());
        HIP_SAFE_CALL(hipMemcpy(input_gpu, input, input_bytes(), hipMemcpyHostToDevice));
        SAFE_ALOC_GPU(output_gpu, 4 * tcbnn_fc_act_words(output_height, output_width));
        return this;
    }
    void set_output_gpu(uin32* _output_gpu) { this->output_gpu = _output_gpu; }
    uin32* get_output_gpu() { return this->output_gpu; }
    void forward(hipStream_t stream = 0) {
        tcbnn_in128_desc d = {input_gpu, output_gpu, input_height, input_width};
        TCBNN_SAFE_CALL(tcbnn_in128_forward(&d, stream));
    }
    uin32* download_output() {  // reference tile layout, PAD8(B)*STEP128(K) 128-bit units
        if (output == NULL) SAFE_ALOC_HOST(output, output_bit_bytes());
        uin32* tmp = NULL;
        SAFE_ALOC_GPU(tmp, output_bit_bytes());
        TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, tmp, output_height, output_width, 0));
        HIP_SAFE_CALL(hipMemcpy(output, tmp, output_bit_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(tmp);
        return this->output;
    }
    // The output in the reference's own tile layout ON THE DEVICE (what get_output_gpu() of the reference
    // holds, kernel.cuh:170): converted on `stream`, after forward(), into a buffer this layer owns.
    uin32* get_output_gpu_reference_fmt(hipStream_t stream = 0) {
        if (output_fmt_gpu == NULL) SAFE_ALOC_GPU(output_fmt_gpu, output_bit_bytes());
        TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, output_fmt_gpu, output_height, output_width, stream));
        return output_fmt_gpu;
    }
    float* download_full_output() {  // +-1.0f [B][K] (UnPackFcOutput128FMT, param.h:87-104)
        float* full_output = NULL;
        SAFE_ALOC_HOST(full_output, output_bytes());
        float* full_output_gpu = NULL;
        SAFE_ALOC_GPU(full_output_gpu, output_bytes());
        TCBNN_SAFE_CALL(tcbnn_unpack_fc_output(output_gpu, full_output_gpu, output_height, output_width, 0));
        HIP_SAFE_CALL(hipMemcpy(full_output, full_output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(full_output_gpu);
        return full_output;
    }
    void release() {
        SAFE_FREE_GPU(input_gpu);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(output_fmt_gpu);
        SAFE_FREE_HOST(output);
    }
    ~In128LayerParam() { release(); }

   public:
    float* input;
    float* input_gpu;
    uin32* output;
    uin32* output_gpu;
    int input_width;
    int input_height;
    int output_width;
    int output_height;
    In128LayerParam* gpu;
    char name[8];
    uin32* output_fmt_gpu = NULL;  // reference-layout copy of the output (no counterpart in the reference)
};

// ======================================================================================
class Fc128LayerParam {  // param.h:224-385
   public:
    Fc128LayerParam(const char* name, int _input_height, int _input_width, int _weight_width)
        : input(NULL), input_gpu(NULL), input_width(_input_width), input_height(_input_height), weight(NULL),
          weight_gpu(NULL), weight_width(_weight_width), weight_height(_input_width), output(NULL),
          output_gpu(NULL), output_width(_weight_width), output_height(_input_height), bn(NULL), bn_gpu(NULL),
          bn_width(_weight_width), gpu(this), variant(TCBNN_VARIANT_AUTO), workspace_gpu(NULL) {
        strncpy(this->name, name, 8);
    }
    int weight_size() { return weight_height * weight_width; }
    int weight_bytes() { return weight_size() * sizeof(float); }
    int output_size() { return output_height * output_width; }
    int output_bytes() { return output_size() * sizeof(float); }
    int output_bit_size() { return PAD8(output_height) * STEP128(output_width); }
    int output_bit_bytes() { return output_bit_size() * 16; }
    int bn_size() { return bn_width; }
    int bn_bytes() { return bn_size() * sizeof(float); }
    size_t workspace_words() { return (size_t)PAD32(weight_width) * input_height; }

    void set_input_gpu(uin32* _input_gpu) { this->input_gpu = _input_gpu; }
    Fc128LayerParam* initialize(tcbnn_host::ConfigSource config_file, uin32* prev_layer_gpu) {
        SAFE_ALOC_HOST(weight, weight_bytes());
        config_file.read(this->weight, weight_size());
        SAFE_ALOC_GPU(weight_gpu, 4 * tcbnn_fc_weight_words(weight_height, weight_width));
        float* weight_float = NULL;
        SAFE_ALOC_GPU(weight_float, weight_bytes());
        HIP_SAFE_CALL(hipMemcpy(weight_float, weight, weight_bytes(), hipMemcpyHostToDevice));
        TCBNN_SAFE_CALL(tcbnn_pack_fc_weight(weight_float, weight_gpu, weight_height, weight_width, 0));
        HIP_SAFE_CALL(hipDeviceSynchronize());
        SAFE_FREE_GPU(weight_float);
        SAFE_ALOC_HOST(bn, bn_bytes());
        config_file.read(this->bn, bn_size());
        SAFE_ALOC_GPU(bn_gpu, bn_bytes());
        HIP_SAFE_CALL(hipMemcpy(bn_gpu, bn, bn_bytes(), hipMemcpyHostToDevice));
        SAFE_ALOC_GPU(output_gpu, 4 * tcbnn_fc_act_words(output_height, output_width));
        SAFE_ALOC_GPU(workspace_gpu, 4 * workspace_words());
        set_input_gpu(prev_layer_gpu);
        CHECK_NULL_POINTER(input_gpu);
        return this;
    }
    uin32* get_output_gpu() { return this->output_gpu; }
    // Reference-layout neighbours (kernel.cuh:187-191 reads, :222-223 writes [B/8][K/128][8][4] tiles): the input
    // is converted on `stream` from a device buffer in that layout into a buffer this layer owns (a copy, so call
    // it again when the source changes), the output after forward() likewise into the reference layout.
    void set_input_gpu_reference_fmt(const uin32* fmt_gpu, hipStream_t stream = 0) {
        CHECK_NULL_POINTER(fmt_gpu);
        if (input_own_gpu == NULL) SAFE_ALOC_GPU(input_own_gpu, 4 * tcbnn_fc_act_words(input_height, input_width));
        TCBNN_SAFE_CALL(tcbnn_fc_from_reference_fmt(fmt_gpu, input_own_gpu, input_height, input_width, stream));
        input_gpu = input_own_gpu;
    }
    uin32* get_output_gpu_reference_fmt(hipStream_t stream = 0) {
        if (output_fmt_gpu == NULL) SAFE_ALOC_GPU(output_fmt_gpu, output_bit_bytes());
        TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, output_fmt_gpu, output_height, output_width, stream));
        return output_fmt_gpu;
    }
    void forward(hipStream_t stream = 0) {
        tcbnn_fc128_desc d = {input_gpu, weight_gpu, bn_gpu,  output_gpu,    input_height,
                              input_width, weight_width, variant, workspace_gpu, workspace_words()};
        TCBNN_SAFE_CALL(tcbnn_fc128_forward(&d, stream));
    }
    uin32* download_output() {
        if (output == NULL) SAFE_ALOC_HOST(output, output_bit_bytes());
        uin32* tmp = NULL;
        SAFE_ALOC_GPU(tmp, output_bit_bytes());
        TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, tmp, output_height, output_width, 0));
        HIP_SAFE_CALL(hipMemcpy(output, tmp, output_bit_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(tmp);
        return this->output;
    }
    float* download_full_output() {
        float* full_output = NULL;
        SAFE_ALOC_HOST(full_output, output_bytes());
        float* full_output_gpu = NULL;
        SAFE_ALOC_GPU(full_output_gpu, output_bytes());
        TCBNN_SAFE_CALL(tcbnn_unpack_fc_output(output_gpu, full_output_gpu, output_height, output_width, 0));
        HIP_SAFE_CALL(hipMemcpy(full_output, full_output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(full_output_gpu);
        return full_output;
    }
    void release() {
        SAFE_FREE_HOST(weight);
        SAFE_FREE_HOST(bn);
        SAFE_FREE_HOST(output);
        SAFE_FREE_GPU(weight_gpu);
        SAFE_FREE_GPU(bn_gpu);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(workspace_gpu);
        SAFE_FREE_GPU(input_own_gpu);
        SAFE_FREE_GPU(output_fmt_gpu);
    }
    ~Fc128LayerParam() { release(); }

   public:
    uin32* input;
    uin32* input_gpu;
    int input_width;
    int input_height;
    float* weight;
    uin32* weight_gpu;
    int weight_width;
    int weight_height;
    uin32* output;
    uin32* output_gpu;
    int output_width;
    int output_height;
    float* bn;
    float* bn_gpu;
    int bn_width;
    Fc128LayerParam* gpu;
    char name[8];
    int variant;             // TCBNN_VARIANT_* (no counterpart in the reference)
    int32_t* workspace_gpu;  // split-K scratch (no counterpart in the reference)
    uin32* input_own_gpu = NULL;   // engine-layout copy of a reference-layout input
    uin32* output_fmt_gpu = NULL;  // reference-layout copy of the output
};

// ======================================================================================
class Out128LayerParam {  // param.h:388-531
   public:
    Out128LayerParam(const char* name, int _input_height, int _input_width, int _weight_width)
        : input(NULL), input_gpu(NULL), input_width(_input_width), input_height(_input_height), weight(NULL),
          weight_gpu(NULL), weight_width(_weight_width), weight_height(_input_width), output(NULL),
          output_gpu(NULL), output_height(_input_height), output_width(_weight_width), has_bn(true),
          bn_scale(NULL), bn_scale_gpu(NULL), bn_bias(NULL), bn_bias_gpu(NULL), gpu(this),
          variant(TCBNN_VARIANT_AUTO) {
        strncpy(this->name, name, 8);
    }
    int weight_size() { return weight_height * weight_width; }
    int weight_bytes() { return weight_size() * sizeof(float); }
    int output_size() { return output_height * output_width; }
    int output_bytes() { return output_size() * sizeof(float); }
    int bn_size() { return output_width; }
    int bn_bytes() { return output_width * sizeof(float); }

    void set_input_gpu(uin32* input_gpu) { this->input_gpu = input_gpu; }
    float* get_output_gpu() { return this->output_gpu; }
    Out128LayerParam* initialize(tcbnn_host::ConfigSource config_file, uin32* prev_layer_gpu) {
        SAFE_ALOC_HOST(weight, weight_bytes());
        config_file.read(this->weight, weight_size());
        SAFE_ALOC_GPU(weight_gpu, 4 * tcbnn_fc_weight_words(weight_height, weight_width));
        float* weight_float = NULL;
        SAFE_ALOC_GPU(weight_float, weight_bytes());
        HIP_SAFE_CALL(hipMemcpy(weight_float, weight, weight_bytes(), hipMemcpyHostToDevice));
        TCBNN_SAFE_CALL(tcbnn_pack_fc_weight(weight_float, weight_gpu, weight_height, weight_width, 0));
        HIP_SAFE_CALL(hipDeviceSynchronize());
        SAFE_FREE_GPU(weight_float);
        SAFE_ALOC_HOST(bn_scale, bn_bytes());
        config_file.read(this->bn_scale, bn_size());
        SAFE_ALOC_GPU(bn_scale_gpu, bn_bytes());
        HIP_SAFE_CALL(hipMemcpy(bn_scale_gpu, bn_scale, bn_bytes(), hipMemcpyHostToDevice));
        SAFE_ALOC_HOST(bn_bias, bn_bytes());
        config_file.read(this->bn_bias, bn_size());
        SAFE_ALOC_GPU(bn_bias_gpu, bn_bytes());
        HIP_SAFE_CALL(hipMemcpy(bn_bias_gpu, bn_bias, bn_bytes(), hipMemcpyHostToDevice));
        SAFE_ALOC_GPU(output_gpu, output_bytes());
        HIP_SAFE_CALL(hipMemset(this->output_gpu, 0, output_bytes()));
        set_input_gpu(prev_layer_gpu);
        CHECK_NULL_POINTER(input_gpu);
        return this;
    }
    // input from a device buffer in the reference's tile layout (kernel.cuh:243-247): see Fc128LayerParam
    void set_input_gpu_reference_fmt(const uin32* fmt_gpu, hipStream_t stream = 0) {
        CHECK_NULL_POINTER(fmt_gpu);
        if (input_own_gpu == NULL) SAFE_ALOC_GPU(input_own_gpu, 4 * tcbnn_fc_act_words(input_height, input_width));
        TCBNN_SAFE_CALL(tcbnn_fc_from_reference_fmt(fmt_gpu, input_own_gpu, input_height, input_width, stream));
        input_gpu = input_own_gpu;
    }
    void forward(hipStream_t stream = 0) {
        tcbnn_out128_desc d = {input_gpu,    weight_gpu,  bn_scale_gpu, bn_bias_gpu, output_gpu,
                               input_height, input_width, weight_width, variant};
        TCBNN_SAFE_CALL(tcbnn_out128_forward(&d, stream));
    }
    float* download_output() {
        if (output == NULL) SAFE_ALOC_HOST(output, output_bytes());
        HIP_SAFE_CALL(hipMemcpy(output, output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        return this->output;
    }
    void release() {
        SAFE_FREE_HOST(weight);
        SAFE_FREE_HOST(output);
        SAFE_FREE_HOST(bn_scale);
        SAFE_FREE_HOST(bn_bias);
        SAFE_FREE_GPU(weight_gpu);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(bn_scale_gpu);
        SAFE_FREE_GPU(bn_bias_gpu);
        SAFE_FREE_GPU(input_own_gpu);
    }
    ~Out128LayerParam() { release(); }

   public:
    uin32* input;
    uin32* input_gpu;
    int input_width;
    int input_height;
    float* weight;
    uin32* weight_gpu;
    int weight_width;
    int weight_height;
    float* output;
    float* output_gpu;
    int output_height;
    int output_width;
    bool has_bn;
    float* bn_scale;
    float* bn_scale_gpu;
    float* bn_bias;
    float* bn_bias_gpu;
    Out128LayerParam* gpu;
    char name[8];
    int variant;
    uin32* input_own_gpu = NULL;  // engine-layout copy of a reference-layout input
};

// ======================================================================================
// Geometry shared by both conv constructors (param.h:719-728, 897-906).
#define TCBNN_CONV_GEOMETRY()                                                                          \
    this->pad_h = tcbnn_conv_pad(input_height, filter_height, stride_height, padding);                 \
    this->pad_w = tcbnn_conv_pad(input_width, filter_width, stride_width, padding);                    \
    buf_height = tcbnn_conv_out(input_height, filter_height, stride_height, padding, 1);               \
    buf_width = tcbnn_conv_out(input_width, filter_width, stride_width, padding, 1);                   \
    output_height = tcbnn_conv_out(input_height, filter_height, stride_height, padding, pool_height);  \
    output_width = tcbnn_conv_out(input_width, filter_width, stride_width, padding, pool_width);

class InConv128LayerParam {  // param.h:701-870
   public:
    InConv128LayerParam(const char* name, int _input_height, int _input_width, int _filter_height,
                        int _filter_width, int _input_channels, int _output_channels, int _batch,
                        int _stride_height = 1, int _stride_width = 1, bool _padding = true,
                        int _pool_height = 1, int _pool_width = 1, bool _save_residual = false)
        : input(NULL), input_gpu(NULL), input_width(_input_width), input_height(_input_height),
          input_channels(_input_channels), filter(NULL), filter_gpu(NULL), filter_width(_filter_width),
          filter_height(_filter_height), output(NULL), output_gpu(NULL), output_channels(_output_channels),
          padding(_padding), bn(NULL), bn_gpu(NULL), batch(_batch), stride_height(_stride_height),
          stride_width(_stride_width), pool_width(_pool_width), pool_height(_pool_height),
          save_residual(_save_residual), output_residual_gpu(NULL), gpu(this) {
        residual_info = tcbnn_host::make_residual_info(_output_channels, INT32_MAX, _batch);
        strncpy(this->name, name, 8);
        TCBNN_CONV_GEOMETRY();
    }
    // upper bound of |first-layer sum| for a batch: the largest sum of |x| under any filter window
    int residual_bound_of(const float* batch_input) {
        return tcbnn_inconv_residual_bound_of_input(batch_input, batch, input_height, input_width, filter_height,
                                                    filter_width, stride_height, stride_width, padding ? 1 : 0);
    }
    int input_size() { return input_channels * input_height * input_width * batch; }
    int input_bytes() { return input_size() * sizeof(float); }
    // On request (before initialize), the un-pooled first layer reads a zero-padded, batch-innermost copy of the
    // input (tcbnn_inconv_pack_input) with a kernel that needs no staging; initialize / set_input then make that
    // copy after the upload: one more pass over the input there, a shorter forward pass.  Without the request,
    // and for pooled layers, the layer reads input_gpu ([batch][3][H][W], kernel.cuh:620-625) itself.
    InConv128LayerParam* use_packed_input(bool on = true) {
        packed_input = on;
        return this;
    }
    size_t input_packed_bytes() {
        if (!packed_input || pool_height != 1 || pool_width != 1) return 0;
        const size_t n = tcbnn_inconv_packed_input_floats(batch, input_height, input_width, filter_height,
                                                          filter_width, stride_height, stride_width, padding ? 1 : 0);
        return n > 0 && n * sizeof(float) < ((size_t)1 << 31) ? n * sizeof(float) : 0;
    }
    void pack_input() {  // input_gpu -> input_packed_gpu
        if (input_packed_gpu == NULL) return;
        TCBNN_SAFE_CALL(tcbnn_inconv_pack_input(input_gpu, input_packed_gpu, batch, input_height, input_width,
                                                filter_height, filter_width, stride_height, stride_width,
                                                padding ? 1 : 0, 0));
        HIP_SAFE_CALL(hipDeviceSynchronize());
    }
    int filter_size() { return output_channels * input_channels * filter_height * filter_width; }
    int filter_bytes() { return filter_size() * sizeof(float); }
    int output_size() { return output_channels * output_height * output_width * batch; }
    int output_bytes() { return output_size() * sizeof(uin32); }
    int output_bit_size() { return STEP128(output_channels) * output_height * output_width * PAD8(batch); }
    int output_bit_bytes() { return output_bit_size() * 16; }
    int bn_size() { return output_channels; }
    int bn_bytes() { return bn_size() * sizeof(float); }
    // engine residual: true sizes (the reference pads to 8 x 128, param.h:756-758), 16 or 32 bits
    size_t residual_size() { return (size_t)output_channels * batch * buf_height * buf_width; }
    size_t residual_bytes() {
        return tcbnn_residual_bytes(buf_height, buf_width, output_channels, batch, residual_info.format);
    }

    InConv128LayerParam* initialize(float* input, tcbnn_host::ConfigSource config_file) {
        CHECK_NULL_POINTER(input);
        this->input = input;
        // |first-layer sum| <= the window's sum of |x|: decides whether the saved residual fits 12 or 16 bits
        residual_info = tcbnn_host::make_residual_info(output_channels, residual_bound_of(input), batch);
        SAFE_ALOC_GPU(input_gpu, input_bytes());
        HIP_SAFE_CALL(hipMemcpy(input_gpu, input, input_bytes(), hipMemcpyHostToDevice));
        if (input_packed_bytes() > 0) {
            SAFE_ALOC_GPU(input_packed_gpu, input_packed_bytes());
            pack_input();
        }
        SAFE_ALOC_HOST(filter, filter_bytes());
        config_file.read(this->filter, filter_size());
        SAFE_ALOC_GPU(filter_gpu,
                      4 * tcbnn_inconv_filter_words(filter_height, filter_width, input_channels, output_channels));
        float* filter_float = NULL;
        SAFE_ALOC_GPU(filter_float, filter_bytes());
        HIP_SAFE_CALL(hipMemcpy(filter_float, filter, filter_bytes(), hipMemcpyHostToDevice));
        TCBNN_SAFE_CALL(tcbnn_pack_inconv_filter(filter_float, filter_gpu, filter_height, filter_width,
                                                 input_channels, output_channels, 0));
        HIP_SAFE_CALL(hipDeviceSynchronize());
        SAFE_FREE_GPU(filter_float);
        SAFE_ALOC_HOST(bn, bn_bytes());
        config_file.read(bn, bn_size());
        SAFE_ALOC_GPU(bn_gpu, bn_bytes());
        HIP_SAFE_CALL(hipMemcpy(this->bn_gpu, this->bn, bn_bytes(), hipMemcpyHostToDevice));
        SAFE_ALOC_GPU(output_gpu, 4 * tcbnn_conv_act_words(output_height, output_width, batch, output_channels));
        if (save_residual) {
            SAFE_ALOC_GPU(output_residual_gpu, residual_bytes());
            tcbnn_host::residual_registry()[output_residual_gpu] = residual_info;
        }
        return this;
    }
    // A new batch for the same layer objects (the reference's objects are single-shot, this engine's are not):
    // uploads `input` into input_gpu.  The format of the saved residual, and of every residual downstream of it,
    // was chosen at initialize() from the first batch's bound.  A batch whose sums can be larger is accepted as long
    // as every one of those tensors still holds its values (the recorded bounds are raised); it is refused (print +
    // exit, like every error here) only when a format would have to change: its values would wrap in 12 or 16
    // bits.  The window scan of the batch is skipped when R*S*3*max|x| already fits.
    void set_input(float* input) {
        CHECK_NULL_POINTER(input);
        CHECK_NULL_POINTER(input_gpu);
        if (save_residual) {
            const tcbnn_host::ResidualInfo* u = tcbnn_host::find_residual(output_residual_gpu);
            const int recorded = u != NULL ? u->bound : residual_info.bound;
            const int coarse = tcbnn_inconv_residual_bound(filter_height, filter_width,
                                                           tcbnn_host_abs_max(input, (size_t)input_size()));
            if (coarse > recorded) {
                const int limit = tcbnn_host::residual_bound_limit(output_residual_gpu);
                const int bound = coarse <= limit ? coarse : residual_bound_of(input);
                if (bound > limit) {
                    fprintf(stderr, "Error: set_input: window sums of |input| up to %d exceed what the residual formats "
                                    "chosen at initialize() hold (up to %d): initialize the layers with the batch of "
                                    "largest magnitude.\n", bound, limit);
                    exit(-1);
                }
                tcbnn_host::raise_residual_bound(output_residual_gpu, bound);
            }
        }
        this->input = input;
        HIP_SAFE_CALL(hipMemcpy(input_gpu, input, input_bytes(), hipMemcpyHostToDevice));
        pack_input();
    }
    uin32* get_output_gpu() { return this->output_gpu; }
    int* get_output_residual_gpu() { return this->output_residual_gpu; }
    void forward(hipStream_t stream = 0) {
        const bool packed = input_packed_gpu != NULL;
        tcbnn_inconv128_desc d = {packed ? input_packed_gpu : input_gpu, filter_gpu, bn_gpu, output_gpu,
                                  output_residual_gpu,
                                  input_height,   input_width,    input_channels, filter_height, filter_width,
                                  output_channels, batch,         stride_height, stride_width, padding ? 1 : 0,
                                  pool_height,    pool_width,     save_residual ? 1 : 0, residual_info.format,
                                  packed ? TCBNN_INCONV_INPUT_PACKED : TCBNN_INCONV_INPUT_NCHW};
        TCBNN_SAFE_CALL(tcbnn_inconv128_forward(&d, stream));
    }
    // Output and saved residual in the reference's own device layouts (kernel.cuh:650-668), converted on `stream`
    // after forward() into buffers this layer owns: [OH][OW][PAD8(B)/8][STEP128(O)][8][4] words, and int32
    // [P][Q][PAD8(B)][PAD128(O)].
    uin32* get_output_gpu_reference_fmt(hipStream_t stream = 0) {
        if (output_fmt_gpu == NULL) SAFE_ALOC_GPU(output_fmt_gpu, output_bit_bytes());
        TCBNN_SAFE_CALL(tcbnn_conv_to_reference_fmt(output_gpu, output_fmt_gpu, output_height, output_width, batch,
                                                    output_channels, stream));
        return output_fmt_gpu;
    }
    int* get_output_residual_gpu_reference(hipStream_t stream = 0) {
        CHECK_NULL_POINTER(output_residual_gpu);
        if (output_residual_ref_gpu == NULL)
            SAFE_ALOC_GPU(output_residual_ref_gpu,
                          (size_t)buf_height * buf_width * PAD8(batch) * PAD128(output_channels) * sizeof(int));
        TCBNN_SAFE_CALL(tcbnn_residual_to_reference(output_residual_gpu, output_residual_ref_gpu, buf_height,
                                                    buf_width, batch, output_channels, residual_info.format, stream));
        return output_residual_ref_gpu;
    }
    unsigned* download_output() {
        if (output == NULL) SAFE_ALOC_HOST(output, output_bit_bytes());
        uin32* tmp = NULL;
        SAFE_ALOC_GPU(tmp, output_bit_bytes());
        TCBNN_SAFE_CALL(
            tcbnn_conv_to_reference_fmt(output_gpu, tmp, output_height, output_width, batch, output_channels, 0));
        HIP_SAFE_CALL(hipMemcpy(output, tmp, output_bit_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(tmp);
        return this->output;
    }
    float* download_full_output() {  // +-1.0f NHWC (UnpackConvOutput32FMT, param.h:661-688)
        float* full_output = NULL;
        SAFE_ALOC_HOST(full_output, output_bytes());
        float* full_output_gpu = NULL;
        SAFE_ALOC_GPU(full_output_gpu, output_bytes());
        TCBNN_SAFE_CALL(tcbnn_unpack_conv_output(output_gpu, full_output_gpu, output_height, output_width,
                                                 output_channels, batch, 0));
        HIP_SAFE_CALL(hipMemcpy(full_output, full_output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(full_output_gpu);
        return full_output;
    }
    void release() {
        SAFE_FREE_HOST(filter);
        SAFE_FREE_HOST(bn);
        SAFE_FREE_HOST(output);
        SAFE_FREE_GPU(input_gpu);
        SAFE_FREE_GPU(input_packed_gpu);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(filter_gpu);
        SAFE_FREE_GPU(bn_gpu);
        if (output_residual_gpu != NULL) tcbnn_host::residual_registry().erase(output_residual_gpu);
        SAFE_FREE_GPU(output_residual_gpu);
        SAFE_FREE_GPU(output_fmt_gpu);
        SAFE_FREE_GPU(output_residual_ref_gpu);
    }
    ~InConv128LayerParam() { release(); }

   public:
    float* input;
    float* input_gpu;
    int input_width;
    int input_height;
    int input_channels;
    float* filter;
    uin32* filter_gpu;
    int filter_width;
    int filter_height;
    uin32* output;
    uin32* output_gpu;
    int output_width;
    int output_height;
    int output_channels;
    bool padding;
    float* bn;
    float* bn_gpu;
    int batch;
    int stride_height;
    int stride_width;
    int pad_h;
    int pad_w;
    int pool_width;
    int pool_height;
    bool save_residual;
    int* output_residual_gpu;
    tcbnn_host::ResidualInfo residual_info;  // channels / bound / format of output_residual_gpu
    InConv128LayerParam* gpu;
    char name[8];
    int buf_height, buf_width;  // conv output size before pooling
    uin32* output_fmt_gpu = NULL;        // reference-layout copies of the output and the saved residual
    int* output_residual_ref_gpu = NULL;
    bool packed_input = false;           // use_packed_input()
    float* input_packed_gpu = NULL;      // [Hp][Wp][batch][3] copy of input_gpu (un-pooled layers, on request)
};

// ======================================================================================
class Conv128LayerParam {  // param.h:872-1065
   public:
    Conv128LayerParam(const char* name, int _input_height, int _input_width, int _filter_height,
                      int _filter_width, int _input_channels, int _output_channels, int _batch,
                      int _stride_height = 1, int _stride_width = 1, bool _padding = true, int _pool_height = 1,
                      int _pool_width = 1, bool _ahead_fc = false, bool _save_residual = false,
                      bool _inject_residual = false, int _residual_channels = 0, bool _residual_pool = false)
        : input(NULL), input_gpu(NULL), input_width(_input_width), input_height(_input_height),
          input_channels(_input_channels), filter(NULL), filter_gpu(NULL), filter_width(_filter_width),
          filter_height(_filter_height), output(NULL), output_gpu(NULL), output_channels(_output_channels),
          bn(NULL), bn_gpu(NULL), batch(_batch), stride_height(_stride_height), stride_width(_stride_width),
          padding(_padding), pool_width(_pool_width), pool_height(_pool_height), ahead_fc(_ahead_fc),
          save_residual(_save_residual), output_residual_gpu(NULL), inject_residual(_inject_residual),
          input_residual_gpu(NULL), residual_channels(_residual_channels), residual_pool(_residual_pool),
          gpu(this), variant(TCBNN_VARIANT_AUTO), input_residual_channels(0) {
        residual_info = input_residual_info = tcbnn_host::make_residual_info(_output_channels, INT32_MAX, _batch);
        strncpy(this->name, name, 8);
        TCBNN_CONV_GEOMETRY();
    }
    int filter_size() { return output_channels * input_channels * filter_height * filter_width; }
    int filter_bytes() { return filter_size() * sizeof(float); }
    int output_size() { return output_channels * output_height * output_width * batch; }
    int output_bytes() { return output_size() * sizeof(uin32); }
    int output_bit_size() { return STEP128(output_channels) * output_height * output_width * PAD8(batch); }
    int output_bit_bytes() { return output_bit_size() * 16; }
    int bn_size() { return output_channels; }
    int bn_bytes() { return bn_size() * sizeof(float); }
    size_t residual_size() { return (size_t)output_channels * batch * buf_height * buf_width; }
    size_t residual_bytes() {
        return tcbnn_residual_bytes(buf_height, buf_width, output_channels, batch, residual_info.format);
    }

    void set_input_gpu(uin32* input_gpu) { this->input_gpu = input_gpu; }
    void set_input_residual_gpu(int* input_residual_gpu) {
        if (inject_residual) {
            tcbnn_host::register_residual_consumer(this->input_residual_gpu, residual_pool, -1, this);
            tcbnn_host::register_residual_consumer(input_residual_gpu, residual_pool, +1, this, &output_residual_gpu,
                                                   input_channels * filter_height * filter_width);
        }
        this->input_residual_gpu = input_residual_gpu;
        std::map<const void*, tcbnn_host::ResidualInfo>& reg = tcbnn_host::residual_registry();
        std::map<const void*, tcbnn_host::ResidualInfo>::iterator it = reg.find(input_residual_gpu);
        // a residual that no layer of this library produced: int32 with the consumer's channel
        // limit and no known bound
        tcbnn_host::ResidualInfo foreign = tcbnn_host::make_residual_info(residual_channels, INT32_MAX, batch);
        foreign.format = TCBNN_RES_I32;
        input_residual_info = it != reg.end() ? it->second : foreign;
        input_residual_channels = input_residual_info.channels;
        const tcbnn_host::ResidualInfo* own = tcbnn_host::find_residual(output_residual_gpu);
        if (output_residual_gpu != NULL &&
            tcbnn_conv_residual_bound(input_channels, filter_height, filter_width,
                                      input_residual_info.bound < INT32_MAX / 4 ? input_residual_info.bound
                                                                                : INT32_MAX / 4) >
                (own != NULL ? own->bound : residual_info.bound)) {
            fprintf(stderr, "Error: the injected residual exceeds the bound the saved residual was sized for.\n");
            exit(-1);
        }
    }
    Conv128LayerParam* initialize(tcbnn_host::ConfigSource config_file, uin32* prev_layer_gpu,
                                  int* input_residual_gpu = NULL) {
        SAFE_ALOC_HOST(filter, filter_bytes());
        config_file.read(filter, filter_size());
        SAFE_ALOC_GPU(filter_gpu,
                      4 * tcbnn_conv_filter_words(filter_height, filter_width, input_channels, output_channels));
        float* filter_float = NULL;
        SAFE_ALOC_GPU(filter_float, filter_bytes());
        HIP_SAFE_CALL(hipMemcpy(filter_float, filter, filter_bytes(), hipMemcpyHostToDevice));
        TCBNN_SAFE_CALL(tcbnn_pack_conv_filter(filter_float, filter_gpu, filter_height, filter_width, input_channels,
                                               output_channels, 0));
        HIP_SAFE_CALL(hipDeviceSynchronize());
        SAFE_FREE_GPU(filter_float);
        SAFE_ALOC_HOST(bn, bn_bytes());
        config_file.read(bn, bn_size());
        SAFE_ALOC_GPU(bn_gpu, bn_bytes());
        HIP_SAFE_CALL(hipMemcpy(bn_gpu, bn, bn_bytes(), hipMemcpyHostToDevice));
        const size_t words =
            ahead_fc ? tcbnn_fc_act_words(batch, output_height * output_width * PAD128(output_channels))
                     : tcbnn_conv_act_words(output_height, output_width, batch, output_channels);
        SAFE_ALOC_GPU(output_gpu, 4 * words);
        set_input_gpu(prev_layer_gpu);
        if (inject_residual) {
            set_input_residual_gpu(input_residual_gpu);
            CHECK_NULL_POINTER(this->input_residual_gpu);
        }
        if (save_residual) {
            const int injected = inject_residual ? input_residual_info.bound : 0;
            residual_info = tcbnn_host::make_residual_info(
                output_channels, injected < INT32_MAX / 4 ? tcbnn_conv_residual_bound(input_channels, filter_height,
                                                                                      filter_width, injected)
                                                          : INT32_MAX, batch);
            SAFE_ALOC_GPU(output_residual_gpu, residual_bytes());
            residual_info.will_pool = &Conv128LayerParam::will_pool_thunk;
            residual_info.producer = this;
            tcbnn_host::residual_registry()[output_residual_gpu] = residual_info;
        }
        CHECK_NULL_POINTER(input_gpu);
        return this;
    }
    uin32* get_output_gpu() { return this->output_gpu; }
    // (every hand-out is counted: see ResidualInfo)
    int* get_output_residual_gpu() { return tcbnn_host::hand_out_residual(this->output_residual_gpu); }
    // Store only the 2x2 maximum of the saved residual in the next forward()?  (see ResidualInfo)
    bool pooled_save_now() {
        const tcbnn_host::ResidualInfo* u = tcbnn_host::find_residual(output_residual_gpu);
        if (u == NULL || u->observed || u->other_consumers != 0 || u->pool_consumers == 0 ||
            u->handed_out != u->pool_consumers)
            return false;
        const tcbnn_conv128_desc d = describe(false);
        return tcbnn_conv128_pooled_save_supported(&d) == 1;
    }
    static bool will_pool_thunk(void* self) { return static_cast<Conv128LayerParam*>(self)->pooled_save_now(); }
    void forward(hipStream_t stream = 0) {
        const tcbnn_conv128_desc d = describe(true);
        TCBNN_SAFE_CALL(tcbnn_conv128_forward(&d, stream));
        tcbnn_host::ResidualInfo* u = tcbnn_host::find_residual(output_residual_gpu);
        if (u != NULL) {
            u->pooled = d.output_residual_pool == 2;
            u->written = true;
        }
    }
    tcbnn_conv128_desc describe(bool decide_pool) {
        tcbnn_conv128_desc d;
        memset(&d, 0, sizeof(d));
        d.input = input_gpu;
        d.filter = filter_gpu;
        d.bn = bn_gpu;
        d.output = output_gpu;
        d.input_residual = inject_residual ? input_residual_gpu : NULL;
        d.output_residual = output_residual_gpu;
        d.input_height = input_height;
        d.input_width = input_width;
        d.input_channels = input_channels;
        d.filter_height = filter_height;
        d.filter_width = filter_width;
        d.output_channels = output_channels;
        d.batch = batch;
        d.stride_height = stride_height;
        d.stride_width = stride_width;
        d.padding = padding ? 1 : 0;
        d.pool_height = pool_height;
        d.pool_width = pool_width;
        d.ahead_fc = ahead_fc ? 1 : 0;
        d.save_residual = save_residual ? 1 : 0;
        d.inject_residual = inject_residual ? 1 : 0;
        d.residual_channels = residual_channels;
        // (a source that already holds the 2x2 maximum is injected as it is)
        d.residual_pool = residual_pool && !(inject_residual && tcbnn_host::residual_holds_window_maximum(input_residual_gpu)) ? 1 : 0;
        d.input_residual_channels = input_residual_channels;
        d.variant = variant;
        d.input_residual_format = input_residual_info.format;
        d.output_residual_format = residual_info.format;
        d.output_residual_pool = decide_pool && pooled_save_now() ? 2 : 0;
        return d;
    }
    // Reference-layout neighbours.  Input bits [H][W][PAD8(B)/8][STEP128(C)][8][4] (read at kernel.cuh:741-749) and
    // an injected residual int32 [Hr][Wr][PAD8(B)][PAD128(residual_channels)] (kernel.cuh:770-791; Hr x Wr is the
    // convolution's output size, twice that with residual_pool) are converted on `stream` from device buffers in
    // those layouts into buffers this layer owns: copies, so call again when the source changes.  Nothing is
    // known about a foreign residual's values: it is kept as int32 with an unknown bound, and a layer that also
    // saves a residual must have been initialized with it, so that its own residual is sized for that.
    void set_input_gpu_reference_fmt(const uin32* fmt_gpu, hipStream_t stream = 0) {
        CHECK_NULL_POINTER(fmt_gpu);
        if (input_own_gpu == NULL)
            SAFE_ALOC_GPU(input_own_gpu, 4 * tcbnn_conv_act_words(input_height, input_width, batch, input_channels));
        TCBNN_SAFE_CALL(tcbnn_conv_from_reference_fmt(fmt_gpu, input_own_gpu, input_height, input_width, batch,
                                                      input_channels, stream));
        input_gpu = input_own_gpu;
    }
    void set_input_residual_gpu_reference(const int* ref_gpu, hipStream_t stream = 0) {
        CHECK_NULL_POINTER(ref_gpu);
        const int scale = residual_pool ? 2 : 1;
        const int rh = buf_height * scale, rw = buf_width * scale;
        if (input_residual_own_gpu == NULL)
            SAFE_ALOC_GPU(input_residual_own_gpu, tcbnn_residual_bytes(rh, rw, residual_channels, batch, TCBNN_RES_I32));
        TCBNN_SAFE_CALL(tcbnn_residual_from_reference(ref_gpu, input_residual_own_gpu, rh, rw, batch,
                                                      residual_channels, TCBNN_RES_I32, stream));
        set_input_residual_gpu(input_residual_own_gpu);  // not in the registry: int32, unknown bound
    }
    // Output (conv tiles, or FC tiles for an FC-ready layer: kernel.cuh:798-815) and saved residual
    // (kernel.cuh:818-824) in the reference's device layouts, converted on `stream` after forward().
    uin32* get_output_gpu_reference_fmt(hipStream_t stream = 0) {
        if (output_fmt_gpu == NULL) SAFE_ALOC_GPU(output_fmt_gpu, output_bit_bytes());
        if (ahead_fc)
            TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, output_fmt_gpu, batch,
                                                      output_height * output_width * PAD128(output_channels), stream));
        else
            TCBNN_SAFE_CALL(tcbnn_conv_to_reference_fmt(output_gpu, output_fmt_gpu, output_height, output_width,
                                                        batch, output_channels, stream));
        return output_fmt_gpu;
    }
    // (The full tensor is asked for: from now on it is what forward() saves, and if the buffer holds the 2x2
    // maximum from the last forward(), the layer is run again first; its inputs are still in place.)
    int* get_output_residual_gpu_reference(hipStream_t stream = 0) {
        CHECK_NULL_POINTER(output_residual_gpu);
        tcbnn_host::ResidualInfo* u = tcbnn_host::find_residual(output_residual_gpu);
        if (u != NULL) {
            u->observed = true;
            if (u->pooled) forward(stream);
        }
        if (output_residual_ref_gpu == NULL)
            SAFE_ALOC_GPU(output_residual_ref_gpu,
                          (size_t)buf_height * buf_width * PAD8(batch) * PAD128(output_channels) * sizeof(int));
        TCBNN_SAFE_CALL(tcbnn_residual_to_reference(output_residual_gpu, output_residual_ref_gpu, buf_height,
                                                    buf_width, batch, output_channels, residual_info.format, stream));
        return output_residual_ref_gpu;
    }
    unsigned* download_output() {
        if (output == NULL) SAFE_ALOC_HOST(output, output_bit_bytes());
        uin32* tmp = NULL;
        SAFE_ALOC_GPU(tmp, output_bit_bytes());
        if (ahead_fc)  // FC-ready: an FC activation of OH*OW*PAD128(O) features (kernel.cuh:798-808)
            TCBNN_SAFE_CALL(tcbnn_fc_to_reference_fmt(output_gpu, tmp, batch,
                                                      output_height * output_width * PAD128(output_channels), 0));
        else
            TCBNN_SAFE_CALL(tcbnn_conv_to_reference_fmt(output_gpu, tmp, output_height, output_width, batch,
                                                        output_channels, 0));
        HIP_SAFE_CALL(hipMemcpy(output, tmp, output_bit_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(tmp);
        return this->output;
    }
    float* download_full_output() {
        float* full_output = NULL;
        SAFE_ALOC_HOST(full_output, output_bytes());
        float* full_output_gpu = NULL;
        SAFE_ALOC_GPU(full_output_gpu, output_bytes());
        if (ahead_fc) {
            fprintf(stderr, "download_full_output(): not available for an FC-ready (ahead_fc) layer.\n");
            exit(-1);
        }
        TCBNN_SAFE_CALL(tcbnn_unpack_conv_output(output_gpu, full_output_gpu, output_height, output_width,
                                                 output_channels, batch, 0));
        HIP_SAFE_CALL(hipMemcpy(full_output, full_output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        SAFE_FREE_GPU(full_output_gpu);
        return full_output;
    }
    void release() {
        SAFE_FREE_HOST(filter);
        SAFE_FREE_HOST(bn);
        SAFE_FREE_HOST(output);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(filter_gpu);
        SAFE_FREE_GPU(bn_gpu);
        if (inject_residual) tcbnn_host::register_residual_consumer(input_residual_gpu, residual_pool, -1, this);
        input_residual_gpu = NULL;
        if (output_residual_gpu != NULL) tcbnn_host::residual_registry().erase(output_residual_gpu);
        SAFE_FREE_GPU(output_residual_gpu);
        SAFE_FREE_GPU(input_own_gpu);
        SAFE_FREE_GPU(input_residual_own_gpu);
        SAFE_FREE_GPU(output_fmt_gpu);
        SAFE_FREE_GPU(output_residual_ref_gpu);
    }
    ~Conv128LayerParam() { release(); }

   public:
    uin32* input;
    uin32* input_gpu;
    int input_width;
    int input_height;
    int input_channels;
    float* filter;
    uin32* filter_gpu;
    int filter_width;
    int filter_height;
    uin32* output;
    uin32* output_gpu;
    int output_width;
    int output_height;
    int output_channels;
    float* bn;
    float* bn_gpu;
    int batch;
    int stride_height;
    int stride_width;
    bool padding;
    int pad_h;
    int pad_w;
    int pool_width;
    int pool_height;
    bool ahead_fc;
    bool save_residual;
    int* output_residual_gpu;
    tcbnn_host::ResidualInfo residual_info;        // of output_residual_gpu
    bool inject_residual;
    int* input_residual_gpu;
    int residual_channels;
    bool residual_pool;
    Conv128LayerParam* gpu;
    char name[8];
    int variant;
    int input_residual_channels;
    tcbnn_host::ResidualInfo input_residual_info;  // of input_residual_gpu
    int buf_height, buf_width;
    uin32* input_own_gpu = NULL;         // engine-layout copies of a reference-layout input / injected residual
    int* input_residual_own_gpu = NULL;
    uin32* output_fmt_gpu = NULL;        // reference-layout copies of the output and the saved residual
    int* output_residual_ref_gpu = NULL;
};

// ======================================================================================
// Layers of the textbook ResNet wiring.  NO counterpart among the reference's classes (its ResNet
// has no pooling layer after the first convolution, no convolutional shortcut and a binarized FC
// head, imagenet_resnet.cu:223-325); same conventions as the classes above.

// Overlapping OR / max pooling of a packed activation tensor and, optionally, its residual.
class Pool128LayerParam {
   public:
    Pool128LayerParam(const char* _name, int _input_height, int _input_width, int _channels, int _batch,
                      int _window = 3, int _stride = 2, int _padding = 1, bool _pool_residual = false)
        : input_gpu(NULL), input_residual_gpu(NULL), output_gpu(NULL), output_residual_gpu(NULL),
          input_height(_input_height), input_width(_input_width), output_channels(_channels), batch(_batch),
          window(_window), stride(_stride), padding(_padding), pool_residual(_pool_residual) {
        strncpy(name, _name, 8);
        output_height = buf_height = tcbnn_pool_out(input_height, window, stride, padding);
        output_width = buf_width = tcbnn_pool_out(input_width, window, stride, padding);
        residual_info = tcbnn_host::make_residual_info(0, 0, _batch);
        residual_info.format = TCBNN_RES_I32;
    }
    ~Pool128LayerParam() { release(); }
    Pool128LayerParam* initialize(uin32* prev_layer_gpu, int* _input_residual_gpu = NULL) {
        CHECK_NULL_POINTER(prev_layer_gpu);
        input_gpu = prev_layer_gpu;
        SAFE_ALOC_GPU(output_gpu, 4 * tcbnn_conv_act_words(output_height, output_width, batch, output_channels));
        if (pool_residual) {
            CHECK_NULL_POINTER(_input_residual_gpu);
            input_residual_gpu = _input_residual_gpu;
            std::map<const void*, tcbnn_host::ResidualInfo>& reg = tcbnn_host::residual_registry();
            std::map<const void*, tcbnn_host::ResidualInfo>::iterator it = reg.find(input_residual_gpu);
            tcbnn_host::ResidualInfo foreign = tcbnn_host::make_residual_info(output_channels, INT32_MAX, batch);
            foreign.format = TCBNN_RES_I32;
            const int keep_bound = it != reg.end() ? it->second.bound : foreign.bound;
            const int keep_format = it != reg.end() ? it->second.format : foreign.format;
            tcbnn_host::register_residual_consumer(input_residual_gpu, false, +1, this, &output_residual_gpu, 0);
            residual_info = foreign;  // a maximum keeps bound and format
            residual_info.bound = keep_bound;
            residual_info.format = keep_format;
            residual_info.channels = output_channels;
            SAFE_ALOC_GPU(output_residual_gpu, tcbnn_residual_bytes(output_height, output_width, output_channels,
                                                                    batch, residual_info.format));
            reg[output_residual_gpu] = residual_info;
        }
        return this;
    }
    uin32* get_output_gpu() { return this->output_gpu; }
    int* get_output_residual_gpu() { return this->output_residual_gpu; }
    void forward(hipStream_t stream = 0) {
        tcbnn_pool128_desc d;
        memset(&d, 0, sizeof(d));
        d.input = input_gpu;
        d.output = output_gpu;
        d.input_residual = input_residual_gpu;
        d.output_residual = output_residual_gpu;
        d.input_height = input_height;
        d.input_width = input_width;
        d.channels = output_channels;
        d.batch = batch;
        d.window = window;
        d.stride = stride;
        d.padding = padding;
        d.residual_format = residual_info.format;
        TCBNN_SAFE_CALL(tcbnn_pool128_forward(&d, stream));
    }
    void release() {
        if (pool_residual && input_residual_gpu != NULL)
            tcbnn_host::register_residual_consumer(input_residual_gpu, false, -1, this);
        input_residual_gpu = NULL;
        if (output_residual_gpu != NULL) tcbnn_host::residual_registry().erase(output_residual_gpu);
        SAFE_FREE_GPU(output_gpu);
        SAFE_FREE_GPU(output_residual_gpu);
    }

   public:
    uin32* input_gpu;
    int* input_residual_gpu;
    uin32* output_gpu;
    int* output_residual_gpu;
    int input_height, input_width, output_height, output_width, buf_height, buf_width;
    int output_channels, batch, window, stride, padding;
    bool pool_residual;
    tcbnn_host::ResidualInfo residual_info;
    char name[8];
};

// Global average pool over a residual tensor + fp32 fully connected layer.  Weight file order: the fp32
// weight matrix [channels][out_features], then the bias.
class AvgPoolFcLayerParam {
   public:
    AvgPoolFcLayerParam(const char* _name, int _input_height, int _input_width, int _channels, int _batch,
                        int _out_features)
        : input_residual_gpu(NULL), weight(NULL), weight_gpu(NULL), bias(NULL), bias_gpu(NULL), output(NULL),
          output_gpu(NULL), input_height(_input_height), input_width(_input_width), channels(_channels),
          batch(_batch), out_features(_out_features) {
        strncpy(name, _name, 8);
        input_residual_info.channels = channels;
        input_residual_info.bound = INT32_MAX;
        input_residual_info.format = TCBNN_RES_I32;
    }
    ~AvgPoolFcLayerParam() { release(); }
    int weight_size() { return channels * out_features; }
    int output_bytes() { return batch * out_features * (int)sizeof(float); }
    AvgPoolFcLayerParam* initialize(tcbnn_host::ConfigSource config_file, int* _input_residual_gpu) {
        CHECK_NULL_POINTER(_input_residual_gpu);
        input_residual_gpu = _input_residual_gpu;
        std::map<const void*, tcbnn_host::ResidualInfo>& reg = tcbnn_host::residual_registry();
        std::map<const void*, tcbnn_host::ResidualInfo>::iterator it = reg.find(input_residual_gpu);
        if (it != reg.end()) input_residual_info = it->second;
        tcbnn_host::register_residual_consumer(input_residual_gpu, false, +1);  // (reads the full tensor)
        SAFE_ALOC_HOST(weight, weight_size() * sizeof(float));
        config_file.read(weight, weight_size());
        SAFE_ALOC_GPU(weight_gpu, weight_size() * sizeof(float));
        HIP_SAFE_CALL(hipMemcpy(weight_gpu, weight, weight_size() * sizeof(float), hipMemcpyHostToDevice));
        SAFE_ALOC_HOST(bias, out_features * sizeof(float));
        config_file.read(bias, out_features);
        SAFE_ALOC_GPU(bias_gpu, out_features * sizeof(float));
        HIP_SAFE_CALL(hipMemcpy(bias_gpu, bias, out_features * sizeof(float), hipMemcpyHostToDevice));
        SAFE_ALOC_GPU(output_gpu, output_bytes());
        return this;
    }
    float* get_output_gpu() { return this->output_gpu; }
    void forward(hipStream_t stream = 0) {
        tcbnn_avgpool_fc_desc d;
        memset(&d, 0, sizeof(d));
        d.input_residual = input_residual_gpu;
        d.weight = weight_gpu;
        d.bias = bias_gpu;
        d.output = output_gpu;
        d.input_height = input_height;
        d.input_width = input_width;
        d.channels = channels;
        d.batch = batch;
        d.out_features = out_features;
        d.residual_format = input_residual_info.format;
        TCBNN_SAFE_CALL(tcbnn_avgpool_fc_forward(&d, stream));
    }
    float* download_output() {
        if (output == NULL) SAFE_ALOC_HOST(output, output_bytes());
        HIP_SAFE_CALL(hipMemcpy(output, output_gpu, output_bytes(), hipMemcpyDeviceToHost));
        return this->output;
    }
    void release() {
        SAFE_FREE_HOST(weight);
        SAFE_FREE_HOST(bias);
        SAFE_FREE_HOST(output);
        SAFE_FREE_GPU(weight_gpu);
        SAFE_FREE_GPU(bias_gpu);
        SAFE_FREE_GPU(output_gpu);
    }

   public:
    int* input_residual_gpu;
    float* weight;
    float* weight_gpu;
    float* bias;
    float* bias_gpu;
    float* output;
    float* output_gpu;
    int input_height, input_width, channels, batch, out_features;
    tcbnn_host::ResidualInfo input_residual_info;
    char name[8];
};

