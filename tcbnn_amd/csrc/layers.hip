// C-ABI entry points of the bit-matmul / bit-convolution layers: descriptor
// validation and translation into the implicit-GEMM problem.
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <thread>
#include <vector>

#include "common.h"

namespace tcbnn {

static thread_local char g_err[512] = "";
static std::atomic<int> g_default_variant{-1};

// ---- split-K scratch of tcbnn_fc128_forward_static_scratch -------------------------------------------------
// Device memory that belongs to the loaded code object, not to an allocation: int32 [NPAD32][B] partial sums of
// a split-K fully connected layer.  Every GPU the library runs on holds its own copy at its own address until the
// process ends.  In host code the array's NAME is only a handle for hipGetSymbolAddress: it is never passed to a
// kernel or a copy; the address that call returns for the current device is.
constexpr size_t kStaticScratchWords = size_t(1) << 20;  // 4 MiB per GPU
static __device__ __align__(256) int32_t scratch[kStaticScratchWords];
constexpr int kMaxDevices = 64;
static std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the current device, resolved once per device with that device current.
static int static_scratch(int32_t** out) {
    int dev = -1;
    if (int rc = check_hip(hipGetDevice(&dev), "hipGetDevice")) return rc;
    if (dev < 0 || dev >= kMaxDevices) return fail(TCBNN_EUNSUPPORTED, "static scratch: device ordinal %d", dev);
    int32_t* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        void* sym = nullptr;
        if (int rc = check_hip(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
        if (sym == nullptr) return fail(TCBNN_EHIP, "static scratch: no device address on device %d", dev);
        ptr = static_cast<int32_t*>(sym);
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // the same value from whichever thread gets here
    }
    *out = ptr;
    return TCBNN_OK;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return TCBNN_OK;
    return fail(TCBNN_EHIP, "%s failed: %s", what, hipGetErrorString(e));
}

// Default engine: the FP4 matrix-core kernels (measured fastest on every layer shape of the
// three networks; the XOR+popcount and int8 engines stay selectable for comparison).
static int variant_from_env() {
    const char* v = getenv("TCBNN_VARIANT");
    if (v == nullptr) return TCBNN_VARIANT_MFMA_F4;
    if (!strcmp(v, "popc")) return TCBNN_VARIANT_POPC;
    if (!strcmp(v, "mfma_i8")) return TCBNN_VARIANT_MFMA_I8;
    if (!strcmp(v, "mfma_f4")) return TCBNN_VARIANT_MFMA_F4;
    return TCBNN_VARIANT_MFMA_F4;
}

int resolve_variant(int requested) {
    if (requested != TCBNN_VARIANT_AUTO) return requested;
    int v = g_default_variant.load();
    if (v < 0) {
        v = variant_from_env();
        g_default_variant.store(v);
    }
    return v;
}

static int run_bgemm(const BgemmParams& p, int variant, hipStream_t stream) {
    const int v = resolve_variant(variant);
    switch (v) {
        case TCBNN_VARIANT_POPC:
            return launch_bgemm_popc(p, stream);
        case TCBNN_VARIANT_MFMA_I8:
        case TCBNN_VARIANT_MFMA_F4:
            return launch_bgemm_mfma(p, v, stream);
        default:
            return fail(TCBNN_EINVAL, "unknown variant %d", v);
    }
}

static BgemmParams fc_problem(const uint32_t* input, const uint32_t* weight, int batch, int k,
                              int n) {
    BgemmParams p;
    memset(&p, 0, sizeof(p));
    p.act = input;
    p.wgt = weight;
    p.wgt_lane_copy = 1;  // (tcbnn_pack_fc_weight wrote it)
    p.H = p.W = 1;
    p.B = batch;
    p.cw = kw128(k);
    p.R = p.S = 1;
    p.stride_h = p.stride_w = 1;
    p.PH = p.PW = p.OH = p.OW = 1;
    p.pool_h = p.pool_w = 1;
    p.N = n;
    p.k_tap = k;
    p.ksplit = 1;
    return p;
}

}  // namespace tcbnn

using namespace tcbnn;

extern "C" {

int tcbnn_abi_version(void) { return 7; }
const char* tcbnn_last_error(void) { return g_err; }

int tcbnn_set_default_variant(int variant) {
    TCBNN_REQUIRE(variant >= TCBNN_VARIANT_POPC && variant <= TCBNN_VARIANT_MFMA_F4,
                  "set_default_variant: unknown variant %d", variant);
    g_default_variant.store(variant);
    return TCBNN_OK;
}
int tcbnn_get_default_variant(void) { return resolve_variant(TCBNN_VARIANT_AUTO); }

int tcbnn_conv_pad(int in_size, int filter, int stride, int padding) {
    if (!padding || stride <= 0) return 0;
    return (((in_size + stride - (in_size % stride)) / stride - 1) * stride + filter - in_size) / 2;
}
int tcbnn_conv_out(int in_size, int filter, int stride, int padding, int pool) {
    if (stride <= 0 || pool <= 0) return 0;
    const int buf = padding ? (in_size + stride - 1) / stride : (in_size - filter) / stride + 1;
    return (buf + pool - 1) / pool;
}

size_t tcbnn_fc_act_words(int batch, int features) { return (size_t)batch * kw128(features); }
size_t tcbnn_conv_act_words(int height, int width, int batch, int ch) {
    return (size_t)height * width * batch * step32(ch);
}
size_t tcbnn_fc_weight_words(int in_features, int out_features) {
    // sign-bit rows, then the same words in the FP4 FC kernel's lane order
    return fc_weight_row_words(pad32(out_features), kw128(in_features)) +
           fc_weight_lane_words(pad32(out_features), kw128(in_features));
}
size_t tcbnn_conv_filter_words(int r, int s, int in_ch, int out_ch) {
    const size_t bits = (size_t)pad32(out_ch) * r * s * step32(in_ch);
    // 3x3 filters of the persistent matrix-core kernel carry a second copy in the order its lanes expand them
    return filter_has_fragments(r, s, in_ch) ? 2 * bits : bits;
}
size_t tcbnn_inconv_filter_words(int r, int s, int in_ch, int out_ch) {
    (void)in_ch;
    return (size_t)r * s * pad32(out_ch) * 5;
}

size_t tcbnn_residual_bytes(int height, int width, int channels, int batch, int format) {
    if (height <= 0 || width <= 0 || channels <= 0 || batch <= 0 || !residual_format_known(format)) return 0;
    const size_t pix_b = (size_t)height * width * batch;
    const size_t per = residual_group_channels(format);
    return pix_b * residual_group_bytes(format) * ((channels + per - 1) / per);
}

int tcbnn_inconv_residual_bound(int filter_height, int filter_width, float input_abs_max) {
    if (filter_height <= 0 || filter_width <= 0 || !(input_abs_max >= 0.0f) || std::isinf(input_abs_max))
        return INT32_MAX;
    // R*S*3 terms of magnitude <= input_abs_max; fp32 rounding of the running sum adds far less
    // than the 0.1 % + 1 of slack taken here
    const double bound = (double)filter_height * filter_width * 3.0 * (double)input_abs_max * 1.001 + 1.0;
    return bound < (double)(INT32_MAX / 2) ? (int)std::ceil(bound) : INT32_MAX;
}

int tcbnn_conv_residual_bound(int input_channels, int filter_height, int filter_width, int injected_bound) {
    if (input_channels <= 0 || filter_height <= 0 || filter_width <= 0 || injected_bound < 0) return INT32_MAX;
    const long long bound = (long long)input_channels * filter_height * filter_width + injected_bound;
    return bound < INT32_MAX / 2 ? (int)bound : INT32_MAX;
}

int tcbnn_residual_format_for_bound(int bound) {
    return bound >= 0 && bound <= 32767 ? TCBNN_RES_I16 : TCBNN_RES_I32;
}

int tcbnn_residual_format_narrowest(int bound, int batch) {
    if (bound >= 0 && bound <= 2047 && batch > 0 && batch % 2 == 0) return TCBNN_RES_I12;
    return tcbnn_residual_format_for_bound(bound);
}

// The first layer's sum at an output pixel is a signed sum of the inputs under the filter window, so its
// magnitude is at most the window's sum of |x| (all three channels); fp32 rounding of the 3*R*S additions adds at
// most 3*R*S*2^-24 of that relative, far inside the 0.1 % + 1 of slack taken here.  Per image: prefix sums of
// |x| down the columns give every window's column sums with one subtraction, a prefix sum along the row gives the
// window (double precision: the cancellation error is below 1e-10 of the sums).  Images are dealt to a few host
// threads.
int tcbnn_inconv_residual_bound_of_input(const float* input_host, int batch, int height, int width,
                                         int filter_height, int filter_width, int stride_height,
                                         int stride_width, int padding) {
    if (input_host == nullptr || batch <= 0 || height <= 0 || width <= 0 || filter_height <= 0 ||
        filter_width <= 0 || stride_height <= 0 || stride_width <= 0)
        return INT32_MAX;
    const int pad_h = tcbnn_conv_pad(height, filter_height, stride_height, padding);
    const int pad_w = tcbnn_conv_pad(width, filter_width, stride_width, padding);
    const int oh = tcbnn_conv_out(height, filter_height, stride_height, padding, 1);
    const int ow = tcbnn_conv_out(width, filter_width, stride_width, padding, 1);
    if (oh <= 0 || ow <= 0) return INT32_MAX;
    const size_t plane = (size_t)height * width;
    const int n_threads = std::max(1, std::min(std::min(batch, 16), (int)std::thread::hardware_concurrency()));
    std::vector<double> worst(n_threads, 0.0);
    std::vector<char> bad(n_threads, 0);
    auto scan = [&](int t) {
        std::vector<double> down((size_t)(height + 1) * width), along(width + 1);
        for (int b = t; b < batch && !bad[t]; b += n_threads) {
            const float* img = input_host + (size_t)b * 3 * plane;
            for (int x = 0; x < width; ++x) down[x] = 0.0;
            for (int y = 0; y < height; ++y)
                for (int x = 0; x < width; ++x) {
                    const size_t i = (size_t)y * width + x;
                    const double a = std::fabs((double)img[i]) + std::fabs((double)img[plane + i]) + std::fabs((double)img[2 * plane + i]);
                    if (!(a <= 1e30)) bad[t] = 1;  // NaN or infinity
                    down[(size_t)(y + 1) * width + x] = down[i] + a;
                }
            for (int y = 0; y < oh; ++y) {
                const int y0 = std::max(0, y * stride_height - pad_h), y1 = std::min(height, y * stride_height - pad_h + filter_height);
                if (y1 <= y0) continue;
                along[0] = 0.0;
                for (int x = 0; x < width; ++x)
                    along[x + 1] = along[x] + (down[(size_t)y1 * width + x] - down[(size_t)y0 * width + x]);
                for (int x = 0; x < ow; ++x) {
                    const int x0 = std::max(0, x * stride_width - pad_w), x1 = std::min(width, x * stride_width - pad_w + filter_width);
                    if (x1 > x0) worst[t] = std::max(worst[t], along[x1] - along[x0]);
                }
            }
        }
    };
    std::vector<std::thread> pool;
    for (int t = 1; t < n_threads; ++t) pool.emplace_back(scan, t);
    scan(0);
    for (std::thread& th : pool) th.join();
    double w = 0.0;
    for (int t = 0; t < n_threads; ++t) {
        if (bad[t]) return INT32_MAX;
        w = std::max(w, worst[t]);
    }
    const double bound = w * 1.001 + 1.0;
    return bound < (double)(INT32_MAX / 2) ? (int)std::ceil(bound) : INT32_MAX;
}

// max |x| over a host array, on a few host threads (NaN or infinity anywhere: +infinity)
float tcbnn_host_abs_max(const float* values_host, size_t count) {
    if (values_host == nullptr || count == 0) return 0.0f;
    const int n_threads = (int)std::max<size_t>(1, std::min<size_t>(std::min<size_t>(count >> 20, 16), std::thread::hardware_concurrency()));
    std::vector<float> part(n_threads, 0.0f);
    auto scan = [&](int t) {
        const size_t lo = count * t / n_threads, hi = count * (t + 1) / n_threads;
        float m = 0.0f;
        bool bad = false;
        for (size_t i = lo; i < hi; ++i) {
            const float a = std::fabs(values_host[i]);
            bad |= !(a <= 3.0e38f);
            m = a > m ? a : m;
        }
        part[t] = bad ? INFINITY : m;
    };
    std::vector<std::thread> pool;
    for (int t = 1; t < n_threads; ++t) pool.emplace_back(scan, t);
    scan(0);
    for (std::thread& th : pool) th.join();
    float m = 0.0f;
    for (float v : part) m = v > m ? v : m;
    return m;
}

int tcbnn_fc128_forward(const tcbnn_fc128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input);
    TCBNN_NOTNULL(d->weight);
    TCBNN_NOTNULL(d->bn);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->weight_width > 0,
                  "fc128: bad shape");
    BgemmParams p = fc_problem(d->input, d->weight, d->input_height, d->input_width,
                               d->weight_width);
    p.mode = EPI_THRESH;
    p.nan_bit = 0;  // kernel.cuh:210-213 uses >=, false when unordered
    p.bn = d->bn;
    p.out_bits = d->output;
    p.bits_pix_stride = 0;
    p.bits_row_words = kw128(d->weight_width);
    if (d->workspace != nullptr &&
        d->workspace_words >= (size_t)pad32(d->weight_width) * d->input_height)
        p.workspace = d->workspace;
    return run_bgemm(p, d->variant, (hipStream_t)stream);
}

int tcbnn_fc128_forward_static_scratch(const tcbnn_fc128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->weight_width > 0, "fc128: bad shape");
    const size_t need = (size_t)pad32(d->weight_width) * (size_t)d->input_height;
    TCBNN_REQUIRE(need <= kStaticScratchWords,
                  "fc128 (static scratch): PAD32(weight_width) * input_height = %zu words exceeds the built-in "
                  "scratch of %zu words; use tcbnn_fc128_forward with a workspace of the caller",
                  need, kStaticScratchWords);
    int32_t* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    tcbnn_fc128_desc own = *d;  // the caller's workspace fields are ignored
    own.workspace = ws;         // the device address, never the array's name
    own.workspace_words = kStaticScratchWords;
    return tcbnn_fc128_forward(&own, stream);
}

int tcbnn_out128_forward(const tcbnn_out128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input);
    TCBNN_NOTNULL(d->weight);
    TCBNN_NOTNULL(d->bn_scale);
    TCBNN_NOTNULL(d->bn_bias);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->weight_width > 0,
                  "out128: bad shape");
    BgemmParams p = fc_problem(d->input, d->weight, d->input_height, d->input_width,
                               d->weight_width);
    p.mode = EPI_AFFINE;
    p.bn_scale = d->bn_scale;
    p.bn_bias = d->bn_bias;
    p.out_f32 = d->output;
    return run_bgemm(p, d->variant, (hipStream_t)stream);
}

// The bit-GEMM problem of a Conv128 layer.  `launch`: the pointers are required (forward);
// otherwise only the shape is checked and nullness of the residual pointers follows the flags
// (kernel name of the launch that forward would make).
static int conv_problem(const tcbnn_conv128_desc* d, bool launch, BgemmParams* out) {
    TCBNN_NOTNULL(d);
    if (launch) {
        TCBNN_NOTNULL(d->input);
        TCBNN_NOTNULL(d->filter);
        TCBNN_NOTNULL(d->bn);
        TCBNN_NOTNULL(d->output);
    }
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->batch > 0 &&
                      d->input_channels > 0 && d->output_channels > 0 && d->filter_height > 0 &&
                      d->filter_width > 0 && d->stride_height > 0 && d->stride_width > 0 &&
                      d->pool_height > 0 && d->pool_width > 0,
                  "conv128: bad shape");
    BgemmParams& p = *out;
    memset(&p, 0, sizeof(p));
    p.act = d->input;
    p.wgt = d->filter;
    p.H = d->input_height;
    p.W = d->input_width;
    p.B = d->batch;
    p.cw = step32(d->input_channels);
    p.R = d->filter_height;
    p.S = d->filter_width;
    p.stride_h = d->stride_height;
    p.stride_w = d->stride_width;
    p.pad_h = tcbnn_conv_pad(p.H, p.R, p.stride_h, d->padding);
    p.pad_w = tcbnn_conv_pad(p.W, p.S, p.stride_w, d->padding);
    p.PH = tcbnn_conv_out(p.H, p.R, p.stride_h, d->padding, 1);
    p.PW = tcbnn_conv_out(p.W, p.S, p.stride_w, d->padding, 1);
    TCBNN_REQUIRE(p.PH > 0 && p.PW > 0, "conv128: empty output");
    p.pool_h = d->pool_height;
    p.pool_w = d->pool_width;
    p.OH = (p.PH + p.pool_h - 1) / p.pool_h;
    p.OW = (p.PW + p.pool_w - 1) / p.pool_w;
    p.N = d->output_channels;
    p.k_tap = d->input_channels;
    p.mode = EPI_THRESH;
    p.nan_bit = 1;  // kernel.cuh:795-796: (res < bn) ? 0 : 1
    p.bn = d->bn;
    p.out_bits = d->output;
    const int ow = step32(p.N);
    // FC-ready output pads every pixel's channels to 128 (kernel.cuh:798-808); with the
    // batch-innermost layout that is the only difference from the normal conv output
    p.bits_row_words = d->ahead_fc ? kw128(p.N) : ow;
    p.bits_pix_stride = (long long)p.bits_row_words * p.B;
    p.ksplit = 1;
    // a stand-in for a residual pointer the name query does not need
    int32_t* const some = reinterpret_cast<int32_t*>(const_cast<tcbnn_conv128_desc*>(d));
    if (d->inject_residual) {
        if (launch) TCBNN_NOTNULL(d->input_residual);
        TCBNN_REQUIRE(d->input_residual_channels > 0, "conv128: input_residual_channels unset");
        TCBNN_REQUIRE(d->residual_channels >= 0, "conv128: negative residual_channels");
        p.res_in = launch ? d->input_residual : some;
        p.res_in_ch = d->input_residual_channels;
        p.res_limit = d->residual_channels;
        p.res_pool = d->residual_pool ? 1 : 0;
        TCBNN_REQUIRE(residual_format_known(d->input_residual_format), "conv128: unknown input_residual_format");
        TCBNN_REQUIRE(d->input_residual_format != TCBNN_RES_I12 || d->batch % 2 == 0,
                      "conv128: a 12-bit residual needs an even batch");
        p.res_in_fmt = d->input_residual_format;
    }
    if (d->save_residual) {
        if (launch) TCBNN_NOTNULL(d->output_residual);
        TCBNN_REQUIRE(residual_format_known(d->output_residual_format), "conv128: unknown output_residual_format");
        TCBNN_REQUIRE(d->output_residual_format != TCBNN_RES_I12 || d->batch % 2 == 0,
                      "conv128: a 12-bit residual needs an even batch");
        p.res_out = launch ? d->output_residual : some;
        p.res_out_fmt = d->output_residual_format;
    }
    if (d->output_residual_pool != 0) {
        TCBNN_REQUIRE(d->output_residual_pool == 2, "conv128: output_residual_pool is 0 or 2");
        TCBNN_REQUIRE(d->save_residual, "conv128: output_residual_pool without save_residual");
        p.res_out_pool = 1;
    }
    return TCBNN_OK;
}

// The saved residual as the maximum over 2x2 windows exists in the persistent 3x3 matrix-core kernel only.
static bool pooled_save_served(const BgemmParams& p, int variant) {
    return resolve_variant(variant) == TCBNN_VARIANT_MFMA_F4 && conv3x3_mfma_applicable(p);
}

int tcbnn_conv128_forward(const tcbnn_conv128_desc* d, void* stream) {
    BgemmParams p;
    if (int rc = conv_problem(d, true, &p)) return rc;
    if (p.res_out_pool && !pooled_save_served(p, d->variant))
        return fail(TCBNN_EUNSUPPORTED, "conv128: output_residual_pool is not available for this layer "
                                        "(tcbnn_conv128_pooled_save_supported tells)");
    return run_bgemm(p, d->variant, (hipStream_t)stream);
}

int tcbnn_conv128_pooled_save_supported(const tcbnn_conv128_desc* d) {
    if (d == nullptr || !d->save_residual) return 0;
    tcbnn_conv128_desc own = *d;
    own.output_residual_pool = 2;
    BgemmParams p;
    if (conv_problem(&own, false, &p) != TCBNN_OK) return 0;
    return pooled_save_served(p, d->variant) ? 1 : 0;
}

static int kernel_name(const BgemmParams& p, int variant, char* buf, size_t len) {
    TCBNN_NOTNULL(buf);
    TCBNN_REQUIRE(len > 0, "kernel_name: empty buffer");
    const int v = resolve_variant(variant);
    if (v == TCBNN_VARIANT_POPC)
        bgemm_popc_kernel_name(p, buf, len);
    else
        bgemm_mfma_kernel_name(p, v, buf, len);
    return TCBNN_OK;
}

int tcbnn_conv128_kernel_name(const tcbnn_conv128_desc* d, char* buf, size_t len) {
    BgemmParams p;
    if (int rc = conv_problem(d, false, &p)) return rc;
    return kernel_name(p, d->variant, buf, len);
}
int tcbnn_fc128_kernel_name(const tcbnn_fc128_desc* d, char* buf, size_t len) {
    TCBNN_NOTNULL(d);
    BgemmParams p = fc_problem(nullptr, nullptr, d->input_height, d->input_width, d->weight_width);
    if (d->workspace != nullptr &&
        d->workspace_words >= (size_t)pad32(d->weight_width) * d->input_height)
        p.workspace = d->workspace;
    return kernel_name(p, d->variant, buf, len);
}

int tcbnn_out128_kernel_name(const tcbnn_out128_desc* d, char* buf, size_t len) {
    TCBNN_NOTNULL(d);
    BgemmParams p = fc_problem(nullptr, nullptr, d->input_height, d->input_width, d->weight_width);
    p.mode = EPI_AFFINE;
    return kernel_name(p, d->variant, buf, len);
}

int tcbnn_bmm(const uint32_t* a, const uint32_t* b, int32_t* c, int m, int n, int k, int variant,
              void* stream) {
    TCBNN_NOTNULL(a);
    TCBNN_NOTNULL(b);
    TCBNN_NOTNULL(c);
    TCBNN_REQUIRE(m > 0 && n > 0 && k > 0, "bmm: empty dimension");
    TCBNN_REQUIRE(k % 32 == 0, "bmm: K must be a multiple of 32");
    TCBNN_REQUIRE(n % 32 == 0, "bmm: N must be a multiple of 32 (B holds one packed row per column)");
    BgemmParams p;
    memset(&p, 0, sizeof(p));
    p.act = a;
    p.wgt = b;
    p.H = p.W = 1;
    p.B = m;
    p.cw = k / 32;
    p.R = p.S = 1;
    p.stride_h = p.stride_w = 1;
    p.PH = p.PW = p.OH = p.OW = 1;
    p.pool_h = p.pool_w = 1;
    p.N = n;
    p.k_tap = k;
    p.mode = EPI_RAW;
    p.ksplit = 1;
    p.out_i32 = c;
    p.raw_pix_stride = 0;
    p.raw_b_stride = n;
    return run_bgemm(p, variant, (hipStream_t)stream);
}

int tcbnn_bconv(const uint32_t* input, const uint32_t* filter, int32_t* output, int batch,
                int height, int width, int in_ch, int out_ch, int r, int s, int stride_h,
                int stride_w, int pad_h, int pad_w, int out_h, int out_w, int variant,
                void* stream) {
    TCBNN_NOTNULL(input);
    TCBNN_NOTNULL(filter);
    TCBNN_NOTNULL(output);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && in_ch > 0 && out_ch > 0 && r > 0 &&
                      s > 0 && stride_h > 0 && stride_w > 0 && out_h > 0 && out_w > 0 &&
                      pad_h >= 0 && pad_w >= 0,
                  "bconv: bad shape");
    BgemmParams p;
    memset(&p, 0, sizeof(p));
    p.act = input;
    p.wgt = filter;
    p.H = height;
    p.W = width;
    p.B = batch;
    p.cw = step32(in_ch);
    p.R = r;
    p.S = s;
    p.stride_h = stride_h;
    p.stride_w = stride_w;
    p.pad_h = pad_h;
    p.pad_w = pad_w;
    p.PH = p.OH = out_h;
    p.PW = p.OW = out_w;
    p.pool_h = p.pool_w = 1;
    p.N = out_ch;
    p.k_tap = in_ch;
    p.mode = EPI_RAW;
    p.ksplit = 1;
    p.out_i32 = output;
    p.raw_pix_stride = out_ch;
    p.raw_b_stride = (long long)out_h * out_w * out_ch;
    return run_bgemm(p, variant, (hipStream_t)stream);
}

}  // extern "C"
