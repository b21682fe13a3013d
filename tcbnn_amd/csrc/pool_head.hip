// Layers of the textbook ResNet wiring that the reference's drivers do not have: overlapping
// OR / max pooling of a packed activation tensor with its residual, and the global-average-pool +
// fp32 fully connected head.  Both are bound by HBM (one pass over their input).
#include "common.h"

namespace tcbnn {
namespace {

constexpr int kThreads = 256;

struct PoolParams {
    const uint32_t* in;
    uint32_t* out;
    const int32_t* rin;
    int32_t* rout;
    int H, W, C, B, OH, OW, cw, groups;  // groups = 16-byte residual groups per pixel
    int window, stride, pad, fmt;
};

// One thread per (output pixel, word or residual group, image); the image index runs fastest,
// so a wavefront reads and writes contiguous runs.
__global__ __launch_bounds__(kThreads) void pool128_kernel(const PoolParams p) {
    const long long per_pix = (long long)(p.cw + p.groups) * p.B;
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= per_pix * p.OH * p.OW) return;
    const int opix = (int)(idx / per_pix);
    const int rem = (int)(idx % per_pix);
    const int u = rem / p.B, b = rem % p.B;  // unit (word, then group) and image
    const int oy = opix / p.OW, ox = opix % p.OW;
    const int y0 = oy * p.stride - p.pad, x0 = ox * p.stride - p.pad;
    if (u < p.cw) {  // OR of the window's words
        uint32_t acc = 0;
        for (int r = 0; r < p.window; ++r)
            for (int s = 0; s < p.window; ++s) {
                const int y = y0 + r, x = x0 + s;
                if (y >= 0 && y < p.H && x >= 0 && x < p.W) acc |= p.in[(((size_t)y * p.W + x) * p.cw + u) * p.B + b];
            }
        p.out[((size_t)opix * p.cw + u) * p.B + b] = acc;
        return;
    }
    const int g = u - p.cw;  // maximum of the window's residual groups
    if (p.fmt == TCBNN_RES_I12) {  // groups of 16 channels, unpacked to ints and packed again
        int m[16], v[16];
        bool none = true;
        for (int r = 0; r < p.window; ++r)
            for (int s = 0; s < p.window; ++s) {
                const int y = y0 + r, x = x0 + s;
                if (y < 0 || y >= p.H || x < 0 || x >= p.W) continue;
                residual_load_group16(p.rin, p.fmt, (size_t)y * p.W + x, p.C, g, p.B, b, v);
#pragma unroll
                for (int e = 0; e < 16; ++e) m[e] = none ? v[e] : max(m[e], v[e]);
                none = false;
            }
        if (none)
#pragma unroll
            for (int e = 0; e < 16; ++e) m[e] = 0;
        residual_store_group16(p.rout, p.fmt, (size_t)opix, p.C, g, p.B, b, m);
        return;
    }
    const int4* __restrict__ src = reinterpret_cast<const int4*>(p.rin);
    int4 m;
    bool first = true;
    for (int r = 0; r < p.window; ++r)
        for (int s = 0; s < p.window; ++s) {
            const int y = y0 + r, x = x0 + s;
            if (y < 0 || y >= p.H || x < 0 || x >= p.W) continue;
            const int4 v = src[(((size_t)y * p.W + x) * p.groups + g) * p.B + b];
            if (first) {
                m = v;
                first = false;
            } else if (p.fmt == TCBNN_RES_I16) {  // two int16 per word
                auto max2 = [](int a, int c) {
                    const int lo = max((int)(short)(a & 0xffff), (int)(short)(c & 0xffff));
                    const int hi = max(a >> 16, c >> 16);
                    return (lo & 0xffff) | (hi << 16);
                };
                m = make_int4(max2(m.x, v.x), max2(m.y, v.y), max2(m.z, v.z), max2(m.w, v.w));
            } else {
                m = make_int4(max(m.x, v.x), max(m.y, v.y), max(m.z, v.z), max(m.w, v.w));
            }
        }
    if (first) m = make_int4(0, 0, 0, 0);  // window entirely outside the frame (cannot happen: padding < window)
    reinterpret_cast<int4*>(p.rout)[((size_t)opix * p.groups + g) * p.B + b] = m;
}

struct HeadParams {
    const int32_t* rin;
    const float* w;
    const float* bias;
    float* out;
    int P, C, B, N, groups, per_group, fmt;  // P = pixels
};

constexpr int kHeadImages = 8;     // images per workgroup
constexpr int kHeadOutputs = 256;  // outputs per workgroup (one per thread)
constexpr int kHeadMaxC = 512;

// Workgroup = 8 images x 256 outputs.  Phase 1: the means of the 8 images, all channels, into LDS.
// Phase 2: thread = output; per channel one coalesced weight load and eight fused multiply-adds on
// means that every lane reads from the same LDS address (broadcast); channels in ascending order.
__global__ __launch_bounds__(kThreads) void avgpool_fc_kernel(const HeadParams p) {
    __shared__ __align__(16) float mean[kHeadMaxC][kHeadImages];
    const int tid = threadIdx.x;
    const int b0 = blockIdx.x * kHeadImages;
    const float npix = (float)p.P;
    const int4* __restrict__ src = reinterpret_cast<const int4*>(p.rin);
    for (int u = tid; u < p.groups * kHeadImages; u += kThreads) {
        const int g = u / kHeadImages, i = u % kHeadImages;  // image fastest: 128-byte runs
        const int bb = min(b0 + i, p.B - 1);
        if (p.fmt == TCBNN_RES_I12) {  // groups of 16 channels
            int s16[16], v16[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) s16[e] = 0;
            for (int pix = 0; pix < p.P; ++pix) {
                residual_load_group16(p.rin, p.fmt, (size_t)pix, p.C, g, p.B, bb, v16);
#pragma unroll
                for (int e = 0; e < 16; ++e) s16[e] += v16[e];
            }
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (16 * g + e < p.C) mean[16 * g + e][i] = (float)s16[e] / npix;
            continue;
        }
        int sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        // eight pixels requested at a time (a load per loop pass waits for each one in turn); integer sums, so
        // the order does not matter
        for (int pix0 = 0; pix0 < p.P; pix0 += 8) {
            int4 v[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = src[((size_t)min(pix0 + q, p.P - 1) * p.groups + g) * p.B + bb];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                if (pix0 + q >= p.P) continue;
                if (p.fmt == TCBNN_RES_I16) {
                    const int wv[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        sum[2 * k] += (int)(short)(wv[k] & 0xffff);
                        sum[2 * k + 1] += wv[k] >> 16;
                    }
                } else {
                    sum[0] += v[q].x;
                    sum[1] += v[q].y;
                    sum[2] += v[q].z;
                    sum[3] += v[q].w;
                }
            }
        }
        for (int k = 0; k < p.per_group; ++k) {
            const int c = g * p.per_group + k;
            if (c < p.C) mean[c][i] = (float)sum[k] / npix;
        }
    }
    __syncthreads();
    const int n = blockIdx.y * kHeadOutputs + tid;
    if (n >= p.N) return;
    float acc[kHeadImages];
#pragma unroll
    for (int i = 0; i < kHeadImages; ++i) acc[i] = 0.0f;
    // weights of the next 16 channels are requested while the current 16 are used; the additions stay in ascending
    // channel order
    float wn[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) wn[q] = p.w[(size_t)min(q, p.C - 1) * p.N + n];
    for (int c0 = 0; c0 < p.C; c0 += 16) {
        float wv[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) wv[q] = wn[q];
#pragma unroll
        for (int q = 0; q < 16; ++q) wn[q] = p.w[(size_t)min(c0 + 16 + q, p.C - 1) * p.N + n];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int c = min(c0 + q, p.C - 1);
            const bool on = c0 + q < p.C;  // a channel past C leaves the sums as they are
            const float4 m0 = *reinterpret_cast<const float4*>(&mean[c][0]);
            const float4 m1 = *reinterpret_cast<const float4*>(&mean[c][4]);
            acc[0] = on ? __fmaf_rn(m0.x, wv[q], acc[0]) : acc[0];
            acc[1] = on ? __fmaf_rn(m0.y, wv[q], acc[1]) : acc[1];
            acc[2] = on ? __fmaf_rn(m0.z, wv[q], acc[2]) : acc[2];
            acc[3] = on ? __fmaf_rn(m0.w, wv[q], acc[3]) : acc[3];
            acc[4] = on ? __fmaf_rn(m1.x, wv[q], acc[4]) : acc[4];
            acc[5] = on ? __fmaf_rn(m1.y, wv[q], acc[5]) : acc[5];
            acc[6] = on ? __fmaf_rn(m1.z, wv[q], acc[6]) : acc[6];
            acc[7] = on ? __fmaf_rn(m1.w, wv[q], acc[7]) : acc[7];
        }
    }
    const float bias = p.bias[n];
#pragma unroll
    for (int i = 0; i < kHeadImages; ++i)
        if (b0 + i < p.B) p.out[(size_t)(b0 + i) * p.N + n] = __fadd_rn(acc[i], bias);
}

}  // namespace
}  // namespace tcbnn

using namespace tcbnn;

extern "C" int tcbnn_pool_out(int in_size, int window, int stride, int padding) {
    if (window <= 0 || stride <= 0 || padding < 0 || in_size + 2 * padding < window) return 0;
    return (in_size + 2 * padding - window) / stride + 1;
}

extern "C" int tcbnn_pool128_forward(const tcbnn_pool128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->channels > 0 && d->batch > 0 && d->window > 0 &&
                      d->stride > 0 && d->padding >= 0 && d->padding < d->window,
                  "pool128: bad shape");
    TCBNN_REQUIRE((d->input_residual == nullptr) == (d->output_residual == nullptr),
                  "pool128: input_residual and output_residual go together");
    TCBNN_REQUIRE(d->input_residual == nullptr || residual_format_known(d->residual_format),
                  "pool128: unknown residual_format");
    TCBNN_REQUIRE(d->input_residual == nullptr || d->residual_format != TCBNN_RES_I12 || d->batch % 2 == 0,
                  "pool128: a 12-bit residual needs an even batch");
    PoolParams p;
    p.in = d->input;
    p.out = d->output;
    p.rin = d->input_residual;
    p.rout = d->output_residual;
    p.H = d->input_height;
    p.W = d->input_width;
    p.C = d->channels;
    p.B = d->batch;
    p.OH = tcbnn_pool_out(p.H, d->window, d->stride, d->padding);
    p.OW = tcbnn_pool_out(p.W, d->window, d->stride, d->padding);
    TCBNN_REQUIRE(p.OH > 0 && p.OW > 0, "pool128: empty output");
    p.cw = step32(p.C);
    p.fmt = d->residual_format;
    p.groups = p.rin == nullptr ? 0 : (int)((p.C + residual_group_channels(p.fmt) - 1) / residual_group_channels(p.fmt));
    p.window = d->window;
    p.stride = d->stride;
    p.pad = d->padding;
    const long long total = (long long)(p.cw + p.groups) * p.B * p.OH * p.OW;
    const long long blocks = (total + kThreads - 1) / kThreads;
    TCBNN_REQUIRE(blocks <= 0x7fffffffLL, "pool128: grid too large");
    hipLaunchKernelGGL(pool128_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    TCBNN_LAUNCH_CHECK("pool128_kernel");
    return TCBNN_OK;
}

extern "C" int tcbnn_avgpool_fc_forward(const tcbnn_avgpool_fc_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input_residual);
    TCBNN_NOTNULL(d->weight);
    TCBNN_NOTNULL(d->bias);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->channels > 0 && d->batch > 0 && d->out_features > 0,
                  "avgpool_fc: bad shape");
    TCBNN_REQUIRE(d->channels <= kHeadMaxC, "avgpool_fc: at most 512 channels");
    TCBNN_REQUIRE(residual_format_known(d->residual_format), "avgpool_fc: unknown residual_format");
    TCBNN_REQUIRE(d->residual_format != TCBNN_RES_I12 || d->batch % 2 == 0,
                  "avgpool_fc: a 12-bit residual needs an even batch");
    HeadParams p;
    p.rin = d->input_residual;
    p.w = d->weight;
    p.bias = d->bias;
    p.out = d->output;
    p.P = d->input_height * d->input_width;
    p.C = d->channels;
    p.B = d->batch;
    p.N = d->out_features;
    p.fmt = d->residual_format;
    p.per_group = (int)residual_group_channels(p.fmt);
    p.groups = (p.C + p.per_group - 1) / p.per_group;
    const dim3 grid((unsigned)((p.B + kHeadImages - 1) / kHeadImages), (unsigned)((p.N + kHeadOutputs - 1) / kHeadOutputs));
    hipLaunchKernelGGL(avgpool_fc_kernel, grid, dim3(kThreads), 0, (hipStream_t)stream, p);
    TCBNN_LAUNCH_CHECK("avgpool_fc_kernel");
    return TCBNN_OK;
}
