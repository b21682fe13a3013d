// First-layer convolution: fp32 3-channel NCHW input, +-1 filters, fp32
// accumulation in the reference's exact order (InConv128LayerFMT,
// kernel.cuh:578-672):
//     acc = 0; for r, for s (in-frame taps only): acc += ((+-f0) + (+-f1)) + (+-f2)
//     bit = !((float)acc < bn[o]);  OR over the pool window;  residual = (int)acc
// One ulp decides a threshold bit, so nothing here may be reassociated: there
// are no multiplies (the sign is applied by flipping the fp32 sign bit with a
// precomputed mask), hence no FMA contraction either.
//
// Mapping: lane = one pooled output pixel of one image, x fastest, so the 64
// lanes of a wave read neighbouring input columns of the same image row; the
// filter sign masks are wave-uniform (scalar loads).  A lane owns 32 output
// channels per pass and builds the packed word in registers.
#include "common.h"

namespace tcbnn {
namespace {

constexpr int kThreads = 256;

struct InConvParams {
    const float* in;       // [B][3][H][W]
    const uint4* masks;    // [taps][opad32] {m0, m1, m2, 0}
    const float* bn;
    uint32_t* out;         // [OH][OW][B][ow]
    int32_t* res;          // [PH][PW][B][O] or null
    int H, W, B, O, opad, ow;
    int R, S, stride_h, stride_w, pad_h, pad_w;
    int PH, PW, pool_h, pool_w, OH, OW;
};

__device__ __forceinline__ float flip(float f, uint32_t m) {
    return __uint_as_float(__float_as_uint(f) ^ m);
}

__global__ __launch_bounds__(kThreads) void inconv_kernel(const InConvParams p) {
    const long long m = (long long)blockIdx.x * kThreads + threadIdx.x;
    const long long total = (long long)p.B * p.OH * p.OW;
    if (m >= total) return;
    const int ox = (int)(m % p.OW);
    const int oy = (int)((m / p.OW) % p.OH);
    const int b = (int)(m / ((long long)p.OW * p.OH));
    const size_t plane = (size_t)p.H * p.W;
    const float* img = p.in + (size_t)b * 3 * plane;

    for (int g = 0; g < p.ow; ++g) {
        uint32_t word = 0;
        for (int py = 0; py < p.pool_h; ++py) {
            for (int px = 0; px < p.pool_w; ++px) {
                const int y = oy * p.pool_h + py, x = ox * p.pool_w + px;
                if (y >= p.PH || x >= p.PW) continue;
                const int ay0 = y * p.stride_h - p.pad_h, ax0 = x * p.stride_w - p.pad_w;
                float acc[32];
#pragma unroll
                for (int n = 0; n < 32; ++n) acc[n] = 0.0f;
                for (int r = 0; r < p.R; ++r) {
                    const int ay = ay0 + r;
                    if (ay < 0 || ay >= p.H) continue;
                    for (int s = 0; s < p.S; ++s) {
                        const int ax = ax0 + s;
                        if (ax < 0 || ax >= p.W) continue;
                        const size_t off = (size_t)ay * p.W + ax;
                        const float f0 = img[off];
                        const float f1 = img[plane + off];
                        const float f2 = img[2 * plane + off];
                        const uint4* mk = p.masks + (size_t)(r * p.S + s) * p.opad + g * 32;
#pragma unroll
                        for (int n = 0; n < 32; ++n) {
                            const uint4 mm = mk[n];
                            acc[n] += (flip(f0, mm.x) + flip(f1, mm.y)) + flip(f2, mm.z);
                        }
                    }
                }
#pragma unroll
                for (int n = 0; n < 32; ++n) {
                    const int ch = g * 32 + n;
                    if (ch < p.O) word |= (acc[n] < p.bn[ch] ? 0u : 1u) << (31 - n);
                }
                if (p.res != nullptr) {
                    int32_t* dst = p.res + (((size_t)y * p.PW + x) * p.B + b) * p.O;
#pragma unroll
                    for (int n = 0; n < 32; ++n)
                        if (g * 32 + n < p.O) dst[g * 32 + n] = (int)acc[n];
                }
            }
        }
        p.out[(((size_t)oy * p.OW + ox) * p.B + b) * p.ow + g] = word;
    }
}

}  // namespace
}  // namespace tcbnn

using namespace tcbnn;

extern "C" int tcbnn_inconv128_forward(const tcbnn_inconv128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input);
    TCBNN_NOTNULL(d->filter);
    TCBNN_NOTNULL(d->bn);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_channels == 3,
                  "inconv128: the first layer takes 3 input channels (kernel.cuh:620-625)");
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->batch > 0 &&
                      d->output_channels > 0 && d->filter_height > 0 && d->filter_width > 0 &&
                      d->stride_height > 0 && d->stride_width > 0 && d->pool_height > 0 &&
                      d->pool_width > 0,
                  "inconv128: bad shape");
    if (d->save_residual) {
        TCBNN_NOTNULL(d->output_residual);
        TCBNN_REQUIRE(d->pool_height == 1 && d->pool_width == 1,
                      "inconv128: save_residual requires pool 1x1");
    }
    InConvParams p;
    p.in = d->input;
    p.masks = reinterpret_cast<const uint4*>(d->filter);
    p.bn = d->bn;
    p.out = d->output;
    p.res = d->save_residual ? d->output_residual : nullptr;
    p.H = d->input_height;
    p.W = d->input_width;
    p.B = d->batch;
    p.O = d->output_channels;
    p.opad = pad32(p.O);
    p.ow = step32(p.O);
    p.R = d->filter_height;
    p.S = d->filter_width;
    p.stride_h = d->stride_height;
    p.stride_w = d->stride_width;
    p.pad_h = tcbnn_conv_pad(p.H, p.R, p.stride_h, d->padding);
    p.pad_w = tcbnn_conv_pad(p.W, p.S, p.stride_w, d->padding);
    p.pool_h = d->pool_height;
    p.pool_w = d->pool_width;
    p.PH = tcbnn_conv_out(p.H, p.R, p.stride_h, d->padding, 1);
    p.PW = tcbnn_conv_out(p.W, p.S, p.stride_w, d->padding, 1);
    TCBNN_REQUIRE(p.PH > 0 && p.PW > 0, "inconv128: empty output");
    p.OH = (p.PH + p.pool_h - 1) / p.pool_h;
    p.OW = (p.PW + p.pool_w - 1) / p.pool_w;
    const long long total = (long long)p.B * p.OH * p.OW;
    const long long blocks = (total + kThreads - 1) / kThreads;
    TCBNN_REQUIRE(blocks <= 0x7fffffffLL, "inconv128: grid too large");
    hipLaunchKernelGGL(inconv_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                       (hipStream_t)stream, p);
    TCBNN_LAUNCH_CHECK("inconv_kernel");
    return TCBNN_OK;
}
