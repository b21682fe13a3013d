// Shared host/device helpers of the gfx950 BNN inference library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string>

#include "../../include/tcbnn_hip.h"

namespace tcbnn {

// STEPn / PADn of the reference (utility.h:33-45).
__host__ __device__ constexpr inline int step32(int x) { return (x + 31) >> 5; }
__host__ __device__ constexpr inline int step128(int x) { return (x + 127) >> 7; }
__host__ __device__ constexpr inline int pad8(int x) { return ((x + 7) >> 3) << 3; }
__host__ __device__ constexpr inline int pad32(int x) { return step32(x) << 5; }
__host__ __device__ constexpr inline int pad128(int x) { return step128(x) << 7; }
// words per FC activation / weight row
__host__ __device__ constexpr inline int kw128(int k) { return 4 * step128(k); }

int fail(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);
int resolve_variant(int requested);

#define TCBNN_REQUIRE(cond, ...)                                  \
    do {                                                          \
        if (!(cond)) return ::tcbnn::fail(TCBNN_EINVAL, __VA_ARGS__); \
    } while (0)
#define TCBNN_NOTNULL(p)                                                              \
    do {                                                                              \
        if ((p) == nullptr) return ::tcbnn::fail(TCBNN_ENULL, "NULL pointer: %s", #p); \
    } while (0)
#define TCBNN_LAUNCH_CHECK(name)                                      \
    do {                                                              \
        int rc__ = ::tcbnn::check_hip(hipGetLastError(), name);       \
        if (rc__) return rc__;                                        \
    } while (0)

// ---------------------------------------------------------------------------
// Implicit-GEMM problem shared by the FC, Out, Conv, bmm and bconv entry points.
// Rows of the GEMM are (pre-pool output pixel, image); columns are output
// neurons/channels; K runs over (filter tap, input-channel word).
//
// Device layouts (batch innermost, so that lane = image makes every activation,
// residual and output access one contiguous run):
//   activations  uint32 [H][W][cw][B]
//   weights      uint32 [npad32][taps*cw]
//   residuals    int32 [P][Q][ceil(O/4)][B][4], int16 [P][Q][ceil(O/8)][B][8] or 12-bit groups of 16 channels
// ---------------------------------------------------------------------------
enum EpilogueMode : int {
    EPI_THRESH = 0,  // threshold -> bit, OR over the pool window, packed store
    EPI_AFFINE = 1,  // (K - 2c)*scale + bias -> fp32 [B][N]
    EPI_RAW = 2,     // +-1 dot product -> int32
};

struct BgemmParams {
    const uint32_t* act;  // [H][W][cw][B]
    const uint32_t* wgt;  // [npad32][taps*cw]
    int wgt_lane_copy;    // wgt is a fully connected layer's buffer: the copy in lane order follows the rows
    int H, W, B, cw;      // input geometry, words per (pixel, image)
    int R, S, stride_h, stride_w, pad_h, pad_w;
    int PH, PW;           // conv output size before pooling
    int pool_h, pool_w;
    int OH, OW;           // after pooling
    int N;                // true number of output columns
    int k_tap;            // true K per tap (Cin, or K for FC)
    int mode;
    int nan_bit;          // bit emitted when the threshold compare is unordered
    // EPI_THRESH: word (pooled pixel, word w, image b) at out_bits[pix*bits_pix_stride + w*B + b]
    const float* bn;
    uint32_t* out_bits;
    long long bits_pix_stride;
    int bits_row_words;  // words per pixel; those past ceil(N/32) are written as 0
    // EPI_AFFINE
    const float* bn_scale;
    const float* bn_bias;
    float* out_f32;  // [B][N]
    // EPI_RAW: out_i32[pix*raw_pix_stride + b*raw_b_stride + n], indexed by pre-pool pixel
    int32_t* out_i32;
    long long raw_pix_stride, raw_b_stride;
    // residuals (pool 1x1 only)
    const int32_t* res_in;  // [Hr][Wr][res_in_ch][B]
    int res_in_ch;          // channels of the source
    int res_limit;          // inject only into n < res_limit
    int res_pool;           // 2x2 max over a source twice the output size
    int32_t* res_out;       // [PH][PW][N][B]
    int res_in_fmt, res_out_fmt;  // TCBNN_RES_* of res_in / res_out
    int res_out_pool;             // res_out holds the maximum over 2x2 windows of output pixels: [PH/2][PW/2][N][B]
    // split-K (FC-shaped problems only): partial popcounts are atomically added into
    // workspace[n*B + b] and a finishing kernel applies the epilogue
    int32_t* workspace;
    int ksplit;
    int ws_is_dot;  // workspace holds +-1 dot products (matrix-core engines) instead of popcounts
};

// One residual value in any storage format.  All of them interleave small groups of channels below the batch
// index, so that a lane (= image) reads or writes whole 16- or 8-byte pieces and consecutive lanes are contiguous:
//   TCBNN_RES_I32: int32 [pix][ceil(ch/4)][B][4]     TCBNN_RES_I16: int16 [pix][ceil(ch/8)][B][8]
//   TCBNN_RES_I12: groups of 16 channels, 12 bits each = 192 bits = six words w0..w5 per image, value e at bits
//                  12e..12e+11 of that string (two's complement); stored as [pix][ceil(ch/16)] x { uint32 [B][4]
//                  (w0..w3), then uint32 [B][2] (w4, w5) }: 24 B bytes per (pixel, group)
__host__ __device__ constexpr inline size_t residual_group_channels(int fmt) {
    return fmt == TCBNN_RES_I12 ? 16 : (fmt == TCBNN_RES_I16 ? 8 : 4);
}
__host__ __device__ constexpr inline size_t residual_group_bytes(int fmt) { return fmt == TCBNN_RES_I12 ? 24 : 16; }
__host__ __device__ constexpr inline bool residual_format_known(int fmt) {
    return fmt == TCBNN_RES_I32 || fmt == TCBNN_RES_I16 || fmt == TCBNN_RES_I12;
}
// word k (0..5) of group g of image b at pixel pix of a 12-bit tensor with G groups per pixel
__device__ __forceinline__ size_t i12_word_index(size_t pix, size_t G, int g, int batch, int b, int k) {
    const size_t base = (pix * G + (size_t)g) * (size_t)batch * 6;
    return k < 4 ? base + (size_t)b * 4 + k : base + (size_t)batch * 4 + (size_t)b * 2 + (k - 4);
}
// eight 12-bit values <-> three words (a 16-channel group is two such units: w0..w2 and w3..w5)
__device__ __forceinline__ void i12_unpack8(uint32_t d0, uint32_t d1, uint32_t d2, int* v) {
    v[0] = ((int)(d0 << 20)) >> 20;
    v[1] = ((int)(d0 << 8)) >> 20;
    v[2] = ((int)__builtin_amdgcn_alignbit(d1, d0, 24) << 20) >> 20;
    v[3] = ((int)(d1 << 16)) >> 20;
    v[4] = ((int)(d1 << 4)) >> 20;
    v[5] = ((int)__builtin_amdgcn_alignbit(d2, d1, 28) << 20) >> 20;
    v[6] = ((int)(d2 << 12)) >> 20;
    v[7] = (int)d2 >> 20;
}
// (only the low 12 bits of each v[] are looked at; 12 instructions: shift-or, and-or, bit-field extract, byte permute)
__device__ __forceinline__ void i12_pack8(const int* v, uint32_t& d0, uint32_t& d1, uint32_t& d2) {
    const uint32_t m = 0xfffu;
    const uint32_t u0 = (uint32_t)v[0], u1 = (uint32_t)v[1], u2 = (uint32_t)v[2], u3 = (uint32_t)v[3], u4 = (uint32_t)v[4],
                   u5 = (uint32_t)v[5], u6 = (uint32_t)v[6], u7 = (uint32_t)v[7];
    const uint32_t a = (u1 << 12) | (u0 & m);                    // v0, v1 in bits 0-23 (above: leftovers of v1)
    d0 = __builtin_amdgcn_perm(u2, a, 0x04020100u);              // ... and the low byte of v2 on top
    const uint32_t lo = (u3 << 4) | __builtin_amdgcn_ubfe(u2, 8, 4);   // bits 0-15: high nibble of v2, v3
    const uint32_t hi = (u5 << 12) | (u4 & m);                         // bits 0-15: v4, low nibble of v5
    d1 = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
    const uint32_t f = (u7 << 12) | (u6 & m);                    // v6, v7 in bits 0-23
    d2 = (f << 8) | __builtin_amdgcn_ubfe(u5, 4, 8);             // high byte of v5 below them
}
__device__ __forceinline__ size_t residual_index(int fmt, size_t pix, int channels, int c, int batch, int b) {
    if (fmt == TCBNN_RES_I16) return ((pix * (size_t)((channels + 7) / 8) + (c >> 3)) * batch + b) * 8 + (c & 7);
    return ((pix * (size_t)((channels + 3) / 4) + (c >> 2)) * batch + b) * 4 + (c & 3);
}
__device__ __forceinline__ int residual_load(const int32_t* __restrict__ base, int fmt, size_t pix, int channels,
                                             int c, int batch, int b) {
    if (fmt == TCBNN_RES_I12) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(base);
        const size_t G = (size_t)((channels + 15) / 16);
        const int g = c >> 4, bit = 12 * (c & 15), k = bit >> 5, sh = bit & 31;
        const uint32_t lo = w[i12_word_index(pix, G, g, batch, b, k)];
        const uint32_t hi = sh > 20 ? w[i12_word_index(pix, G, g, batch, b, k + 1)] : 0u;  // the value straddles two words
        const uint64_t both = ((uint64_t)hi << 32) | lo;
        return ((int)((uint32_t)(both >> sh) << 20)) >> 20;
    }
    const size_t i = residual_index(fmt, pix, channels, c, batch, b);
    return fmt == TCBNN_RES_I16 ? (int)reinterpret_cast<const int16_t*>(base)[i] : base[i];
}
// Stores of single values exist for the 32- and 16-bit formats only (a 12-bit value shares its words with its
// neighbours); every producer writes whole groups of a 12-bit tensor with residual_store_group16.
__device__ __forceinline__ void residual_store(int32_t* __restrict__ base, int fmt, size_t pix, int channels, int c,
                                               int batch, int b, int v) {
    const size_t i = residual_index(fmt, pix, channels, c, batch, b);
    if (fmt == TCBNN_RES_I16)
        reinterpret_cast<int16_t*>(base)[i] = (int16_t)v;
    else
        base[i] = v;
}
// Channels 16g .. 16g+15 of one image and pixel (values of channels >= `channels` are whatever the caller passes;
// consumers never look at them), in any format.
__device__ __forceinline__ void residual_store_group16(int32_t* __restrict__ base, int fmt, size_t pix, int channels,
                                                       int g, int batch, int b, const int* v) {
    if (fmt == TCBNN_RES_I12) {
        uint32_t* w = reinterpret_cast<uint32_t*>(base);
        const size_t G = (size_t)((channels + 15) / 16);
        uint32_t d[6];
        i12_pack8(v, d[0], d[1], d[2]);
        i12_pack8(v + 8, d[3], d[4], d[5]);
        *reinterpret_cast<uint4*>(w + i12_word_index(pix, G, g, batch, b, 0)) = make_uint4(d[0], d[1], d[2], d[3]);
        *reinterpret_cast<uint2*>(w + i12_word_index(pix, G, g, batch, b, 4)) = make_uint2(d[4], d[5]);
        return;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e)
        if (16 * g + e < channels) residual_store(base, fmt, pix, channels, 16 * g + e, batch, b, v[e]);
}
__device__ __forceinline__ void residual_load_group16(const int32_t* __restrict__ base, int fmt, size_t pix, int channels,
                                                      int g, int batch, int b, int* v) {
    if (fmt == TCBNN_RES_I12) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(base);
        const size_t G = (size_t)((channels + 15) / 16);
        const uint4 a = *reinterpret_cast<const uint4*>(w + i12_word_index(pix, G, g, batch, b, 0));
        const uint2 c2 = *reinterpret_cast<const uint2*>(w + i12_word_index(pix, G, g, batch, b, 4));
        i12_unpack8(a.x, a.y, a.z, v);
        i12_unpack8(a.w, c2.x, c2.y, v + 8);
        return;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = 16 * g + e < channels ? residual_load(base, fmt, pix, channels, 16 * g + e, batch, b) : 0;
}

int launch_bgemm_popc(const BgemmParams& p, hipStream_t stream);
int launch_bgemm_mfma(const BgemmParams& p, int variant, hipStream_t stream);
int validate_bgemm(const BgemmParams& p);
// zero the split-K workspace / apply the epilogue to it (shared by both engines)
int launch_splitk_clear(const BgemmParams& p, hipStream_t stream);
int launch_splitk_finish(const BgemmParams& p, hipStream_t stream);
// profiler-style kernel names for a problem
void bgemm_popc_kernel_name(const BgemmParams& p, char* buf, size_t len);
void bgemm_mfma_kernel_name(const BgemmParams& p, int variant, char* buf, size_t len);
// A packed 3x3 filter with Cin = 64 / 128 / 192 / 256 / 384 / 512 carries, after its [OPAD32][9*cw] sign-bit rows, the
// same words in MFMA fragment order: uint32 [OPAD32/32][9*cw/2][64 lanes] (written once by tcbnn_pack_conv_filter;
// the persistent kernel loads a fragment's 64 words with one contiguous request and expands them on the way to LDS).
inline bool filter_has_fragments(int r, int s, int in_ch) {
    return r == 3 && s == 3 &&
           (in_ch == 64 || in_ch == 128 || in_ch == 192 || in_ch == 256 || in_ch == 384 || in_ch == 512);
}
// Packed FC weights carry, after their [NPAD32][KW128] sign-bit rows, the same words in the order the FP4 matrix-core
// FC kernel's lanes load them: uint32 [NPAD32/32][ceil(KW128/8)][64 lanes][4] (lane (j, h) of K group g holds words
// 8g + 4h .. 8g + 4h + 3 of neuron 32 tile + row_to_channel(j); words past KW128 are 0), written once by
// tcbnn_pack_fc_weight: a wave then loads a group with ONE contiguous 1 KB request instead of 16 bytes from each of 64
// rows.
__host__ __device__ inline size_t fc_weight_row_words(int npad, int kw) { return (size_t)npad * kw; }
__host__ __device__ inline size_t fc_weight_lane_words(int npad, int kw) { return (size_t)npad * 8 * ((kw + 7) / 8); }
// persistent FP4 matrix-core kernel for 3x3 convolutions with Cin = 64 / 128 / 192 / 256 / 384 / 512
bool conv3x3_mfma_applicable(const BgemmParams& p);
int launch_conv3x3_mfma(const BgemmParams& p, hipStream_t stream);
void conv3x3_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len);
// FP4 matrix-core kernel for small fully connected layers (K split over the waves of a workgroup)
// large unmasked bit-GEMMs (stand-alone product, FC layers at large batch)
bool gemm_mfma_applicable(const BgemmParams& p);
int launch_gemm_mfma(const BgemmParams& p, hipStream_t stream);
void gemm_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len);
bool fc_mfma_applicable(const BgemmParams& p);
int launch_fc_mfma(const BgemmParams& p, hipStream_t stream);
void fc_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len);
// number of K splits wanted for a problem (1 = none)
int choose_ksplit(const BgemmParams& p);

}  // namespace tcbnn
