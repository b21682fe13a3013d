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
//   residuals    int32 [P][Q][ceil(O/4)][B][4] or int16 [P][Q][ceil(O/8)][B][8]
// ---------------------------------------------------------------------------
enum EpilogueMode : int {
    EPI_THRESH = 0,  // threshold -> bit, OR over the pool window, packed store
    EPI_AFFINE = 1,  // (K - 2c)*scale + bias -> fp32 [B][N]
    EPI_RAW = 2,     // +-1 dot product -> int32
};

struct BgemmParams {
    const uint32_t* act;  // [H][W][cw][B]
    const uint32_t* wgt;  // [npad32][taps*cw]
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
    // split-K (FC-shaped problems only): partial popcounts are atomically added into
    // workspace[n*B + b] and a finishing kernel applies the epilogue
    int32_t* workspace;
    int ksplit;
    int ws_is_dot;  // workspace holds +-1 dot products (matrix-core engines) instead of popcounts
};

// One residual value in either storage format.  Both interleave small groups of channels below
// the batch index, so that a lane (= image) reads or writes 16 contiguous bytes per access:
//   TCBNN_RES_I32: int32 [pix][ceil(ch/4)][B][4]     TCBNN_RES_I16: int16 [pix][ceil(ch/8)][B][8]
__device__ __forceinline__ size_t residual_index(int fmt, size_t pix, int channels, int c, int batch, int b) {
    if (fmt == TCBNN_RES_I16) return ((pix * (size_t)((channels + 7) / 8) + (c >> 3)) * batch + b) * 8 + (c & 7);
    return ((pix * (size_t)((channels + 3) / 4) + (c >> 2)) * batch + b) * 4 + (c & 3);
}
__device__ __forceinline__ int residual_load(const int32_t* __restrict__ base, int fmt, size_t pix, int channels,
                                             int c, int batch, int b) {
    const size_t i = residual_index(fmt, pix, channels, c, batch, b);
    return fmt == TCBNN_RES_I16 ? (int)reinterpret_cast<const int16_t*>(base)[i] : base[i];
}
__device__ __forceinline__ void residual_store(int32_t* __restrict__ base, int fmt, size_t pix, int channels, int c,
                                               int batch, int b, int v) {
    const size_t i = residual_index(fmt, pix, channels, c, batch, b);
    if (fmt == TCBNN_RES_I16)
        reinterpret_cast<int16_t*>(base)[i] = (int16_t)v;
    else
        base[i] = v;
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
