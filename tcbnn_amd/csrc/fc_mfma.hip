// FP4 matrix-core kernel for small fully connected layers (Fc128LayerFMT / Out128LayerFMT,
// kernel.cuh:174-280) at inference batch sizes: a few hundred images times a few hundred
// neurons is only some hundred 32 x 32 output tiles, far too few to fill 1024 SIMDs when one
// wave walks the whole K of a tile, and K can be long (25088 for the first FC of ResNet-18).
//
//   workgroup = one 32-image x 32-neuron output tile, up to 16 waves;
//   wave      = a contiguous slice of K: it requests its activation and weight words (128-bit
//               weight loads: the K order inside a group of 8 words is chosen so that a lane
//               owns 4 consecutive words), multiplies them, and adds its partial tile into LDS
//               with integer atomics (the partial sums are exact integers);
//   wave 0    = epilogue: threshold + pack (FC) or scale + bias (output layer).
// No split-K workspace in HBM, no clearing or finishing launch.
#include <algorithm>
#include <type_traits>

#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

using namespace mfma;

constexpr int kMaxWaves = 16;
constexpr int FC_THRESH = 0, FC_AFFINE = 1;

// PRE > 0: the wave's K slice is at most PRE groups and is requested whole before the first multiply.
template <int MODE, int PRE>
__global__ __launch_bounds__(64 * kMaxWaves) void fc_mfma_f4_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const float* __restrict__ bias, int n_tiles, int groups_per_wave) {
    __shared__ int red[16 * 64];
    __shared__ float par[64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int j = lane & 31;
    const int h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kwaves = blockDim.x >> 6;
    const int nt = blockIdx.x % n_tiles, bt = blockIdx.x / n_tiles;
    const int n0 = nt * 32, b0 = bt * 32;
    const int b = b0 + j;
    const int bl = min(b, p.B - 1);
    const int cw = p.cw;  // words per image / per neuron; a multiple of 4
    // The weights in lane order (after the [NPAD32][cw] rows): a group is 64 lanes x 4 words, contiguous; rows >= N
    // and words >= cw hold zeros (their outputs are discarded / they multiply activation words that read as 0).
    const int groups = (cw + 7) / 8;
    const v4i* __restrict__ wlane = reinterpret_cast<const v4i*>(wgt + fc_weight_row_words(n_tiles * 32, cw)) +
                                    (size_t)nt * groups * 64 + lane;

    // K order: group g = words 8g .. 8g+7; step 4g+i multiplies words 8g+i (lanes 0-31) and 8g+4+i
    // (lanes 32-63) of both operands.
    const int g_begin = wave * groups_per_wave, g_end = min(groups, g_begin + groups_per_wave);

    auto load_group = [&](int g, v4i& a, uint32_t (&bw)[4]) {
        const int w0 = 8 * g + 4 * h;
        a = wlane[(size_t)g * 64];  // (one contiguous 1 KB request per wave)
        if (w0 < cw) {  // cw % 4 == 0: the lane's four activation words exist or none does
#pragma unroll
            for (int i = 0; i < 4; ++i) bw[i] = act[(size_t)(w0 + i) * p.B + bl];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) bw[i] = 0;
        }
    };
    v16f acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    auto compute_group = [&](int g, const v4i& a, const uint32_t (&bw)[4]) {
        const int w0 = 8 * g + 4 * h;
        if (32 * (8 * g + 8) <= p.k_tap) {  // uniform: every bit of the group is a true input
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = Acc<FMT_F4>::mma(expand_f4((uint32_t)a[i]), expand_f4(bw[i]), acc);
        } else {  // K tail: pad bits (and words past cw) must multiply as 0, not as +1
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int nbits = p.k_tap - 32 * (w0 + i);
                const uint32_t valid = nbits >= 32 ? 0xffffffffu : (nbits <= 0 ? 0u : 0xffffffffu << (32 - nbits));
                acc = Acc<FMT_F4>::mma(expand_f4_masked((uint32_t)a[i], valid), expand_f4(bw[i]), acc);
            }
        }
    };

    // Epilogue parameters (thresholds, or scales and biases) of the tile's 32 neurons: one per lane, requested here,
    // ahead of the K loop, so that their round trip hides behind the operands'.  Neurons past N read the last valid
    // entry and are discarded.  Wave 0 passes them through LDS into the epilogue's layout (16 neurons per lane).
    const float my_thr = bnp[min(n0 + j, p.N - 1)];
    const float my_bias = MODE == FC_AFFINE ? bias[min(n0 + j, p.N - 1)] : 0.0f;

    if constexpr (PRE > 0) {
        // short slice: every operand word of the wave is requested before the first multiply (one round trip)
        v4i a[PRE];
        uint32_t bw[PRE][4];
#pragma unroll
        for (int u = 0; u < PRE; ++u)
            if (g_begin + u < g_end) load_group(g_begin + u, a[u], bw[u]);
#pragma unroll
        for (int u = 0; u < PRE; ++u)
            if (g_begin + u < g_end) compute_group(g_begin + u, a[u], bw[u]);
    } else {
        // two groups (8 k-steps) per stage, double-buffered in registers
        v4i a0[2], a1[2];
        uint32_t w0[2][4], w1[2][4];
        auto load_stage = [&](int g, v4i (&a)[2], uint32_t (&bw)[2][4]) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (g + u < g_end) load_group(g + u, a[u], bw[u]);
        };
        auto compute_stage = [&](int g, v4i (&a)[2], uint32_t (&bw)[2][4]) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (g + u < g_end) compute_group(g + u, a[u], bw[u]);
        };
        int g = g_begin;
        if (g < g_end) load_stage(g, a0, w0);
        while (g < g_end) {
            if (g + 2 < g_end) load_stage(g + 2, a1, w1);
            compute_stage(g, a0, w0);
            g += 2;
            if (g >= g_end) break;
            if (g + 2 < g_end) load_stage(g + 2, a0, w0);
            compute_stage(g, a1, w1);
            g += 2;
        }
    }

    // ---- sum the K slices of the waves (exact integers) in LDS
    int dot[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) dot[v] = (int)acc[v];
    if (wave == 0) {
        par[j] = my_thr;
        if constexpr (MODE == FC_AFFINE) par[32 + j] = my_bias;
    }
    if (kwaves > 1) {
        if (wave == 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) red[v * 64 + lane] = dot[v];
        }
        __syncthreads();
        if (wave != 0) {
#pragma unroll
            for (int v = 0; v < 16; ++v) atomicAdd(&red[v * 64 + lane], dot[v]);
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int v = 0; v < 16; ++v) dot[v] = red[v * 64 + lane];
    } else {
        __syncthreads();
    }

    // ---- epilogue (wave 0): the lane holds neurons cbase + v of image b
    const int cbase = n0 + 16 * h;
    float thr[16], bia[MODE == FC_AFFINE ? 16 : 1];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        thr[v] = par[16 * h + v];
        if constexpr (MODE == FC_AFFINE) bia[v] = par[32 + 16 * h + v];
    }
    if constexpr (MODE == FC_THRESH) {
        uint32_t hw = 0;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int c = cbase + v;
            const uint32_t bit = c < p.N ? thresh_bit(dot[v], thr[v], p.nan_bit) : 0u;
            hw = hw + hw + bit;
        }
        const uint32_t other = (uint32_t)__shfl_xor((int)hw, 32);
        if (h == 0 && b < p.B) {
            if (nt < p.bits_row_words) p.out_bits[(size_t)nt * p.B + b] = (hw << 16) | other;
            if (nt == n_tiles - 1)  // padding words of the 128-padded feature axis
                for (int w = n_tiles; w < p.bits_row_words; ++w) p.out_bits[(size_t)w * p.B + b] = 0;
        }
    } else {
        if (b < p.B) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int c = cbase + v;
                // the +-1 dot product equals (float)K - (float)popc*2.0f exactly (kernel.cuh:258-270)
                if (c < p.N) p.out_f32[(size_t)b * p.N + c] = __fadd_rn(__fmul_rn((float)dot[v], thr[v]), bia[v]);
            }
        }
    }
}

}  // namespace

bool fc_mfma_applicable(const BgemmParams& p) {
    // (a 1 x 1 convolution on a 1 x 1 frame has this shape too, but its filter buffer holds no copy in lane order)
    if (!p.wgt_lane_copy) return false;
    if (p.PH * p.PW != 1 || p.R * p.S != 1 || p.res_in != nullptr || p.res_out != nullptr) return false;
    if (p.mode != EPI_THRESH && p.mode != EPI_AFFINE) return false;
    if (p.cw % 4 != 0 || p.k_tap > 32 * p.cw) return false;
    // larger problems fill the machine with one wave per tile and are served by the generic kernel
    const long long tiles = (long long)((p.B + 31) / 32) * ((p.N + 31) / 32);
    return tiles <= 16384;
}

namespace {
// Split of K over the waves of a workgroup: waves per tile, 8-word groups per wave, and how many groups the
// kernel requests ahead of its first multiply (0: a streaming loop).
struct FcPlan {
    int n_tiles, b_tiles, kwaves, gpw, pre;
};
FcPlan fc_plan(const BgemmParams& p) {
    FcPlan f;
    f.n_tiles = (p.N + 31) / 32;
    f.b_tiles = (p.B + 31) / 32;
    const int groups = (p.cw + 7) / 8;
    // waves per tile: at least 4 groups (16 k-steps) each, no more than fill the machine a few times
    int kwaves = std::max(1, std::min(kMaxWaves, groups / 4));
    while (kwaves > 1 && (long long)f.n_tiles * f.b_tiles * kwaves > 8192) --kwaves;
    f.gpw = (groups + kwaves - 1) / kwaves;
    f.kwaves = (groups + f.gpw - 1) / f.gpw;
    f.pre = f.gpw <= 2 ? 2 : (f.gpw <= 7 ? 7 : 0);
    return f;
}
}  // namespace

void fc_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    snprintf(buf, len, "fc_mfma_f4_kernel<%d, %d>", p.mode == EPI_AFFINE ? FC_AFFINE : FC_THRESH, fc_plan(p).pre);
}

int launch_fc_mfma(const BgemmParams& p, hipStream_t stream) {
    const FcPlan f = fc_plan(p);
    const int n_tiles = f.n_tiles, b_tiles = f.b_tiles, kwaves = f.kwaves, gpw = f.gpw;
    const dim3 grid((unsigned)(n_tiles * b_tiles)), block(64 * kwaves);
    auto launch = [&](auto mode, auto pre) {
        constexpr int MODE = decltype(mode)::value, PRE = decltype(pre)::value;
        hipLaunchKernelGGL((fc_mfma_f4_kernel<MODE, PRE>), grid, block, 0, stream, p, p.act, p.wgt,
                           MODE == FC_AFFINE ? p.bn_scale : p.bn, MODE == FC_AFFINE ? p.bn_bias : p.bn, n_tiles, gpw);
    };
    auto by_slice = [&](auto mode) {
        if (f.pre == 2) launch(mode, std::integral_constant<int, 2>{});
        else if (f.pre == 7) launch(mode, std::integral_constant<int, 7>{});
        else launch(mode, std::integral_constant<int, 0>{});
    };
    if (p.mode == EPI_AFFINE) by_slice(std::integral_constant<int, FC_AFFINE>{});
    else by_slice(std::integral_constant<int, FC_THRESH>{});
    TCBNN_LAUNCH_CHECK("fc_mfma_f4_kernel");
    return TCBNN_OK;
}

}  // namespace tcbnn
