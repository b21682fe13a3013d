// Persistent FP4 matrix-core kernel for the 3x3 bit convolutions that carry almost all of a
// binarized ResNet / VGG (Conv128LayerFMT, kernel.cuh:676-827, pool 1x1, Cin = 64 .. 512).
//
// Same operand mapping as bgemm_mfma.hip (MFMA "A" = 32 output channels, "B" = 32 images, a lane
// of the accumulator owns one image and 16 channels), plus what a short-K convolution needs to
// keep the matrix cores fed on a machine whose memory latency (~1 us) is longer than the whole
// K loop of one tile (9 taps x Cin = 576..2304 bits: 36..144 MFMAs):
//   - persistent workgroups: the expanded FP4 weight fragments of a 64-channel group (18..72
//     KiB) and its thresholds are staged in LDS ONCE, then every wave walks a strided list of
//     (pixel, 64-image) tiles; no barrier after the staging;
//   - whole-chunk register prefetch: all activation words a wave needs for the next chunk of
//     taps (the whole tile for Cin <= 128, one filter row for Cin = 256, one tap for Cin = 512)
//     are requested while
//     the current chunk is multiplied, double-buffered across tile boundaries, so the loads of
//     tile i+1 fly under the MFMAs and the epilogue of tile i;
//   - wave-uniform border handling: a tap outside the frame is a cleared bit in a scalar mask
//     (its loads and MFMAs are skipped), which is exactly the reference's "exclude" rule;
//   - epilogue straight from the accumulator: fp32 compare against the threshold (the
//     accumulator is an exact integer), shift the bit into a 16-channel half-word, one lane^32
//     swap, 128-byte stores of the batch-innermost layouts; int32 residual add / save as
//     contiguous runs.
#include <algorithm>
#include <cmath>

#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

using namespace mfma;

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int NT = 2;  // 32-channel tiles per wave

// SPT = k-steps (64 bits) per filter tap = Cin / 64; MT = 32-image tiles per wave (2 for plain
// layers; 1 for residual layers, whose int32 traffic wants more waves per SIMD in flight)
template <int SPT, int MM, int MT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void
conv3x3_mfma_f4_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const int32_t* __restrict__ rin, int n_groups, int b_groups,
    int pix_streams) {
    constexpr int TPC = SPT == 8 ? 1 : (SPT == 4 ? 3 : 9);  // taps per prefetch chunk
    constexpr int NCH = 9 / TPC;           // chunks per tile
    constexpr int NQ = 9 * SPT;            // k-steps per tile
    extern __shared__ v4i lds_dyn[];
    v4i* lds_w = lds_dyn;  // [NQ][NT][64] fragments
    float* lds_thr = reinterpret_cast<float*>(lds_dyn + NQ * NT * 64);  // [NT*32]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int j = lane & 31;
    const int h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ng = blockIdx.x % n_groups;
    const int bg = (blockIdx.x / n_groups) % b_groups;
    const int stream = blockIdx.x / (n_groups * b_groups);
    const int n0 = ng * (32 * NT);
    const int kw_tot = 9 * p.cw;

    // ---- stage this channel group's weights (expanded, fragment order) and thresholds
    for (int f = wave; f < NQ * NT; f += kWaves) {
        const int q = f / NT, nt = f % NT;
        const int tap = q / SPT, t = q % SPT;
        const int c = n0 + nt * 32 + row_to_channel(j);
        uint32_t x = 0, valid = 0;
        if (c < p.N) {
            x = wgt[(size_t)c * kw_tot + tap * p.cw + 2 * t + h];
            valid = 0xffffffffu;
        }
        lds_w[f * 64 + lane] = expand_f4_masked(x, valid);
    }
    if (tid < NT * 32) lds_thr[tid] = n0 + tid < p.N ? bnp[n0 + tid] : 0.0f;
    __syncthreads();

    const int npix = p.PH * p.PW;
    int pi = stream * kWaves + wave;
    const int dpi = pix_streams * kWaves;
    int y = pi / p.PW, x = pi % p.PW;
    const int dy = dpi / p.PW, dx = dpi % p.PW;

    int bimg[MT], bload[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        bimg[mt] = (bg * MT + mt) * 32 + j;
        bload[mt] = min(bimg[mt], p.B - 1);
    }

    // Requests the activation words of chunk `chunk` of the tile at pixel (yy, xx); returns the
    // wave-uniform mask of its in-frame taps.
    auto load_chunk = [&](int yy, int xx, int chunk, uint32_t (*buf)[MT]) {
        uint32_t mask = 0;
#pragma unroll
        for (int tl = 0; tl < TPC; ++tl) {
            const int r = TPC == 9 ? tl / 3 : (TPC == 3 ? chunk : chunk / 3);
            const int s = TPC == 1 ? chunk % 3 : tl % 3;
            const int ay = yy * p.stride_h - p.pad_h + r, ax = xx * p.stride_w - p.pad_w + s;
            if (ay >= 0 && ay < p.H && ax >= 0 && ax < p.W) {
                mask |= 1u << tl;
                const uint32_t* src = act + ((size_t)(ay * p.W + ax) * p.cw + h) * p.B;
#pragma unroll
                for (int t = 0; t < SPT; ++t)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        buf[tl * SPT + t][mt] = src[(size_t)(2 * t) * p.B + bload[mt]];
            }
        }
        return mask;
    };

    v16f acc[MT][NT];
    auto zero_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[mt][nt][v] = 0.0f;
    };

    auto compute_chunk = [&](int chunk, uint32_t (*buf)[MT], uint32_t mask) {
#pragma unroll
        for (int tl = 0; tl < TPC; ++tl) {
            if (!((mask >> tl) & 1u)) continue;  // wave-uniform
            const int tap = chunk * TPC + tl;
#pragma unroll
            for (int t = 0; t < SPT; ++t) {
                v4i bfrag[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) bfrag[mt] = expand_f4(buf[tl * SPT + t][mt]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const v4i afrag = lds_w[((tap * SPT + t) * NT + nt) * 64 + lane];
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][nt] = Acc<FMT_F4>::mma(afrag, bfrag[mt], acc[mt][nt]);
                }
            }
        }
    };

    // Residual operand of the tile at pixel (yy, xx), requested before the tile's last chunk is
    // multiplied so that the loads fly under the MFMAs (kernel.cuh:770-794).
    int rv[MM == MM_THRESH_RES ? MT : 1][NT][16];
    auto load_residual = [&](int yy, int xx) {
        if constexpr (MM == MM_THRESH_RES) {
            const size_t pix = (size_t)yy * p.PW + xx;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int c = n0 + nt * 32 + 16 * h + v;
                        const int bb = bload[mt];
                        int val = 0;
                        if (rin != nullptr && c < p.res_limit && c < p.res_in_ch && c < p.N) {
                            if (p.res_pool) {
                                const size_t rw2 = 2 * (size_t)p.PW;
                                const int32_t* s00 =
                                    rin + (((size_t)(2 * yy) * rw2 + 2 * xx) * p.res_in_ch + c) * p.B + bb;
                                const size_t ddx = (size_t)p.res_in_ch * p.B, ddy = rw2 * ddx;
                                val = max(max(s00[0], s00[ddx]), max(s00[ddy], s00[ddy + ddx]));
                            } else {
                                val = rin[(pix * p.res_in_ch + c) * p.B + bb];
                            }
                        }
                        rv[mt][nt][v] = val;
                    }
        }
    };

    auto epilogue = [&](int yy, int xx) {
        const size_t pix = (size_t)yy * p.PW + xx;
        uint32_t* dst_bits = p.out_bits + pix * p.bits_pix_stride;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int cbase = n0 + nt * 32 + 16 * h;  // this lane's channels: cbase + v
            float thr[16];
            {
                const float4* t4 = reinterpret_cast<const float4*>(lds_thr + nt * 32 + 16 * h);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float4 tv = t4[k];
                    thr[4 * k + 0] = tv.x;
                    thr[4 * k + 1] = tv.y;
                    thr[4 * k + 2] = tv.z;
                    thr[4 * k + 3] = tv.w;
                }
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int b = bimg[mt];
                const bool b_ok = b < p.B;
                uint32_t hw = 0;
                if constexpr (MM == MM_THRESH_RES) {
                    int32_t* __restrict__ rout = p.res_out;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int c = cbase + v;
                        const int res = (int)acc[mt][nt][v] + rv[mt][nt][v];
                        if (rout != nullptr && b_ok && c < p.N) rout[(pix * p.N + c) * p.B + b] = res;
                        const uint32_t bit = (c < p.N && !((float)res < thr[v])) ? 1u : 0u;
                        hw = hw + hw + bit;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        // the accumulator is the exact integer sum: compare it directly
                        const uint32_t bit = (cbase + v < p.N && !(acc[mt][nt][v] < thr[v])) ? 1u : 0u;
                        hw = hw + hw + bit;
                    }
                }
                const uint32_t other = (uint32_t)__shfl_xor((int)hw, 32);
                const int w = ng * NT + nt;
                if (h == 0 && b_ok && w < p.bits_row_words) dst_bits[(size_t)w * p.B + b] = (hw << 16) | other;
            }
        }
        if (ng == n_groups - 1 && h == 0) {  // zero the pixel's padding words
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                if (bimg[mt] < p.B)
                    for (int w = max((p.N + 31) / 32, n_groups * NT); w < p.bits_row_words; ++w)
                        dst_bits[(size_t)w * p.B + bimg[mt]] = 0;
        }
    };

    // ---- persistent loop over this wave's tiles, chunks double-buffered in registers
    uint32_t buf0[TPC * SPT][MT], buf1[TPC * SPT][MT];
    uint32_t m0 = 0, m1 = 0;
    int chunk = 0;
    bool have = pi < npix;
    if (have) m0 = load_chunk(y, x, 0, buf0);
    zero_acc();

    auto step = [&](uint32_t (*cur)[MT], uint32_t mcur, uint32_t (*nxt)[MT], uint32_t& mnxt) {
        int nchunk = chunk + 1, ny = y, nx = x, npi = pi;
        if (nchunk == NCH) {
            nchunk = 0;
            npi = pi + dpi;
            nx = x + dx;
            ny = y + dy;
            if (nx >= p.PW) {
                nx -= p.PW;
                ++ny;
            }
        }
        const bool nhave = npi < npix;
        if (nhave) mnxt = load_chunk(ny, nx, nchunk, nxt);
        if (chunk == NCH - 1) load_residual(y, x);
        compute_chunk(chunk, cur, mcur);
        if (chunk == NCH - 1) {
            epilogue(y, x);
            zero_acc();
        }
        chunk = nchunk;
        y = ny;
        x = nx;
        pi = npi;
        have = nhave;
    };

    while (have) {
        step(buf0, m0, buf1, m1);
        if (!have) break;
        step(buf1, m1, buf0, m0);
    }
}

template <int SPT, int MM, int MT>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    constexpr int NQ = 9 * SPT;
    const size_t lds_bytes = (size_t)NQ * NT * 64 * 16 + NT * 32 * sizeof(float);
    static bool attr_set = false;  // per instantiation
    if (!attr_set) {
        if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv3x3_mfma_f4_kernel<SPT, MM, MT>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes),
                               "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"))
            return rc;
        attr_set = true;
    }
    const int n_groups = (p.N + 32 * NT - 1) / (32 * NT);
    const int b_groups = (p.B + 32 * MT - 1) / (32 * MT);
    const int quads = (p.PH * p.PW + kWaves - 1) / kWaves;  // pixel quads (one pixel per wave)
    // about two (plain) or three (residual) workgroups per CU, with the pixel quads spread as
    // evenly as possible
    const int target = std::max(1, (MT == 1 ? 768 : 512) / (n_groups * b_groups));
    int best = std::min(target, quads);
    double best_waste = 1e30;
    for (int ps = std::max(1, target / 2); ps <= std::min(quads, target * 2); ++ps) {
        const int per = (quads + ps - 1) / ps;
        const double waste = (double)per * ps / quads + 0.02 * std::abs(ps - target) / (double)target;
        if (waste < best_waste) {
            best_waste = waste;
            best = ps;
        }
    }
    const long long blocks = (long long)best * n_groups * b_groups;
    hipLaunchKernelGGL((conv3x3_mfma_f4_kernel<SPT, MM, MT>), dim3((unsigned)blocks), dim3(kThreads), lds_bytes,
                       stream, p, p.act, p.wgt, p.bn, p.res_in, n_groups, b_groups, best);
    TCBNN_LAUNCH_CHECK("conv3x3_mfma_f4_kernel");
    return TCBNN_OK;
}

template <int SPT>
int launch_m(const BgemmParams& p, hipStream_t stream) {
    if (p.res_in != nullptr || p.res_out != nullptr) return launch_t<SPT, MM_THRESH_RES, 1>(p, stream);
    return launch_t<SPT, MM_THRESH, 2>(p, stream);
}

}  // namespace

bool conv3x3_mfma_applicable(const BgemmParams& p) {
    return p.R == 3 && p.S == 3 && p.pool_h == 1 && p.pool_w == 1 && p.mode == EPI_THRESH && p.nan_bit == 1 &&
           p.ksplit <= 1 && (p.cw == 2 || p.cw == 4 || p.cw == 8 || p.cw == 16) && p.k_tap == 32 * p.cw &&
           (long long)p.PH * p.PW < (1 << 24);
}

void conv3x3_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    const bool res = p.res_in != nullptr || p.res_out != nullptr;
    snprintf(buf, len, "conv3x3_mfma_f4_kernel<%d, %d, %d>", p.cw / 2, res ? MM_THRESH_RES : MM_THRESH,
             res ? 1 : 2);
}

int launch_conv3x3_mfma(const BgemmParams& p, hipStream_t stream) {
    switch (p.cw) {
        case 2:
            return launch_m<1>(p, stream);
        case 4:
            return launch_m<2>(p, stream);
        case 8:
            return launch_m<4>(p, stream);
        default:
            return launch_m<8>(p, stream);
    }
}

}  // namespace tcbnn
