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

// Residual mode of an instantiation.
constexpr int RM_NONE = 0;    // threshold only
constexpr int RM_PLAIN = 1;   // residual injected from a source of the same size and / or saved
constexpr int RM_POOLED = 2;  // residual injected as the 2x2 max of a source twice the size

// Waves per SIMD the register allocator is asked to make room for: the residual layers are
// bound by HBM and want more memory requests in flight, the plain layers want registers.
constexpr int waves_hint(int spt, int rm, int nt) { return rm == RM_PLAIN && spt * nt <= 2 ? 3 : 2; }

// SPT = k-steps (64 bits) per filter tap = Cin / 64; MT = 32-image tiles per wave (2 for plain
// layers, 1 for residual layers); NT = 32-channel tiles per wave.
template <int SPT, int RM, int MT, int NT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(waves_hint(SPT, RM, NT)))) void
conv3x3_mfma_f4_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const int32_t* __restrict__ rin, int32_t* __restrict__ rout, int res_lim,
    int rin_fmt, int rout_fmt, int n_groups, int b_groups, int pix_streams) {
    static_assert(RM == RM_NONE || MT == 1, "residual instantiations own one image tile per wave");
    constexpr int TPC = SPT >= 4 ? 3 : 9;  // taps per prefetch chunk (a filter row, or all of it)
    constexpr int NCH = 9 / TPC;           // chunks per tile
    constexpr int NQ = 9 * SPT;            // k-steps per tile
    // A tile of one chunk is shorter than the memory latency: its residual operand is then
    // requested a whole tile ahead (double-buffered); otherwise with the tile's first chunk.
    constexpr bool kAhead = RM != RM_NONE && NCH == 1;
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

    // ---- residual operand (kernel.cuh:770-794).  A lane owns channels n0 + 32 nt + 16 h + v of
    // image bload[0]; every load is a wave-uniform base plus this per-lane element offset.
    // TCBNN_RES_I16 tensors hold two channels per word: 8 loads per channel tile instead of 16,
    // unpacked (and, for a pooled source, reduced) by finish_residual.
    constexpr int NRV = RM != RM_NONE ? NT : 1;
    constexpr int NTMP = RM == RM_POOLED ? 3 : 1;
    int tmp[NTMP][NRV][16];  // pooled: the other three pixels of the 2x2 window
    const unsigned lane_off = (unsigned)(16 * h) * (unsigned)p.B + (unsigned)bload[0];
    const unsigned lane_off16 = (unsigned)(8 * h) * (unsigned)p.B + (unsigned)bload[0];

    auto request_residual = [&](int yy, int xx, int (*rv)[16]) {
        if constexpr (RM != RM_NONE) {
            const bool i16 = rin_fmt == TCBNN_RES_I16;  // wave-uniform
            // words per source pixel, words between channel rows of a lane, lane offset
            const size_t ch_b = (size_t)(i16 ? (p.res_in_ch + 1) / 2 : p.res_in_ch) * p.B;
            const unsigned loff = i16 ? lane_off16 : lane_off;
            const int nld = i16 ? 8 : 16;
            const size_t pix = RM == RM_POOLED ? ((size_t)(2 * yy) * (2 * p.PW) + 2 * xx) : ((size_t)yy * p.PW + xx);
            const size_t ddy = (size_t)(2 * p.PW) * ch_b;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int cb = n0 + nt * 32;
                const int32_t* __restrict__ base = rin + pix * ch_b + (size_t)(i16 ? cb / 2 : cb) * p.B;  // uniform
                if (cb + 32 <= res_lim) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        if (v >= nld) continue;  // uniform
                        const int32_t* s = base + (size_t)v * p.B;
                        rv[nt][v] = s[loff];
                        if constexpr (RM == RM_POOLED) {
                            tmp[0][nt][v] = s[ch_b + loff];
                            tmp[1][nt][v] = s[ddy + loff];
                            tmp[2][nt][v] = s[ddy + ch_b + loff];
                        }
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        if (v >= nld) continue;  // uniform
                        const bool ok = cb + 16 * h + (i16 ? 2 * v : v) < res_lim;
                        const int32_t* s = base + (size_t)v * p.B;
                        rv[nt][v] = ok ? s[loff] : 0;
                        if constexpr (RM == RM_POOLED) {
                            tmp[0][nt][v] = ok ? s[ch_b + loff] : 0;
                            tmp[1][nt][v] = ok ? s[ddy + loff] : 0;
                            tmp[2][nt][v] = ok ? s[ddy + ch_b + loff] : 0;
                        }
                    }
                }
            }
        }
    };
    // Turns what request_residual loaded into one int per channel: unpack 16-bit pairs, take the
    // 2x2 maximum of a pooled source, clear channels that receive no residual.
    auto finish_residual = [&](int (*rv)[16]) {
        if constexpr (RM != RM_NONE) {
            if (rin_fmt == TCBNN_RES_I16) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int cb = n0 + nt * 32;
#pragma unroll
                    for (int k = 7; k >= 0; --k) {  // downwards: slot k is read before 2k, 2k+1 are written
                        const int w = rv[nt][k];
                        int lo = (int)(short)(w & 0xffff), hi = w >> 16;
                        if constexpr (RM == RM_POOLED) {
#pragma unroll
                            for (int t = 0; t < 3; ++t) {
                                const int wt = tmp[t][nt][k];
                                lo = max(lo, (int)(short)(wt & 0xffff));
                                hi = max(hi, wt >> 16);
                            }
                        }
                        if (cb + 32 > res_lim) {  // uniform: partial channel tile
                            if (cb + 16 * h + 2 * k >= res_lim) lo = 0;
                            if (cb + 16 * h + 2 * k + 1 >= res_lim) hi = 0;
                        }
                        rv[nt][2 * k] = lo;
                        rv[nt][2 * k + 1] = hi;
                    }
                }
            } else if constexpr (RM == RM_POOLED) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        rv[nt][v] = max(max(rv[nt][v], tmp[0][nt][v]), max(tmp[1][nt][v], tmp[2][nt][v]));
            }
        }
    };

    auto epilogue = [&](int yy, int xx, int (*rv)[16]) {
        const size_t pix = (size_t)yy * p.PW + xx;
        uint32_t* dst_bits = p.out_bits + pix * p.bits_pix_stride;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int cbase = n0 + nt * 32 + 16 * h;  // this lane's channels: cbase + v
            const bool n_full = n0 + nt * 32 + 32 <= p.N;  // wave-uniform
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
                if constexpr (RM != RM_NONE) {
                    int res[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) res[v] = (int)acc[mt][nt][v] + rv[nt][v];
                    if (rout != nullptr && b_ok) {
                        if (rout_fmt == TCBNN_RES_I16) {  // two channels per word
                            int32_t* __restrict__ dst =
                                rout + (pix * ((p.N + 1) / 2) + (n0 + nt * 32) / 2) * p.B;  // wave-uniform
                            const unsigned off = (unsigned)(8 * h) * (unsigned)p.B + (unsigned)b;
#pragma unroll
                            for (int k = 0; k < 8; ++k) {
                                const int c0 = cbase + 2 * k;
                                const int hi = (n_full || c0 + 1 < p.N) ? res[2 * k + 1] : 0;
                                if (n_full || c0 < p.N) (dst + (size_t)k * p.B)[off] = (res[2 * k] & 0xffff) | (hi << 16);
                            }
                        } else {
                            int32_t* __restrict__ dst = rout + (pix * p.N + n0 + nt * 32) * p.B;  // wave-uniform
                            const unsigned off = (unsigned)(16 * h) * (unsigned)p.B + (unsigned)b;
                            if (n_full) {
#pragma unroll
                                for (int v = 0; v < 16; ++v) (dst + (size_t)v * p.B)[off] = res[v];
                            } else {
#pragma unroll
                                for (int v = 0; v < 16; ++v)
                                    if (cbase + v < p.N) (dst + (size_t)v * p.B)[off] = res[v];
                            }
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const uint32_t bit = ((n_full || cbase + v < p.N) && !((float)res[v] < thr[v])) ? 1u : 0u;
                        hw = hw + hw + bit;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        // the accumulator is the exact integer sum: compare it directly
                        const uint32_t bit =
                            ((n_full || cbase + v < p.N) && !(acc[mt][nt][v] < thr[v])) ? 1u : 0u;
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
    int rv0[NRV][16], rv1[kAhead ? NRV : 1][kAhead ? 16 : 1];
    uint32_t m0 = 0, m1 = 0;
    int chunk = 0;
    bool have = pi < npix;
    if (have) {
        m0 = load_chunk(y, x, 0, buf0);
        if constexpr (kAhead) {
            request_residual(y, x, rv0);
            if constexpr (RM == RM_POOLED) finish_residual(rv0);
        }
    }
    zero_acc();

    auto step = [&](uint32_t (*cur)[MT], uint32_t mcur, uint32_t (*nxt)[MT], uint32_t& mnxt, int (*rcur)[16],
                    int (*rnxt)[16]) {
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
        if constexpr (kAhead) {
            if (nhave) request_residual(ny, nx, rnxt);
        } else if constexpr (RM != RM_NONE) {
            if (chunk == 0) request_residual(y, x, rcur);
        }
        compute_chunk(chunk, cur, mcur);
        // a pooled source is reduced as soon as its tile has been multiplied (frees the registers of the
        // window); otherwise the operand is left in flight until its own epilogue
        if constexpr (kAhead && RM == RM_POOLED) {
            if (nhave) finish_residual(rnxt);
        }
        if (chunk == NCH - 1) {
            if constexpr (!(kAhead && RM == RM_POOLED)) finish_residual(rcur);
            epilogue(y, x, rcur);
            zero_acc();
        }
        chunk = nchunk;
        y = ny;
        x = nx;
        pi = npi;
        have = nhave;
    };

    while (have) {
        if constexpr (kAhead) {
            step(buf0, m0, buf1, m1, rv0, rv1);
            if (!have) break;
            step(buf1, m1, buf0, m0, rv1, rv0);
        } else {
            step(buf0, m0, buf1, m1, rv0, rv0);
            if (!have) break;
            step(buf1, m1, buf0, m0, rv0, rv0);
        }
    }
}

template <int SPT, int RM, int MT, int NT>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    constexpr int NQ = 9 * SPT;
    const size_t lds_bytes = (size_t)NQ * NT * 64 * 16 + NT * 32 * sizeof(float);
    static bool attr_set = false;  // per instantiation
    if (!attr_set) {
        if (int rc = check_hip(
                hipFuncSetAttribute(reinterpret_cast<const void*>(&conv3x3_mfma_f4_kernel<SPT, RM, MT, NT>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes),
                "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"))
            return rc;
        attr_set = true;
    }
    const int n_groups = (p.N + 32 * NT - 1) / (32 * NT);
    const int b_groups = (p.B + 32 * MT - 1) / (32 * MT);
    const int quads = (p.PH * p.PW + kWaves - 1) / kWaves;  // pixel quads (one pixel per wave)
    // as many workgroups as are resident at once (two per CU for plain layers, three for residual
    // layers, fewer when their LDS does not fit), so that the weights are staged once per CU
    // slot, with the pixel quads spread as evenly as possible
    const int wg_per_cu = std::max(1, std::min(MT == 1 ? 3 : 2, (int)(160 * 1024 / lds_bytes)));
    const int target = std::max(1, 256 * wg_per_cu / (n_groups * b_groups));
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
    // channels that receive an injected residual: o < residual_channels, and only those the
    // source tensor holds (kernel.cuh:770)
    const int res_lim = p.res_in != nullptr ? std::min(std::min(p.res_limit, p.res_in_ch), p.N) : 0;
    const long long blocks = (long long)best * n_groups * b_groups;
    hipLaunchKernelGGL((conv3x3_mfma_f4_kernel<SPT, RM, MT, NT>), dim3((unsigned)blocks), dim3(kThreads), lds_bytes,
                       stream, p, p.act, p.wgt, p.bn, p.res_in, p.res_out, res_lim, p.res_in_fmt, p.res_out_fmt, n_groups,
                       b_groups, best);
    TCBNN_LAUNCH_CHECK("conv3x3_mfma_f4_kernel");
    return TCBNN_OK;
}

// Which instantiation serves a layer.  Measured on ResNet-18 at batch 256: the HBM-bound residual
// layers run best with one image tile per wave and, from Cin = 256 on, one channel tile (more
// workgroups fit a CU's LDS, so more residual requests are in flight); plain layers want the 2 x 2
// tile (each operand fragment feeds two MFMAs) until the weights of 64 channels no longer leave
// room for a second workgroup (Cin = 512).
struct Pick {
    int rm, mt, nt;
};
constexpr int pick_nt(int spt, int rm) {
    return rm == RM_POOLED ? 1 : (rm == RM_PLAIN ? (spt >= 4 ? 1 : 2) : (spt >= 8 ? 1 : 2));
}
Pick pick(const BgemmParams& p) {
    const int rm = p.res_in == nullptr && p.res_out == nullptr ? RM_NONE
                                                                : (p.res_in != nullptr && p.res_pool ? RM_POOLED : RM_PLAIN);
    return {rm, rm == RM_NONE ? 2 : 1, pick_nt(p.cw / 2, rm)};
}

template <int SPT>
int launch_m(const BgemmParams& p, hipStream_t stream) {
    switch (pick(p).rm) {
        case RM_NONE:
            return launch_t<SPT, RM_NONE, 2, pick_nt(SPT, RM_NONE)>(p, stream);
        case RM_PLAIN:
            return launch_t<SPT, RM_PLAIN, 1, pick_nt(SPT, RM_PLAIN)>(p, stream);
        default:
            return launch_t<SPT, RM_POOLED, 1, pick_nt(SPT, RM_POOLED)>(p, stream);
    }
}

}  // namespace

bool conv3x3_mfma_applicable(const BgemmParams& p) {
    return p.R == 3 && p.S == 3 && p.pool_h == 1 && p.pool_w == 1 && p.mode == EPI_THRESH && p.nan_bit == 1 &&
           p.ksplit <= 1 && (p.cw == 2 || p.cw == 4 || p.cw == 8 || p.cw == 16) && p.k_tap == 32 * p.cw &&
           (long long)p.PH * p.PW < (1 << 24);
}

void conv3x3_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    const Pick k = pick(p);
    snprintf(buf, len, "conv3x3_mfma_f4_kernel<%d, %d, %d, %d>", p.cw / 2, k.rm, k.mt, k.nt);
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
