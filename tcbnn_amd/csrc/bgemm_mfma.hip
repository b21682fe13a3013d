// Matrix-core variants of the bit implicit GEMM for gfx950.
//
// CDNA4 has no 1-bit MFMA, so the packed +-1 operands are expanded on the fly to the
// narrowest type the matrix cores multiply exactly:
//   FMT_F4: FP4 E2M1 nibbles (+1.0 = 0x2, -1.0 = 0xA, 0 = 0x0), v_mfma_f32_32x32x64_f8f6f4.
//           Products are exactly +-1 or 0 and every partial sum is an integer below 2^24,
//           so the fp32 accumulator is exact whatever the internal summation order.
//   FMT_I8: int8 bytes (+1 = 0x01, -1 = 0xFF, 0), v_mfma_i32_32x32x32_i8, int32 accumulate.
// A 32-bit word of packed bits becomes 4 dwords of FP4 with 7 VALU ops (shift, and-or),
// which is amortised over the 32*NT output channels the wave multiplies it with.
//
// Operand roles are transposed with respect to the usual GEMM: the MFMA "A" operand holds
// 32 output channels (weights), the "B" operand 32 images, so in the accumulator a lane owns
// ONE image and 16 channels.  With the batch-innermost layouts this gives
//   - activation loads: lane (image j, k-half h) reads word 2t+h of its image: two contiguous
//     128-byte runs per wave load;
//   - epilogue: threshold -> bit -> shift/or builds a 16-channel half-word in the lane, one
//     cross-lane swap (lane ^ 32) completes the 32-channel word, 128-byte contiguous stores;
//     residual loads/stores are contiguous runs as well; no atomics, pool windows are a
//     sequential loop (OR), every output word is written exactly once.
// The weight rows of a channel tile are permuted when they are staged so that accumulator
// register v of lane half h is channel 16h+v.  Weights are expanded once per workgroup into
// LDS in MFMA-fragment order ([k-step][channel tile][lane] x 16 bytes, conflict-free
// ds_read_b128); pad bits and out-of-range channels are staged as zeros, so the true K / Cin
// enters the result without any correction term, and zero padding of the convolution is
// simply a skipped tap (kernel.cuh:752-768 "exclude").
//
// Semantics: Fc128LayerFMT / Out128LayerFMT / Conv128LayerFMT (kernel.cuh:174-280, 676-827),
// BMMAS / BTC_Conv2d_balance (tensorcore_kernel.cu:305-356, bmma_kernel.cu:101-165).
#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

using namespace mfma;

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int kNT = 2;    // 32-channel tiles per wave
constexpr int kQB = 24;   // k-steps of weights staged in LDS at a time (24 * kNT KiB); a multiple of 4

// Without an occupancy target the compiler schedules the unrolled epilogue across up to 512 registers (one wave
// per SIMD); most launches of this kernel are many short workgroups, which need several resident at a time.
template <int FMT, int MT, int MM>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(MT == 4 || MM == MM_THRESH_RES ? 2 : 3))) void bgemm_mfma_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const int32_t* __restrict__ rin, int n_groups, int row_waves,
    int b_groups, int row_blocks) {
    using A = Acc<FMT>;
    using acc_t = typename A::type;
    __shared__ v4i lds_w[kQB * kNT * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int j = lane & 31;   // image within a 32-image tile
    const int h = lane >> 5;   // k half (operands) / channel half (accumulator)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ng = blockIdx.x % n_groups;
    const int rb = (blockIdx.x / n_groups) % row_blocks;
    const int ks = blockIdx.x / (n_groups * row_blocks);
    const int rw = rb * kWaves + wave;
    const bool active = rw < row_waves;
    const int n0 = ng * (32 * kNT);

    const int taps = p.R * p.S;
    const int kw_tot = taps * p.cw;
    const int steps = FMT == FMT_F4 ? (p.cw + 1) / 2 : p.cw;  // k-steps per tap
    const int nq_all = taps * steps;
    const int q_per = (nq_all + p.ksplit - 1) / p.ksplit;
    const int q_begin = ks * q_per;
    const int q_end = min(nq_all, q_begin + q_per);
    const bool single_block = q_end - q_begin <= kQB;

    const int opix = active ? rw / b_groups : 0;
    const int bg = active ? rw % b_groups : 0;
    const int oy = opix / p.OW, ox = opix % p.OW;

    int bimg[MT], bload[MT], voff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        bimg[mt] = (bg * MT + mt) * 32 + j;
        bload[mt] = min(bimg[mt], p.B - 1);
        voff[mt] = ((FMT == FMT_F4 ? h * p.B : 0) + bload[mt]) * 4;  // byte offset inside a pixel's [cw][B] words
    }

    // stage k-steps [q0, q0+cnt) of this channel group, expanded, in fragment order
    auto stage_weights = [&](int q0) {
        const int cnt = min(kQB, q_end - q0);
        for (int f = wave; f < cnt * kNT; f += kWaves) {
            const int ql = f / kNT, nt = f % kNT;
            const int q = q0 + ql;
            const int tap = q / steps, t = q % steps;
            const int c = n0 + nt * 32 + row_to_channel(j);
            const int word = FMT == FMT_F4 ? 2 * t + h : t;  // word of the tap this lane expands
            uint32_t x = 0, valid = 0;
            if (word < p.cw && c < p.N) {
                x = wgt[(size_t)c * kw_tot + tap * p.cw + word];
                const int nbits = p.k_tap - 32 * word;  // true bits in this word
                valid = nbits >= 32 ? 0xffffffffu : (nbits <= 0 ? 0u : 0xffffffffu << (32 - nbits));
            }
            lds_w[(ql * kNT + nt) * 64 + lane] =
                FMT == FMT_F4 ? expand_f4_masked(x, valid) : expand_i8_masked(x, valid, h);
        }
    };

    if (single_block && q_end > q_begin) {
        stage_weights(q_begin);
        __syncthreads();
    }

    uint32_t outword[MT][kNT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) outword[mt][nt] = 0;

    const int pool_n = p.pool_h * p.pool_w;
    for (int pp = 0; pp < pool_n; ++pp) {
        const int y = oy * p.pool_h + pp / p.pool_w;
        const int x = ox * p.pool_w + pp % p.pool_w;
        // Every pixel of the pool window is computed, also those past the convolution's own output when the
        // pooled size is rounded up (kernel.cuh:685-690 walks pool * output rows and columns): such a pixel sums
        // the taps that still lie inside the frame, none at all in the limit (sum 0), and its bit is ORed in.
        const bool valid = active;  // wave-uniform
        const int ay0 = y * p.stride_h - p.pad_h;
        const int ax0 = x * p.stride_w - p.pad_w;

        acc_t acc[MT][kNT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[mt][nt][v] = 0;

        // Activation words this lane needs for k-step (tap row tr, tap col ts, step t).  The words of one input
        // pixel ([cw][B]) are addressed as a buffer: the pixel and the step are wave-uniform (descriptor base and
        // scalar offset, computed on the scalar unit), the lane contributes one constant offset per image tile,
        // so a step costs no vector address arithmetic (it was ~45 of the ~75 VALU instructions per step).  With
        // an odd cw the upper half-wave's word of the last step lies past the pixel's range and reads 0; the
        // weight side of a pad word is 0 anyway.
        auto load_step = [&](int tr, int ts, int t, uint32_t* dst) {
            const int ay = ay0 + tr, ax = ax0 + ts;
            const bool in_frame = valid && ay >= 0 && ay < p.H && ax >= 0 && ax < p.W;
            if (in_frame) {
                const uint32_t* pixel = act + (size_t)(ay * p.W + ax) * p.cw * p.B;
                const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<uint32_t*>(pixel), 0, p.cw * p.B * 4, 0x00020000);
                const int soff = (FMT == FMT_F4 ? 2 * t : t) * p.B * 4;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    dst[mt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, voff[mt], soff, 0);
            }
            return in_frame;
        };

        if constexpr (MM == MM_OTHER) {
            // Activation words are requested kAhead k-steps before they are multiplied, through a ring of kAhead
            // register slots (slot d is asked for step q + kAhead as soon as step q has been expanded from it): one
            // step of 2-8 MFMAs is far shorter than a memory round trip, and with a prefetch distance of one step every
            // step waited for it.
            constexpr int kAhead = 4;  // divides kQB
            int ltr = (q_begin / steps) / p.S, lts = (q_begin / steps) % p.S, lt = q_begin % steps;  // next step to request
            int lq = q_begin;
            uint32_t ring[kAhead][MT];
            bool ring_ok[kAhead];
            auto request = [&](uint32_t* dst) {
                bool ok = false;
                if (lq < q_end) {
                    ok = load_step(ltr, lts, lt, dst);
                    ++lq;
                    if (++lt == steps) {
                        lt = 0;
                        if (++lts == p.S) {
                            lts = 0;
                            ++ltr;
                        }
                    }
                }
                return ok;
            };
#pragma unroll
            for (int d = 0; d < kAhead; ++d) ring_ok[d] = request(ring[d]);
            for (int q0 = q_begin; q0 < q_end; q0 += kQB) {
                if (!single_block) {
                    __syncthreads();
                    stage_weights(q0);
                    __syncthreads();
                }
                const int cnt = min(kQB, q_end - q0);  // a multiple of kAhead except in the last block
                for (int ql = 0; ql < cnt; ql += kAhead) {
#pragma unroll
                    for (int d = 0; d < kAhead; ++d) {
                        if (ql + d >= cnt) break;  // past the last step: nothing was requested into these slots
                        v4i bfrag[MT];
                        const bool ok = ring_ok[d];
                        if (ok) {
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt)
                                bfrag[mt] = FMT == FMT_F4 ? expand_f4(ring[d][mt]) : expand_i8(ring[d][mt], h);
                        }
                        ring_ok[d] = request(ring[d]);
                        if (ok) {
#pragma unroll
                            for (int nt = 0; nt < kNT; ++nt) {
                                const v4i afrag = lds_w[((ql + d) * kNT + nt) * 64 + lane];
#pragma unroll
                                for (int mt = 0; mt < MT; ++mt)
                                    acc[mt][nt] = A::mma(afrag, bfrag[mt], acc[mt][nt]);
                            }
                        }
                    }
                }
            }
        } else {
            // one step ahead: the threshold epilogues leave no registers for a ring (it spilled and was slower)
            int tr = (q_begin / steps) / p.S, ts = (q_begin / steps) % p.S, t = q_begin % steps;
            uint32_t cur[MT], nxt[MT];
            bool cur_ok = q_begin < q_end ? load_step(tr, ts, t, cur) : false;
            for (int q0 = q_begin; q0 < q_end; q0 += kQB) {
                if (!single_block) {
                    __syncthreads();
                    stage_weights(q0);
                    __syncthreads();
                }
                const int cnt = min(kQB, q_end - q0);
                for (int ql = 0; ql < cnt; ++ql) {
                    // advance the (tap, step) counters and prefetch the next step's words
                    int ntr = tr, nts = ts, nt_ = t + 1;
                    if (nt_ == steps) {
                        nt_ = 0;
                        if (++nts == p.S) {
                            nts = 0;
                            ++ntr;
                        }
                    }
                    const bool nxt_ok = (q0 + ql + 1 < q_end) ? load_step(ntr, nts, nt_, nxt) : false;
                    if (cur_ok) {
                        v4i bfrag[MT];
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            bfrag[mt] = FMT == FMT_F4 ? expand_f4(cur[mt]) : expand_i8(cur[mt], h);
#pragma unroll
                        for (int nt = 0; nt < kNT; ++nt) {
                            const v4i afrag = lds_w[(ql * kNT + nt) * 64 + lane];
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt)
                                acc[mt][nt] = A::mma(afrag, bfrag[mt], acc[mt][nt]);
                        }
                    }
                    tr = ntr;
                    ts = nts;
                    t = nt_;
                    cur_ok = nxt_ok;
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) cur[mt] = nxt[mt];
                }
            }
        }

        if (!valid) continue;

        // ---------------- epilogue for pre-pool pixel (y, x) ----------------
        const size_t pix = (size_t)y * p.PW + x;
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) {
            const int cbase = n0 + nt * 32 + 16 * h;  // this lane's channels: cbase + v
            // the lane's 16 thresholds, requested together and shared by its image tiles (a load per use, each
            // under its own bounds test, was a chain of 16 * MT * kNT memory round trips)
            float thr[16];
            if constexpr (MM == MM_THRESH || MM == MM_THRESH_RES) {
#pragma unroll
                for (int v = 0; v < 16; ++v) thr[v] = bnp[min(cbase + v, p.N - 1)];
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int b = bimg[mt];
                const bool b_ok = b < p.B;
                const int bb = bload[mt];
                if constexpr (MM == MM_THRESH || MM == MM_THRESH_RES) {
                    int rv[16];
                    if constexpr (MM == MM_THRESH_RES) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) rv[v] = 0;
                        if (rin != nullptr && cbase < p.res_in_ch) {  // wave-uniform but for the channel half
                            // the lane's 16 channels are whole 16-byte groups of the source: 128-bit loads
                            const bool r16 = p.res_in_fmt == TCBNN_RES_I16;
                            const size_t ngrp = r16 ? (p.res_in_ch + 7) / 8 : (p.res_in_ch + 3) / 4;
                            const int4* __restrict__ src = reinterpret_cast<const int4*>(rin);
                            auto fetch = [&](size_t sp, int* dst) {
                                if (p.res_in_fmt == TCBNN_RES_I12) {  // the lane's 16 channels are one 12-bit group
                                    residual_load_group16(rin, TCBNN_RES_I12, sp, p.res_in_ch, cbase / 16, p.B, bb, dst);
                                } else if (r16) {
                                    const size_t g0 = (sp * ngrp + cbase / 8) * p.B + bb;
#pragma unroll
                                    for (int g = 0; g < 2; ++g) {
                                        int4 q = make_int4(0, 0, 0, 0);
                                        if (cbase + 8 * g < p.res_in_ch) q = src[g0 + (size_t)g * p.B];
                                        const int w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                                        for (int e = 0; e < 4; ++e) {
                                            dst[8 * g + 2 * e] = (w[e] << 16) >> 16;
                                            dst[8 * g + 2 * e + 1] = w[e] >> 16;
                                        }
                                    }
                                } else {
                                    const size_t g0 = (sp * ngrp + cbase / 4) * p.B + bb;
#pragma unroll
                                    for (int g = 0; g < 4; ++g) {
                                        int4 q = make_int4(0, 0, 0, 0);
                                        if (cbase + 4 * g < p.res_in_ch) q = src[g0 + (size_t)g * p.B];
                                        dst[4 * g] = q.x;
                                        dst[4 * g + 1] = q.y;
                                        dst[4 * g + 2] = q.z;
                                        dst[4 * g + 3] = q.w;
                                    }
                                }
                            };
                            if (p.res_pool) {
                                const size_t rw2 = 2 * (size_t)p.PW, p00 = (size_t)(2 * y) * rw2 + 2 * x;
                                fetch(p00, rv);
                                const size_t others[3] = {p00 + 1, p00 + rw2, p00 + rw2 + 1};
                                for (int k = 0; k < 3; ++k) {
                                    int t[16];
                                    fetch(others[k], t);
#pragma unroll
                                    for (int v = 0; v < 16; ++v) rv[v] = max(rv[v], t[v]);
                                }
                            } else {
                                fetch(pix, rv);
                            }
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                const int c = cbase + v;
                                if (!(c < p.res_limit && c < p.res_in_ch && c < p.N)) rv[v] = 0;
                            }
                        }
                    }
                    int32_t* __restrict__ rout = p.res_out;
                    uint32_t hw = 0;
                    int resv[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int c = cbase + v;
                        int res = A::to_int(acc[mt][nt][v]);
                        uint32_t bit = 0;
                        if (c < p.N) {
                            if constexpr (MM == MM_THRESH_RES) res += rv[v];
                            bit = thresh_bit(res, thr[v], p.nan_bit);
                        }
                        resv[v] = c < p.N ? res : 0;  // channels past N are stored as 0 inside a group
                        hw = (hw << 1) | bit;
                    }
                    if constexpr (MM == MM_THRESH_RES) {
                        // a lane's 16 channels are whole 16-byte groups of the residual layouts: 128-bit stores
                        if (rout != nullptr && b_ok && cbase < p.N) {
                            int4* __restrict__ dst = reinterpret_cast<int4*>(rout);
                            if (p.res_out_fmt == TCBNN_RES_I12) {
                                residual_store_group16(rout, TCBNN_RES_I12, pix, p.N, cbase / 16, p.B, b, resv);
                            } else if (p.res_out_fmt == TCBNN_RES_I16) {
                                const size_t g0 = (pix * (size_t)((p.N + 7) / 8) + cbase / 8) * p.B + b;
#pragma unroll
                                for (int g = 0; g < 2; ++g)
                                    if (cbase + 8 * g < p.N)
                                        dst[g0 + (size_t)g * p.B] = make_int4(
                                            (resv[8 * g] & 0xffff) | (resv[8 * g + 1] << 16),
                                            (resv[8 * g + 2] & 0xffff) | (resv[8 * g + 3] << 16),
                                            (resv[8 * g + 4] & 0xffff) | (resv[8 * g + 5] << 16),
                                            (resv[8 * g + 6] & 0xffff) | (resv[8 * g + 7] << 16));
                            } else {
                                const size_t g0 = (pix * (size_t)((p.N + 3) / 4) + cbase / 4) * p.B + b;
#pragma unroll
                                for (int g = 0; g < 4; ++g)
                                    if (cbase + 4 * g < p.N)
                                        dst[g0 + (size_t)g * p.B] =
                                            make_int4(resv[4 * g], resv[4 * g + 1], resv[4 * g + 2], resv[4 * g + 3]);
                            }
                        }
                    }
                    const uint32_t other = (uint32_t)__shfl_xor((int)hw, 32);
                    outword[mt][nt] |= h == 0 ? (hw << 16) | other : (other << 16) | hw;
                    // one tile's epilogue at a time: interleaving them multiplies the live temporaries
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    if (!b_ok) continue;
                    if (p.ksplit > 1) {  // partial dot products; the finishing kernel does the rest
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (cbase + v < p.N)
                                atomicAdd(p.workspace + (size_t)(cbase + v) * p.B + b,
                                          A::to_int(acc[mt][nt][v]));
                    } else if (p.mode == EPI_AFFINE) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int c = cbase + v;
                            // the +-1 dot product equals (float)K - (float)popc*2.0f exactly
                            if (c < p.N)
                                p.out_f32[(size_t)b * p.N + c] = __fadd_rn(
                                    __fmul_rn((float)A::to_int(acc[mt][nt][v]), bnp[c]), p.bn_bias[c]);
                        }
                    } else {
                        int32_t* dst = p.out_i32 + pix * p.raw_pix_stride + (size_t)b * p.raw_b_stride + cbase;
                        // a lane's 16 values are consecutive in memory: four 128-bit stores where the
                        // run is whole and aligned
                        if (cbase + 16 <= p.N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
#pragma unroll
                            for (int g = 0; g < 4; ++g)
                                reinterpret_cast<int4*>(dst)[g] =
                                    make_int4(A::to_int(acc[mt][nt][4 * g]), A::to_int(acc[mt][nt][4 * g + 1]),
                                              A::to_int(acc[mt][nt][4 * g + 2]), A::to_int(acc[mt][nt][4 * g + 3]));
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v)
                                if (cbase + v < p.N) dst[v] = A::to_int(acc[mt][nt][v]);
                        }
                    }
                }
            }
        }
    }

    if ((MM == MM_THRESH || MM == MM_THRESH_RES) && active && h == 0) {
        const int n_words = (p.N + 31) / 32;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (bimg[mt] >= p.B) continue;
            uint32_t* dst = p.out_bits + (size_t)opix * p.bits_pix_stride + bimg[mt];
#pragma unroll
            for (int nt = 0; nt < kNT; ++nt) {
                const int w = ng * kNT + nt;
                if (w < p.bits_row_words) dst[(size_t)w * p.B] = outword[mt][nt];
            }
            if (ng == n_groups - 1)  // zero the pixel's padding words
                for (int w = max(n_words, n_groups * kNT); w < p.bits_row_words; ++w)
                    dst[(size_t)w * p.B] = 0;
        }
    }
}

int images_per_wave_tiles(const BgemmParams& p) {
    const long long pix = (long long)p.OH * p.OW;
    const int n_groups = (p.N + 32 * kNT - 1) / (32 * kNT);
    // the residual epilogue does not fit 256 registers next to the accumulators of four image tiles
    const int mt_max = (p.res_in != nullptr || p.res_out != nullptr) ? 2 : 4;
    for (int mt = mt_max; mt > 1; mt >>= 1) {
        if (p.B <= 32 * (mt / 2)) continue;
        const long long waves = pix * ((p.B + 32 * mt - 1) / (32 * mt)) * n_groups * p.ksplit;
        if (waves >= 2048) return mt;
    }
    return 1;
}

int mfma_mode(const BgemmParams& p) {
    if (p.ksplit > 1 || p.mode != EPI_THRESH) return MM_OTHER;
    return (p.res_in != nullptr || p.res_out != nullptr) ? MM_THRESH_RES : MM_THRESH;
}

template <int FMT, int MT, int MM>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    const int n_groups = (p.N + 32 * kNT - 1) / (32 * kNT);
    const int b_groups = (p.B + 32 * MT - 1) / (32 * MT);
    const long long row_waves = (long long)p.OH * p.OW * b_groups;
    const long long row_blocks = (row_waves + kWaves - 1) / kWaves;
    const long long blocks = row_blocks * n_groups * p.ksplit;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return fail(TCBNN_EINVAL, "bgemm grid too large");
    hipLaunchKernelGGL((bgemm_mfma_kernel<FMT, MT, MM>), dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, p, p.act, p.wgt, p.mode == EPI_AFFINE ? p.bn_scale : p.bn, p.res_in,
                       n_groups, (int)row_waves, b_groups, (int)row_blocks);
    TCBNN_LAUNCH_CHECK("bgemm_mfma_kernel");
    return TCBNN_OK;
}

template <int FMT, int MT>
int launch_m(const BgemmParams& p, hipStream_t stream) {
    switch (mfma_mode(p)) {
        case MM_THRESH:
            return launch_t<FMT, MT, MM_THRESH>(p, stream);
        case MM_THRESH_RES:
            return launch_t<FMT, MT, MM_THRESH_RES>(p, stream);
        default:
            return launch_t<FMT, MT, MM_OTHER>(p, stream);
    }
}

template <int FMT>
int launch_f(const BgemmParams& p, hipStream_t stream) {
    switch (images_per_wave_tiles(p)) {
        case 4:
            return launch_m<FMT, 4>(p, stream);
        case 2:
            return launch_m<FMT, 2>(p, stream);
        default:
            return launch_m<FMT, 1>(p, stream);
    }
}

int mfma_ksplit(const BgemmParams& p, int variant) {
    if (p.workspace == nullptr || p.PH * p.PW != 1 || p.R * p.S != 1 || p.res_in || p.res_out)
        return 1;
    const int n_groups = (p.N + 32 * kNT - 1) / (32 * kNT);
    const long long waves = (long long)((p.B + 31) / 32) * n_groups;
    const int steps = variant == TCBNN_VARIANT_MFMA_F4 ? (p.cw + 1) / 2 : p.cw;
    int ks = (int)(2048 / waves);
    ks = min(ks, steps / 8);
    return ks < 2 ? 1 : min(ks, 64);
}

}  // namespace

void bgemm_mfma_kernel_name(const BgemmParams& p, int variant, char* buf, size_t len) {
    if (variant == TCBNN_VARIANT_MFMA_F4 && conv3x3_mfma_applicable(p)) {
        conv3x3_mfma_kernel_name(p, buf, len);
        return;
    }
    if (variant == TCBNN_VARIANT_MFMA_F4 && gemm_mfma_applicable(p)) {
        gemm_mfma_kernel_name(p, buf, len);
        return;
    }
    if (variant == TCBNN_VARIANT_MFMA_F4 && fc_mfma_applicable(p)) {
        fc_mfma_kernel_name(p, buf, len);
        return;
    }
    BgemmParams q = p;
    q.ksplit = mfma_ksplit(p, variant);
    snprintf(buf, len, "bgemm_mfma_kernel<%d, %d, %d>", variant == TCBNN_VARIANT_MFMA_F4 ? FMT_F4 : FMT_I8,
             images_per_wave_tiles(q), mfma_mode(q));
}

int launch_bgemm_mfma(const BgemmParams& p_in, int variant, hipStream_t stream) {
    if (int rc = validate_bgemm(p_in)) return rc;
    if (variant == TCBNN_VARIANT_MFMA_F4 && conv3x3_mfma_applicable(p_in))
        return launch_conv3x3_mfma(p_in, stream);
    if (variant == TCBNN_VARIANT_MFMA_F4 && gemm_mfma_applicable(p_in)) return launch_gemm_mfma(p_in, stream);
    if (variant == TCBNN_VARIANT_MFMA_F4 && fc_mfma_applicable(p_in)) return launch_fc_mfma(p_in, stream);
    if ((long long)p_in.cw * p_in.B * 4 >= (1LL << 31))
        return fail(TCBNN_EUNSUPPORTED, "bgemm: one pixel's activation words must stay below 2 GiB");
    BgemmParams p = p_in;
    p.ksplit = mfma_ksplit(p, variant);
    p.ws_is_dot = 1;
    if (p.ksplit > 1)
        if (int rc = launch_splitk_clear(p, stream)) return rc;
    const int rc = variant == TCBNN_VARIANT_MFMA_F4 ? launch_f<FMT_F4>(p, stream) : launch_f<FMT_I8>(p, stream);
    if (rc) return rc;
    if (p.ksplit > 1) return launch_splitk_finish(p, stream);
    return TCBNN_OK;
}

}  // namespace tcbnn
