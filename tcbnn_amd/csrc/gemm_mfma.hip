// FP4 matrix-core kernel for LARGE bit-GEMMs: the stand-alone bit matrix product (BMMAS_new,
// tensorcore_kernel.cu:336-356: C = K - 2 popc(A xor B)) and fully connected layers at large batch
// (Fc128LayerFMT / Out128LayerFMT, kernel.cuh:174-280; e.g. the 1024 -> 1024 layers of the MLP at batch
// 8192), where K is a whole number of 64-bit words per row.  The generic implicit-GEMM
// kernel serves the same problems, but pays for its generality in every k-step (tap bookkeeping, frame and
// range tests, weights expanded with masks behind two barriers per block).
//
//   workgroup = 4 waves = (4 x MT x 32 rows of the batch / of A) x 64 output columns;
//   wave      = MT image tiles x 2 column tiles: 2 MT MFMAs (32 x 32 x 64, FP4) per k-step;
//   weights   : the 64 columns' words are expanded to MFMA "A" fragments in LDS, 16 k-steps at a time,
//               double-buffered: the words of the next block are requested before the current block is
//               multiplied and expanded into the other buffer after it, one barrier per block;
//   rows      : a lane's words come straight from memory through buffer addressing (one per-lane constant
//               offset per image tile, the k-step in the scalar offset), four k-steps ahead of their use.
// Operand roles, fragment order and the accumulator layout are those of bgemm_mfma.hip.
#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

using namespace mfma;

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int kNT = 2;     // 32-column tiles per wave
constexpr int kBlk = 16;   // k-steps of weights per LDS buffer (16 * kNT KiB)
constexpr int kAhead = 8;  // k-steps a row word is requested ahead of its use; divides kBlk
constexpr int kFrags = kBlk * kNT / kWaves;  // fragments a wave stages per block

// Row words are expanded without shifts (expand_rows_f4 in mfma_util.h): the accumulator ends as the dot product
// plus a per-column constant, which the staging lanes count as they go and the epilogue takes off.
template <int MT, int EPI>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void gemm_mfma_f4_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const float* __restrict__ bias, int n_groups) {
    __shared__ v4i lds_w[2][kBlk * kNT * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int j = lane & 31;  // image within a 32-image tile
    const int h = lane >> 5;  // k half (operands) / column half (accumulator)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ng = blockIdx.x % n_groups, rb = blockIdx.x / n_groups;
    const int n0 = ng * (32 * kNT);
    const int b0 = (rb * kWaves + wave) * (32 * MT);
    // 64-bit k-steps (cw is even, host checked), run in whole groups of kAhead.  Nothing is masked: a pad bit is 0 in
    // both operands (the layouts' convention), and so is every bit of a step past K (rows: outside the descriptor's
    // range; weights: staged as 0).  A 0 bit expands to +1.0 on both sides, so each such position adds exactly +1
    // to the dot product, and the known count is taken off in the epilogue.
    const int true_steps = p.cw / 2;
    const int steps = (true_steps + kAhead - 1) / kAhead * kAhead;
    const int corr = 32 * p.cw - p.k_tap + 64 * (steps - true_steps);

    // ---- weights: this wave stages fragments f = wave + 4 i = (k-step ql = wave/2 + 2 i, column tile wave % 2)
    const int snt = wave & 1, sq = wave >> 1;
    // a row past N (stand-alone product: the rows do not exist) reads the last row; its results are discarded
    const uint32_t* __restrict__ wrow = wgt + (size_t)min(n0 + snt * 32 + row_to_channel(j), p.N - 1) * p.cw + h;
    uint32_t wx[kFrags];
    auto stage_load = [&](int q0) {
#pragma unroll
        for (int i = 0; i < kFrags; ++i) {
            const int q = q0 + sq + 2 * i;
            wx[i] = q < true_steps ? wrow[2 * q] : 0u;
        }
    };
    int csum = 0;  // this lane's share of its column's constant C: the words it stages, pad steps included
    auto stage_store = [&](int buf, int q0) {
#pragma unroll
        for (int i = 0; i < kFrags; ++i) {
            lds_w[buf][((sq + 2 * i) * kNT + snt) * 64 + lane] = expand_weights_f4(wx[i]);
            if (q0 + sq + 2 * i < steps) csum += class_sum(wx[i]);
        }
    };

    // ---- rows: words [cw][B]; lane (j, h) of image tile mt reads word 2 q + h of image b0 + 32 mt + j
    int bimg[MT], voff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        bimg[mt] = b0 + mt * 32 + j;
        voff[mt] = (h * p.B + min(bimg[mt], p.B - 1)) * 4;
    }
    const __amdgpu_buffer_rsrc_t r_act =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(act), 0, p.cw * p.B * 4, 0x00020000);
    const int step_bytes = 2 * p.B * 4;
    uint32_t ring[kAhead][MT];
    int lq = 0;  // next k-step to request
    // no test for the end of K: a request past it lies outside the descriptor's range, touches no memory and
    // returns 0 (such words are never multiplied), and the k-steps stay free of branches
    auto request = [&](uint32_t* dst) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            dst[mt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r_act, voff[mt], lq * step_bytes, 0);
        ++lq;
    };

    v16f acc[MT][kNT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mt][nt][v] = 0.0f;

#pragma unroll
    for (int d = 0; d < kAhead; ++d) request(ring[d]);
    stage_load(0);
    stage_store(0, 0);
    __syncthreads();

    // Software pipeline, one k-step deep: while step q is multiplied, the weight fragments of step q + 1 are on
    // their way from LDS and its row words are expanded (their ring slot is then asked for step q + 5).  Step q's
    // words sit in ring slot q % kAhead; kBlk is a multiple of kAhead, so the slot of step ql + d of a block is d.
    v4i anext[kNT], bnext[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) bnext[mt] = expand_rows_f4(ring[0][mt]);
    request(ring[0]);

    int buf = 0;
    for (int q0 = 0; q0 < steps; q0 += kBlk) {
        const bool more = q0 + kBlk < steps;  // uniform
        if (more) stage_load(q0 + kBlk);
        const int cnt = min(kBlk, steps - q0);  // a multiple of kAhead
        const v4i* __restrict__ wl = lds_w[buf];
#pragma unroll
        for (int nt = 0; nt < kNT; ++nt) anext[nt] = wl[nt * 64 + lane];
        for (int ql = 0; ql < cnt; ql += kAhead) {
#pragma unroll
            for (int d = 0; d < kAhead; ++d) {
                v4i acur[kNT], bcur[MT];
#pragma unroll
                for (int nt = 0; nt < kNT; ++nt) acur[nt] = anext[nt];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) bcur[mt] = bnext[mt];
                const int qn = min(ql + d + 1, kBlk - 1);  // after a block's last step: read again, not used
#pragma unroll
                for (int nt = 0; nt < kNT; ++nt) anext[nt] = wl[(qn * kNT + nt) * 64 + lane];
                const int dn = (d + 1) % kAhead;  // a constant once the loop over d is unrolled
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) bnext[mt] = expand_rows_f4(ring[dn][mt]);
                request(ring[dn]);
#pragma unroll
                for (int nt = 0; nt < kNT; ++nt)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][nt] = Acc<FMT_F4>::mma(acur[nt], bcur[mt], acc[mt][nt]);
                // issue order of the step: fragment reads first, then each MFMA followed by a few of the next
                // step's expansion instructions (they run while the matrix pipeline is busy), the row requests
                // in the middle
                __builtin_amdgcn_sched_group_barrier(0x100, kNT, 0);  // LDS reads
#pragma unroll
                for (int i = 0; i < kNT * MT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x002, (4 * MT + kNT * MT - 1) / (kNT * MT), 0);  // VALU
                    if (i == kNT * MT / 2) __builtin_amdgcn_sched_group_barrier(0x020, MT, 0);  // row requests
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the other buffer was last read in the previous block, which every wave left before the barrier below
        if (more) stage_store(buf ^ 1, q0 + kBlk);
        __syncthreads();
        buf ^= 1;
    }

    // ---- the columns' constants: four lanes (two k-halves of two waves) staged each column's words.  The weight
    // buffers are free now (every wave has passed the loop's last barrier).
    int* colc = reinterpret_cast<int*>(&lds_w[0][0]);  // [kNT * 32]
    if (tid < kNT * 32) colc[tid] = 0;
    __syncthreads();
    atomicAdd(&colc[snt * 32 + row_to_channel(j)], csum);
    __syncthreads();

    // int32 output, all 64 columns of the group exist and every row's run of them is 16-byte aligned (uniform): the
    // sums leave through LDS, a row at a time (below)
    const bool raw_rows = EPI == EPI_RAW && n0 + 32 * kNT <= p.N && p.raw_b_stride % 4 == 0 &&
                          (reinterpret_cast<uintptr_t>(p.out_i32) & 15) == 0;

    // ---- epilogue: the lane holds columns cbase + v of image bimg[mt]
#pragma unroll
    for (int nt = 0; nt < kNT; ++nt) {
        const int cbase = n0 + nt * 32 + 16 * h;
        int off[16];  // what the accumulator holds beyond the dot product
#pragma unroll
        for (int v = 0; v < 16; ++v) off[v] = corr + colc[nt * 32 + 16 * h + v];
        float thr[16], bia[EPI == EPI_AFFINE ? 16 : 1];
        if constexpr (EPI != EPI_RAW) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                thr[v] = bnp[min(cbase + v, p.N - 1)];
                if constexpr (EPI == EPI_AFFINE) bia[v] = bias[min(cbase + v, p.N - 1)];
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int b = bimg[mt];
            const bool b_ok = b < p.B;
            if constexpr (EPI == EPI_THRESH) {
                uint32_t hw = 0;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const uint32_t bit = cbase + v < p.N ? thresh_bit((int)acc[mt][nt][v] - off[v], thr[v], p.nan_bit) : 0u;
                    hw = hw + hw + bit;
                }
                const uint32_t other = (uint32_t)__shfl_xor((int)hw, 32);
                const int w = ng * kNT + nt;
                if (h == 0 && b_ok) {
                    if (w < p.bits_row_words) p.out_bits[(size_t)w * p.B + b] = (hw << 16) | other;
                    if (ng == n_groups - 1 && nt == kNT - 1)  // padding words of the 128-padded feature axis
                        for (int z = max((p.N + 31) / 32, n_groups * kNT); z < p.bits_row_words; ++z)
                            p.out_bits[(size_t)z * p.B + b] = 0;
                }
            } else if constexpr (EPI == EPI_AFFINE) {
                if (b_ok) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        // the +-1 dot product equals (float)K - (float)popc*2.0f exactly (kernel.cuh:258-270)
                        if (cbase + v < p.N)
                            p.out_f32[(size_t)b * p.N + cbase + v] =
                                __fadd_rn(__fmul_rn((float)((int)acc[mt][nt][v] - off[v]), thr[v]), bia[v]);
                }
            } else if (raw_rows) {
                // (int32 output of whole, aligned column groups: written further down, a row at a time)
            } else {
                if (b_ok) {
                    int32_t* dst = p.out_i32 + (size_t)b * p.raw_b_stride + cbase;
                    // a lane's 16 values are consecutive in memory: four 128-bit stores where the run is whole
                    // and aligned
                    if (cbase + 16 <= p.N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            reinterpret_cast<int4*>(dst)[g] =
                                make_int4((int)acc[mt][nt][4 * g] - off[4 * g], (int)acc[mt][nt][4 * g + 1] - off[4 * g + 1],
                                          (int)acc[mt][nt][4 * g + 2] - off[4 * g + 2],
                                          (int)acc[mt][nt][4 * g + 3] - off[4 * g + 3]);
                    } else {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (cbase + v < p.N) dst[v] = (int)acc[mt][nt][v] - off[v];
                    }
                }
            }
        }
    }

    // int32 output [rows][N] (BMMAS_new, tensorcore_kernel.cu:355): in the accumulator a lane holds 16 columns of ONE
    // row, so a direct store scatters 16-byte pieces over 64 different rows per instruction (the product writes
    // 4 M N bytes: a quarter of the 8192^3 launch was this).  The sums of a 32-row tile go through a per-wave LDS
    // area instead (row = image, pitch 68 words: conflict-free both ways; the weight buffers are free by now) and
    // leave as 128-bit stores in which 16 consecutive lanes cover one row's whole run of 64 columns (4 runs of
    // 256 bytes per instruction).
    if constexpr (EPI == EPI_RAW) {
        if (raw_rows) {
            constexpr int kPitch = 32 * kNT + 4;
            // (behind the column constants, which stay where they are)
            int* mine = reinterpret_cast<int*>(&lds_w[0][0]) + kNT * 32 + wave * (32 * kPitch);
            const int rl = lane >> 4, cl = lane & 15;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int nt = 0; nt < kNT; ++nt) {
                    int off[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) off[v] = corr + colc[nt * 32 + 16 * h + v];
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *reinterpret_cast<v4i*>(mine + j * kPitch + nt * 32 + 16 * h + 4 * g) =
                            v4i{(int)acc[mt][nt][4 * g] - off[4 * g], (int)acc[mt][nt][4 * g + 1] - off[4 * g + 1],
                                (int)acc[mt][nt][4 * g + 2] - off[4 * g + 2], (int)acc[mt][nt][4 * g + 3] - off[4 * g + 3]};
                }
                // (same wave writes and reads: program order and the wait for LDS are all the synchronisation)
                const int row0 = b0 + mt * 32;
#pragma unroll
                for (int part = 0; part < 2; ++part) {
                    v4i q[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) q[k] = *reinterpret_cast<const v4i*>(mine + (16 * part + 4 * k + rl) * kPitch + 4 * cl);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int row = row0 + 16 * part + 4 * k + rl;
                        if (row < p.B)
                            *reinterpret_cast<v4i*>(p.out_i32 + (size_t)row * p.raw_b_stride + n0 + 4 * cl) = q[k];
                    }
                }
            }
        }
    }
}

// image tiles per wave: 4 when that still gives every CU two workgroups
int gemm_mt(const BgemmParams& p) {
    const long long n_groups = (p.N + 32 * kNT - 1) / (32 * kNT);
    return ((p.B + 32 * 4 * kWaves - 1) / (32 * 4 * kWaves)) * n_groups >= 512 ? 4 : 2;
}

}  // namespace

bool gemm_mfma_applicable(const BgemmParams& p) {
    if (p.PH * p.PW != 1 || p.R * p.S != 1 || p.pool_h * p.pool_w != 1) return false;
    if (p.res_in != nullptr || p.res_out != nullptr) return false;
    if (p.mode != EPI_THRESH && p.mode != EPI_AFFINE && p.mode != EPI_RAW) return false;
    if (p.cw % 2 != 0 || p.k_tap > 32 * p.cw) return false;               // whole 64-bit k-steps
    if ((long long)p.cw * p.B * 4 >= (1LL << 31)) return false;          // 32-bit buffer offsets
    // large enough to give every CU a workgroup with two image tiles per wave; smaller problems are bound by
    // launch and fill and stay with the kernels written for them
    const long long wgs = (long long)((p.B + 32 * 2 * kWaves - 1) / (32 * 2 * kWaves)) * ((p.N + 32 * kNT - 1) / (32 * kNT));
    return wgs >= 256;
}

void gemm_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    snprintf(buf, len, "gemm_mfma_f4_kernel<%d, %d>", gemm_mt(p), p.mode);
}

template <int MT>
static int launch_gemm_mt(const BgemmParams& p, hipStream_t stream) {
    const int n_groups = (p.N + 32 * kNT - 1) / (32 * kNT);
    const long long row_blocks = (p.B + 32 * MT * kWaves - 1) / (32 * MT * kWaves);
    const long long blocks = row_blocks * n_groups;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return fail(TCBNN_EINVAL, "gemm grid too large");
    const dim3 grid((unsigned)blocks), block(kThreads);
    switch (p.mode) {
        case EPI_THRESH:
            hipLaunchKernelGGL((gemm_mfma_f4_kernel<MT, EPI_THRESH>), grid, block, 0, stream, p, p.act, p.wgt, p.bn,
                               p.bn, n_groups);
            break;
        case EPI_AFFINE:
            hipLaunchKernelGGL((gemm_mfma_f4_kernel<MT, EPI_AFFINE>), grid, block, 0, stream, p, p.act, p.wgt,
                               p.bn_scale, p.bn_bias, n_groups);
            break;
        default:
            hipLaunchKernelGGL((gemm_mfma_f4_kernel<MT, EPI_RAW>), grid, block, 0, stream, p, p.act, p.wgt, p.bn,
                               p.bn, n_groups);
    }
    TCBNN_LAUNCH_CHECK("gemm_mfma_f4_kernel");
    return TCBNN_OK;
}

int launch_gemm_mfma(const BgemmParams& p, hipStream_t stream) {
    return gemm_mt(p) == 4 ? launch_gemm_mt<4>(p, stream) : launch_gemm_mt<2>(p, stream);
}

}  // namespace tcbnn
