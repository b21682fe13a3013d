// XOR + popcount implicit GEMM for gfx950 (the VALU variant of the bit-matmul /
// bit-convolution hot path).
//
// Mapping (64-lane wavefronts):
//   lane            = one image b of a batch tile; a wave holds RPL batch tiles of 64
//                     images (RPL rows per lane) that all sit on the SAME output pixel,
//                     so the zero-padding predicate of a filter tap is wave-uniform
//                     (a scalar branch) and, with the batch-innermost activation layout
//                     [H][W][cw][B], every activation word load is one contiguous
//                     256-byte run.
//   workgroup       = 4 waves (4 different (pixel, batch-tile) rows) x one tile of 32
//                     output channels.  The weights of that channel tile are staged
//                     once in LDS as [k-chunk][32 channels][CH words]; every lane reads
//                     the same LDS address (broadcast ds_read_b128), so a weight word
//                     costs no VGPR traffic and no bank conflicts.
//   inner product   = v_xor_b32 + v_bcnt_u32_b32 (accumulating form): 2 VALU ops per
//                     32 +-1 multiply-accumulates.
//   epilogue        = in-lane: the lane owns all 32 channel sums of its row, so
//                     threshold -> bit -> shift/or builds the packed output word with
//                     no ballot, no LDS round trip and no atomics; residual tensors keep
//                     the batch below small channel groups, so consecutive lanes touch
//                     consecutive 16-byte slots.  Pool windows are a sequential
//                     loop in the same lane (OR of the words), so every output word is
//                     written exactly once and re-runs are idempotent.
//   split-K         = FC-shaped problems with few rows split K over blockIdx; partial
//                     popcounts are atomically added into an int32 workspace and a small
//                     finishing kernel applies the epilogue.
//
// Semantics follow Fc128LayerFMT / Out128LayerFMT / Conv128LayerFMT
// (kernel.cuh:174-280, 676-827) and BMMAS / BTC_Conv2d_balance
// (tensorcore_kernel.cu:305-356, bmma_kernel.cu:101-165).
#include "common.h"

namespace tcbnn {

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kThreads = 64 * kWavesPerBlock;
constexpr int kNTile = 32;
constexpr int kLdsWords = 8192;  // 32 KiB of weights per staging block

template <int CH>
struct WordVec;
template <>
struct WordVec<4> {
    using type = uint4;
};
template <>
struct WordVec<2> {
    using type = uint2;
};
template <>
struct WordVec<1> {
    using type = uint32_t;
};

// acc += popcount(x) in ONE instruction: v_bcnt_u32_b32 adds its second operand.  (Written
// as inline asm because the compiler otherwise popcounts into temporaries and sums them with
// v_add3_u32: 5 instead of 4 VALU operations per two words.)
__device__ __forceinline__ void popc_acc(int& acc, uint32_t x) {
    asm("v_bcnt_u32_b32 %0, %1, %0" : "+v"(acc) : "v"(x));
}
__device__ __forceinline__ void xpopc(int& acc, const uint32_t* a, uint4 w) {
    popc_acc(acc, a[0] ^ w.x);
    popc_acc(acc, a[1] ^ w.y);
    popc_acc(acc, a[2] ^ w.z);
    popc_acc(acc, a[3] ^ w.w);
}
__device__ __forceinline__ void xpopc(int& acc, const uint32_t* a, uint2 w) {
    popc_acc(acc, a[0] ^ w.x);
    popc_acc(acc, a[1] ^ w.y);
}
__device__ __forceinline__ void xpopc(int& acc, const uint32_t* a, uint32_t w) { popc_acc(acc, a[0] ^ w); }

// Threshold compare of the reference: conv layers emit (res < bn) ? 0 : 1
// (kernel.cuh:795-796), FC layers emit (res >= bn) (kernel.cuh:210-213); the two differ
// only when bn is NaN.
__device__ __forceinline__ uint32_t thresh_bit(int res, float thr, int nan_bit) {
    const float rf = (float)res;
    return nan_bit ? (rf < thr ? 0u : 1u) : (rf >= thr ? 1u : 0u);
}

// Epilogue selected at compile time so that each instance only keeps its own operands live.
enum KernelMode : int {
    KM_THRESH = 0,      // threshold + pack (+ pooling)
    KM_THRESH_RES = 1,  // threshold + pack with residual inject and/or save
    KM_AFFINE = 2,      // fp32 affine output
    KM_RAW = 3,         // int32 dot products
    KM_PARTIAL = 4,     // split-K partial popcounts -> workspace
    KM_THRESH_FC = 5,   // threshold + pack with the FC compare (res >= bn: 0 when bn is NaN)
};

// register budget: 32*RPL accumulators + operands; keep as many waves per SIMD as that allows
template <int RPL, int CH, int KM>
__global__ __launch_bounds__(kThreads)
    __attribute__((amdgpu_waves_per_eu(RPL == 1 ? 4 : (RPL == 2 ? 3 : 2)))) void bgemm_popc_kernel(
        const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
        const float* __restrict__ bnp, const int32_t* __restrict__ rin, int n_tiles, int row_waves,
        int b_tiles, int row_blocks) {
    // act / wgt / bnp / rin repeat p.act / p.wgt / p.bn (or p.bn_scale) / p.res_in as __restrict__
    // arguments: read-only and unaliased, so wave-uniform loads from them become scalar loads
    using V = typename WordVec<CH>::type;
    __shared__ __attribute__((aligned(16))) uint32_t lds_w[kLdsWords];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = blockIdx.x % n_tiles;
    const int rb = (blockIdx.x / n_tiles) % row_blocks;
    const int ks = blockIdx.x / (n_tiles * row_blocks);  // K split index
    const int rw = rb * kWavesPerBlock + wave;
    const bool active = rw < row_waves;

    const int cw_chunks = p.cw / CH;
    const int taps = p.R * p.S;
    const int nq_all = taps * cw_chunks;  // k-chunks in total
    const int kw_tot = taps * p.cw;       // words per weight row
    constexpr int kQB = kLdsWords / (kNTile * CH);  // chunks per staging block
    // this block's K range (the whole K unless split)
    const int q_per = (nq_all + p.ksplit - 1) / p.ksplit;
    const int q_begin = ks * q_per;
    const int q_end = min(nq_all, q_begin + q_per);
    const int nq = q_end - q_begin;
    const bool single_block = nq <= kQB;

    const int opix = active ? rw / b_tiles : 0;  // pooled output pixel
    const int bt = active ? rw % b_tiles : 0;
    const int oy = opix / p.OW, ox = opix % p.OW;

    int brow[RPL];
    int bload[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        brow[r] = (bt * RPL + r) * 64 + lane;
        bload[r] = brow[r] < p.B ? brow[r] : p.B - 1;
    }

    auto stage_weights = [&](int q0) {
        const int cnt = min(kQB, q_end - q0);
        const int blk_words = cnt * CH;  // words per weight row in this block
        const uint32_t* wrow = wgt + (size_t)nt * kNTile * kw_tot + (size_t)q0 * CH;
        for (int idx = tid; idx < blk_words * kNTile; idx += kThreads) {
            const int n = idx / blk_words;
            const int kk = idx - n * blk_words;
            lds_w[((kk / CH) * kNTile + n) * CH + (kk % CH)] = wrow[(size_t)n * kw_tot + kk];
        }
    };

    if (single_block && nq > 0) {
        stage_weights(q_begin);
        __syncthreads();
    }

    uint32_t outword[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) outword[r] = 0;

    const int n0 = nt * kNTile;
    const int pool_n = p.pool_h * p.pool_w;
    for (int pp = 0; pp < pool_n; ++pp) {
        const int y = oy * p.pool_h + pp / p.pool_w;
        const int x = ox * p.pool_w + pp % p.pool_w;
        // Every pixel of the pool window is computed, also those past the convolution's own output when the
        // pooled size is rounded up (kernel.cuh:685-690 walks pool * output rows and columns): such a pixel sums
        // the taps that still lie inside the frame (all others count as excluded) and its bit is ORed in.
        const bool valid = active;  // wave-uniform
        const int ay0 = y * p.stride_h - p.pad_h;
        const int ax0 = x * p.stride_w - p.pad_w;

        int acc[RPL][kNTile];
#pragma unroll
        for (int r = 0; r < RPL; ++r)
#pragma unroll
            for (int n = 0; n < kNTile; ++n) acc[r][n] = 0;
        int exclude = 0;

        // Activation words of one k-chunk for this lane's rows; returns the (wave-uniform)
        // in-frame predicate.  Loads are issued one chunk ahead of their use so that their
        // latency overlaps the 32*RPL*CH xor+popcount pairs of the current chunk.
        auto load_chunk = [&](int tr, int ts, int kc, uint32_t (*dst)[CH]) {
            const int ay = ay0 + tr, ax = ax0 + ts;
            const bool in_frame = valid && ay >= 0 && ay < p.H && ax >= 0 && ax < p.W;
            if (in_frame) {
                const uint32_t* src = act + ((size_t)(ay * p.W + ax) * p.cw + kc * CH) * p.B;
#pragma unroll
                for (int j = 0; j < CH; ++j)
#pragma unroll
                    for (int r = 0; r < RPL; ++r) dst[r][j] = src[(size_t)j * p.B + bload[r]];
            }
            return in_frame;
        };

        // running (tap row, tap col, chunk) counters: no integer division in the loop
        int tr = (q_begin / cw_chunks) / p.S, ts = (q_begin / cw_chunks) % p.S,
            kc = q_begin % cw_chunks;
        uint32_t a[RPL][CH], a_next[RPL][CH];
        bool in_frame = q_begin < q_end ? load_chunk(tr, ts, kc, a) : false;
        for (int q0 = q_begin; q0 < q_end; q0 += kQB) {
            if (!single_block) {
                __syncthreads();
                stage_weights(q0);
                __syncthreads();
            }
            const int cnt = min(kQB, q_end - q0);
            for (int ql = 0; ql < cnt; ++ql) {
                int ntr = tr, nts = ts, nkc = kc + 1;
                if (nkc == cw_chunks) {
                    nkc = 0;
                    if (++nts == p.S) {
                        nts = 0;
                        ++ntr;
                    }
                }
                const bool next_in_frame =
                    (q0 + ql + 1 < q_end) ? load_chunk(ntr, nts, nkc, a_next) : false;
                if (in_frame) {
                    const V* wl = reinterpret_cast<const V*>(lds_w) + ql * kNTile;
#pragma unroll
                    for (int n = 0; n < kNTile; ++n) {
                        const V w = wl[n];
#pragma unroll
                        for (int r = 0; r < RPL; ++r) xpopc(acc[r][n], a[r], w);
                    }
                } else if (valid && kc == 0) {
                    ++exclude;
                }
                tr = ntr;
                ts = nts;
                kc = nkc;
                in_frame = next_in_frame;
#pragma unroll
                for (int r = 0; r < RPL; ++r)
#pragma unroll
                    for (int j = 0; j < CH; ++j) a[r][j] = a_next[r][j];
            }
        }

        if (!valid) continue;

        // ---------------- epilogue for pre-pool pixel (y, x) ----------------
        if constexpr (KM == KM_PARTIAL) {  // partial popcounts only; the finishing kernel does the rest
#pragma unroll
            for (int r = 0; r < RPL; ++r) {
                if (brow[r] >= p.B) continue;
#pragma unroll
                for (int n = 0; n < kNTile; ++n)
                    atomicAdd(p.workspace + (size_t)(n0 + n) * p.B + brow[r], acc[r][n]);
            }
            continue;
        }

        const int base = p.k_tap * taps - exclude * p.k_tap;
        const size_t pix = (size_t)y * p.PW + x;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            if (brow[r] >= p.B) continue;
            const int b = brow[r];
            if constexpr (KM == KM_THRESH || KM == KM_THRESH_RES || KM == KM_THRESH_FC) {
                uint32_t word = 0;
                int rv[kNTile];
                if constexpr (KM == KM_THRESH_RES) {
                    // all residual loads first (one contiguous run per channel across the
                    // wave), so they are in flight together before any store is issued
#pragma unroll
                    for (int n = 0; n < kNTile; ++n) {
                        const int ch = n0 + n;
                        int v = 0;
                        if (rin != nullptr && ch < p.res_limit && ch < p.res_in_ch && ch < p.N) {
                            if (p.res_pool) {
                                const size_t rw2 = 2 * (size_t)p.PW, p00 = (size_t)(2 * y) * rw2 + 2 * x;
                                auto at = [&](size_t sp) {
                                    return residual_load(rin, p.res_in_fmt, sp, p.res_in_ch, ch, p.B, b);
                                };
                                v = max(max(at(p00), at(p00 + 1)), max(at(p00 + rw2), at(p00 + rw2 + 1)));
                            } else {
                                v = residual_load(rin, p.res_in_fmt, pix, p.res_in_ch, ch, p.B, b);
                            }
                        }
                        rv[n] = v;
                    }
                }
                const float* __restrict__ bn = bnp;
                int32_t* __restrict__ rout = p.res_out;
                const bool by_group = KM == KM_THRESH_RES && rout != nullptr && p.res_out_fmt == TCBNN_RES_I12;
#pragma unroll
                for (int n = 0; n < kNTile; ++n) {
                    const int ch = n0 + n;
                    uint32_t bit = 0;
                    if (ch < p.N) {  // wave-uniform
                        int res = base - 2 * acc[r][n];
                        if constexpr (KM == KM_THRESH_RES) {
                            res += rv[n];
                            if (by_group)
                                rv[n] = res;  // 12-bit values share words: the tile's two groups are stored whole below
                            else if (rout != nullptr)
                                residual_store(rout, p.res_out_fmt, pix, p.N, ch, p.B, b, res);
                        }
                        if constexpr (KM == KM_THRESH_FC)
                            bit = (float)res >= bn[ch] ? 1u : 0u;
                        else
                            bit = (float)res < bn[ch] ? 0u : 1u;
                    }
                    word = word + word + bit;  // shift the next channel in (MSB first)
                }
                if constexpr (KM == KM_THRESH_RES) {
                    if (by_group) {
#pragma unroll
                        for (int g = 0; g < 2; ++g)
                            if (n0 + 16 * g < p.N)
                                residual_store_group16(rout, TCBNN_RES_I12, pix, p.N, (n0 >> 4) + g, p.B, b, &rv[16 * g]);
                    }
                }
                outword[r] |= word;
            } else if constexpr (KM == KM_AFFINE) {
                float* dst = p.out_f32 + (size_t)b * p.N;
#pragma unroll
                for (int n = 0; n < kNTile; ++n) {
                    const int ch = n0 + n;
                    if (ch < p.N) {
                        // (float)K - (float)c*2.0f is exact; multiply and add are kept
                        // separate (no FMA contraction) so the result is reproducible.
                        const float d = (float)p.k_tap - (float)acc[r][n] * 2.0f;
                        dst[ch] = __fadd_rn(__fmul_rn(d, bnp[ch]), p.bn_bias[ch]);
                    }
                }
            } else if constexpr (KM == KM_RAW) {
                int32_t* dst = p.out_i32 + pix * p.raw_pix_stride + (size_t)b * p.raw_b_stride;
#pragma unroll
                for (int n = 0; n < kNTile; ++n)
                    if (n0 + n < p.N) dst[n0 + n] = base - 2 * acc[r][n];
            }
        }
    }

    if ((KM == KM_THRESH || KM == KM_THRESH_RES || KM == KM_THRESH_FC) && active) {
#pragma unroll
        for (int r = 0; r < RPL; ++r)
            if (brow[r] < p.B) {
                uint32_t* dst = p.out_bits + (size_t)opix * p.bits_pix_stride + brow[r];
                dst[(size_t)nt * p.B] = outword[r];
                if (nt == n_tiles - 1)  // zero the pixel's padding words
                    for (int w = n_tiles; w < p.bits_row_words; ++w) dst[(size_t)w * p.B] = 0;
            }
    }
}

// ---- split-K helpers: workspace int32 [npad32][B] of popcounts -----------------------
__global__ void splitk_clear_kernel(int32_t* ws, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) ws[i] = 0;
}

__global__ __launch_bounds__(256) void splitk_finish_kernel(const BgemmParams p, int n_tiles) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)n_tiles * p.B) return;
    const int b = (int)(i % p.B);
    const int nt = (int)(i / p.B);
    const int n0 = nt * kNTile;
    // the +-1 dot product from what the engine accumulated
    auto dot = [&](int n) {
        const int w = p.workspace[(size_t)(n0 + n) * p.B + b];
        return p.ws_is_dot ? w : p.k_tap - 2 * w;
    };
    if (p.mode == EPI_THRESH) {
        uint32_t word = 0;
        for (int n = 0; n < kNTile && n0 + n < p.N; ++n)
            word |= thresh_bit(dot(n), p.bn[n0 + n], p.nan_bit) << (31 - n);
        p.out_bits[(size_t)nt * p.B + b] = word;
        if (nt == n_tiles - 1)
            for (int w = n_tiles; w < p.bits_row_words; ++w) p.out_bits[(size_t)w * p.B + b] = 0;
    } else if (p.mode == EPI_AFFINE) {
        for (int n = 0; n < kNTile && n0 + n < p.N; ++n)
            p.out_f32[(size_t)b * p.N + n0 + n] =
                __fadd_rn(__fmul_rn((float)dot(n), p.bn_scale[n0 + n]), p.bn_bias[n0 + n]);
    } else {
        for (int n = 0; n < kNTile && n0 + n < p.N; ++n)
            p.out_i32[(size_t)b * p.raw_b_stride + n0 + n] = dot(n);
    }
}

int rows_per_lane(const BgemmParams& p) {
    // as many 64-image tiles per lane as the batch holds, but never so many that the
    // launch no longer fills the chip
    const long long pix = (long long)p.OH * p.OW;
    const int n_tiles = (p.N + kNTile - 1) / kNTile;
    for (int rpl = 4; rpl > 1; rpl >>= 1) {
        if (p.B <= 64 * (rpl / 2)) continue;
        const long long waves = pix * ((p.B + 64 * rpl - 1) / (64 * rpl)) * n_tiles * p.ksplit;
        if (waves >= 2048) return rpl;
    }
    return 1;
}

template <int RPL, int CH, int KM>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    const int n_tiles = (p.N + kNTile - 1) / kNTile;
    const int b_tiles = (p.B + 64 * RPL - 1) / (64 * RPL);
    const long long row_waves = (long long)p.OH * p.OW * b_tiles;
    const long long row_blocks = (row_waves + kWavesPerBlock - 1) / kWavesPerBlock;
    const long long blocks = row_blocks * n_tiles * p.ksplit;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return fail(TCBNN_EINVAL, "bgemm grid too large");
    hipLaunchKernelGGL((bgemm_popc_kernel<RPL, CH, KM>), dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, p, p.act, p.wgt, p.mode == EPI_AFFINE ? p.bn_scale : p.bn, p.res_in, n_tiles,
                       (int)row_waves, b_tiles, (int)row_blocks);
    TCBNN_LAUNCH_CHECK("bgemm_popc_kernel");
    return TCBNN_OK;
}

int kernel_mode(const BgemmParams& p) {
    if (p.ksplit > 1) return KM_PARTIAL;
    if (p.mode == EPI_AFFINE) return KM_AFFINE;
    if (p.mode == EPI_RAW) return KM_RAW;
    if (p.res_in != nullptr || p.res_out != nullptr) return KM_THRESH_RES;
    // the FC compare differs from the conv compare only for NaN thresholds; it is only
    // instantiated for FC-shaped problems (whole 128-bit words per row)
    return (p.nan_bit == 0 && p.cw % 4 == 0) ? KM_THRESH_FC : KM_THRESH;
}

template <int RPL, int CH>
int launch_m(const BgemmParams& p, hipStream_t stream) {
    switch (kernel_mode(p)) {
        case KM_THRESH:
            return launch_t<RPL, CH, KM_THRESH>(p, stream);
        case KM_THRESH_RES:
            return launch_t<RPL, CH, KM_THRESH_RES>(p, stream);
        case KM_AFFINE:
            return launch_t<RPL, CH, KM_AFFINE>(p, stream);
        case KM_RAW:
            return launch_t<RPL, CH, KM_RAW>(p, stream);
        case KM_THRESH_FC:
            if constexpr (CH == 4) return launch_t<RPL, CH, KM_THRESH_FC>(p, stream);
            return fail(TCBNN_EINVAL, "bgemm: FC compare needs 128-bit aligned rows");
        default:
            return launch_t<RPL, CH, KM_PARTIAL>(p, stream);
    }
}

template <int CH>
int launch_r(const BgemmParams& p, hipStream_t stream) {
    if constexpr (CH == 1) {  // odd word counts are rare: one instance
        return launch_m<1, CH>(p, stream);
    } else {
        switch (rows_per_lane(p)) {
            case 4:
                return launch_m<4, CH>(p, stream);
            case 2:
                return launch_m<2, CH>(p, stream);
            default:
                return launch_m<1, CH>(p, stream);
        }
    }
}

int chunk_words(const BgemmParams& p) { return p.cw % 4 == 0 ? 4 : (p.cw % 2 == 0 ? 2 : 1); }

}  // namespace

int validate_bgemm(const BgemmParams& p) {
    TCBNN_NOTNULL(p.act);
    TCBNN_NOTNULL(p.wgt);
    TCBNN_REQUIRE(p.H > 0 && p.W > 0 && p.B > 0 && p.cw > 0 && p.N > 0, "bgemm: empty dimension");
    TCBNN_REQUIRE(p.R > 0 && p.S > 0 && p.stride_h > 0 && p.stride_w > 0, "bgemm: bad filter");
    TCBNN_REQUIRE(p.pool_h > 0 && p.pool_w > 0 && p.PH > 0 && p.PW > 0, "bgemm: bad pooling");
    TCBNN_REQUIRE(p.OH == (p.PH + p.pool_h - 1) / p.pool_h && p.OW == (p.PW + p.pool_w - 1) / p.pool_w,
                  "bgemm: pooled size mismatch");
    TCBNN_REQUIRE((long long)p.k_tap * p.R * p.S < (1 << 24),
                  "bgemm: K too large for exact fp32 compare");
    if (p.mode == EPI_THRESH) {
        TCBNN_NOTNULL(p.bn);
        TCBNN_NOTNULL(p.out_bits);
    } else if (p.mode == EPI_AFFINE) {
        TCBNN_NOTNULL(p.bn_scale);
        TCBNN_NOTNULL(p.bn_bias);
        TCBNN_NOTNULL(p.out_f32);
        TCBNN_REQUIRE(p.PH == 1 && p.PW == 1, "bgemm: affine epilogue is FC only");
    } else {
        TCBNN_NOTNULL(p.out_i32);
    }
    if (p.res_in != nullptr || p.res_out != nullptr)
        TCBNN_REQUIRE(p.pool_h == 1 && p.pool_w == 1, "residual save/inject requires pool 1x1");
    if (p.mode != EPI_THRESH)
        TCBNN_REQUIRE(p.pool_h == 1 && p.pool_w == 1, "pooling needs the threshold epilogue");
    return TCBNN_OK;
}

int choose_ksplit(const BgemmParams& p) {
    // only FC-shaped problems (one pixel, one tap) with a workspace are split
    if (p.workspace == nullptr || p.PH * p.PW != 1 || p.R * p.S != 1 || p.res_in || p.res_out)
        return 1;
    const int n_tiles = (p.N + kNTile - 1) / kNTile;
    const long long waves = (long long)((p.B + 63) / 64) * n_tiles;
    const int chunks = p.cw / chunk_words(p);
    int ks = (int)(2048 / waves);
    ks = min(ks, chunks / 8);
    return ks < 2 ? 1 : min(ks, 64);
}

int launch_splitk_clear(const BgemmParams& p, hipStream_t stream) {
    const size_t n = (size_t)pad32(p.N) * p.B;
    hipLaunchKernelGGL(splitk_clear_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                       p.workspace, n);
    TCBNN_LAUNCH_CHECK("splitk_clear_kernel");
    return TCBNN_OK;
}

int launch_splitk_finish(const BgemmParams& p, hipStream_t stream) {
    const int n_tiles = (p.N + kNTile - 1) / kNTile;
    const size_t n = (size_t)n_tiles * p.B;
    hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                       p, n_tiles);
    TCBNN_LAUNCH_CHECK("splitk_finish_kernel");
    return TCBNN_OK;
}

void bgemm_popc_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    BgemmParams q = p;
    q.ksplit = choose_ksplit(p);
    const int ch = chunk_words(q);
    snprintf(buf, len, "bgemm_popc_kernel<%d, %d, %d>", ch == 1 ? 1 : rows_per_lane(q), ch, kernel_mode(q));
}

int launch_bgemm_popc(const BgemmParams& p_in, hipStream_t stream) {
    if (int rc = validate_bgemm(p_in)) return rc;
    BgemmParams p = p_in;
    p.ksplit = choose_ksplit(p);
    if (p.ksplit > 1)
        if (int rc = launch_splitk_clear(p, stream)) return rc;
    int rc;
    switch (chunk_words(p)) {
        case 4:
            rc = launch_r<4>(p, stream);
            break;
        case 2:
            rc = launch_r<2>(p, stream);
            break;
        default:
            rc = launch_r<1>(p, stream);
    }
    if (rc) return rc;
    if (p.ksplit > 1) return launch_splitk_finish(p, stream);
    return TCBNN_OK;
}

}  // namespace tcbnn
