// XOR + popcount implicit GEMM for gfx950 (the VALU variant of the bit-matmul /
// bit-convolution hot path).
//
// Mapping (64-lane wavefronts):
//   lane            = one image b of a batch tile; a wave holds RPL batch tiles of 64
//                     images (RPL rows per lane) that all sit on the SAME output pixel,
//                     so the zero-padding predicate of a filter tap is wave-uniform
//                     (a scalar branch) and the activation load of a tap is one
//                     coalesced run of 64*cw words.
//   workgroup       = 4 waves (4 different (pixel, batch-tile) rows) x one tile of 32
//                     output channels.  The weights of that channel tile are staged
//                     once in LDS as [k-chunk][32 channels][CH words]; every lane reads
//                     the same LDS address (broadcast ds_read_b128), so a weight word
//                     costs no VGPR traffic and no bank conflicts.
//   inner product   = v_xor_b32 + v_bcnt_u32_b32 (accumulating form): 2 VALU ops per
//                     32 +-1 multiply-accumulates.
//   epilogue        = in-lane: the lane owns all 32 channel sums of its row, so
//                     threshold -> bit -> shift/or builds the packed output word with
//                     no ballot, no LDS round trip and no atomics.  Pool windows are a
//                     sequential loop in the same lane (OR of the words), so every
//                     output word is written exactly once and re-runs are idempotent.
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

__device__ __forceinline__ int xpopc(uint4 a, uint4 w) {
    return __popc(a.x ^ w.x) + __popc(a.y ^ w.y) + __popc(a.z ^ w.z) + __popc(a.w ^ w.w);
}
__device__ __forceinline__ int xpopc(uint2 a, uint2 w) {
    return __popc(a.x ^ w.x) + __popc(a.y ^ w.y);
}
__device__ __forceinline__ int xpopc(uint32_t a, uint32_t w) { return __popc(a ^ w); }

template <int RPL, int CH>
__global__ __launch_bounds__(kThreads) void bgemm_popc_kernel(const BgemmParams p, int n_tiles,
                                                              int row_waves, int b_tiles) {
    using V = typename WordVec<CH>::type;
    __shared__ __attribute__((aligned(16))) uint32_t lds_w[kLdsWords];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nt = blockIdx.x % n_tiles;
    const int rw = (blockIdx.x / n_tiles) * kWavesPerBlock + wave;
    const bool active = rw < row_waves;

    const int cw_chunks = p.cw / CH;
    const int taps = p.R * p.S;
    const int nq = taps * cw_chunks;           // k-chunks in total
    const int kw_tot = taps * p.cw;            // words per weight row
    constexpr int kQB = kLdsWords / (kNTile * CH);  // chunks per staging block
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
        const int cnt = min(kQB, nq - q0);
        const int blk_words = cnt * CH;  // words per weight row in this block
        const uint32_t* wrow = p.wgt + (size_t)nt * kNTile * kw_tot + (size_t)q0 * CH;
        for (int idx = tid; idx < blk_words * kNTile; idx += kThreads) {
            const int n = idx / blk_words;
            const int kk = idx - n * blk_words;
            lds_w[((kk / CH) * kNTile + n) * CH + (kk % CH)] = wrow[(size_t)n * kw_tot + kk];
        }
    };

    if (single_block) {
        stage_weights(0);
        __syncthreads();
    }

    uint32_t outword[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) outword[r] = 0;

    const int pool_n = p.pool_h * p.pool_w;
    for (int pp = 0; pp < pool_n; ++pp) {
        const int y = oy * p.pool_h + pp / p.pool_w;
        const int x = ox * p.pool_w + pp % p.pool_w;
        const bool valid = active && y < p.PH && x < p.PW;  // wave-uniform
        const int ay0 = y * p.stride_h - p.pad_h;
        const int ax0 = x * p.stride_w - p.pad_w;

        int acc[RPL][kNTile];
#pragma unroll
        for (int r = 0; r < RPL; ++r)
#pragma unroll
            for (int n = 0; n < kNTile; ++n) acc[r][n] = 0;
        int exclude = 0;

        // running (tap row, tap col, chunk) counters: no integer division in the loop
        int tr = 0, ts = 0, kc = 0;
        for (int q0 = 0; q0 < nq; q0 += kQB) {
            if (!single_block) {
                __syncthreads();
                stage_weights(q0);
                __syncthreads();
            }
            const int cnt = min(kQB, nq - q0);
            for (int ql = 0; ql < cnt; ++ql) {
                const int ay = ay0 + tr, ax = ax0 + ts;
                const bool in_frame = ay >= 0 && ay < p.H && ax >= 0 && ax < p.W;
                if (valid) {
                    if (in_frame) {
                        V a[RPL];
                        const size_t pix = (size_t)(ay * p.W + ax) * p.B;
#pragma unroll
                        for (int r = 0; r < RPL; ++r)
                            a[r] = *reinterpret_cast<const V*>(p.act + (pix + bload[r]) * p.cw +
                                                               kc * CH);
                        const V* wl = reinterpret_cast<const V*>(lds_w) + ql * kNTile;
#pragma unroll
                        for (int n = 0; n < kNTile; ++n) {
                            const V w = wl[n];
#pragma unroll
                            for (int r = 0; r < RPL; ++r) acc[r][n] += xpopc(a[r], w);
                        }
                    } else if (kc == 0) {
                        ++exclude;
                    }
                }
                if (++kc == cw_chunks) {
                    kc = 0;
                    if (++ts == p.S) {
                        ts = 0;
                        ++tr;
                    }
                }
            }
        }

        if (!valid) continue;

        // ---------------- epilogue for pre-pool pixel (y, x) ----------------
        const int base = p.k_tap * taps - exclude * p.k_tap;
        const int n0 = nt * kNTile;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
            if (brow[r] >= p.B) continue;
            const int b = brow[r];
            int res[kNTile];
#pragma unroll
            for (int n = 0; n < kNTile; ++n) res[n] = base - 2 * acc[r][n];

            if (p.res_in != nullptr) {
#pragma unroll
                for (int n = 0; n < kNTile; ++n) {
                    const int ch = n0 + n;
                    if (ch < p.res_limit && ch < p.res_in_ch) {
                        int v;
                        if (p.res_pool) {
                            const int rw2 = 2 * p.PW;
                            v = INT_MIN;
#pragma unroll
                            for (int i = 0; i < 2; ++i)
#pragma unroll
                                for (int j = 0; j < 2; ++j)
                                    v = max(v, p.res_in[(((size_t)(2 * y + i) * rw2 + (2 * x + j)) *
                                                             p.B +
                                                         b) *
                                                            p.res_in_ch +
                                                        ch]);
                        } else {
                            v = p.res_in[(((size_t)y * p.PW + x) * p.B + b) * p.res_in_ch + ch];
                        }
                        res[n] += v;
                    }
                }
            }

            if (p.mode == EPI_THRESH) {
                uint32_t word = 0;
#pragma unroll
                for (int n = 0; n < kNTile; ++n) {
                    const int ch = n0 + n;
                    if (ch < p.N) {
                        const float rf = (float)res[n];
                        const float thr = p.bn[ch];
                        const bool bit = p.nan_bit ? !(rf < thr) : (rf >= thr);
                        word |= (bit ? 1u : 0u) << (31 - n);
                    }
                }
                outword[r] |= word;
                if (p.res_out != nullptr) {
                    int32_t* dst = p.res_out + (((size_t)y * p.PW + x) * p.B + b) * p.N;
#pragma unroll
                    for (int n = 0; n < kNTile; ++n)
                        if (n0 + n < p.N) dst[n0 + n] = res[n];
                }
            } else if (p.mode == EPI_AFFINE) {
                float* dst = p.out_f32 + (size_t)b * p.N;
#pragma unroll
                for (int n = 0; n < kNTile; ++n) {
                    const int ch = n0 + n;
                    if (ch < p.N) {
                        // (float)K - (float)c*2.0f is exact; multiply and add are kept
                        // separate (no FMA contraction) so the result is reproducible.
                        const float d = (float)p.k_tap - (float)acc[r][n] * 2.0f;
                        dst[ch] = __fadd_rn(__fmul_rn(d, p.bn_scale[ch]), p.bn_bias[ch]);
                    }
                }
            } else {  // EPI_RAW
                int32_t* dst = p.out_i32 + ((size_t)y * p.PW + x) * p.raw_pix_stride +
                               (size_t)b * p.raw_b_stride;
#pragma unroll
                for (int n = 0; n < kNTile; ++n)
                    if (n0 + n < p.N) dst[n0 + n] = res[n];
            }
        }
    }

    if (p.mode == EPI_THRESH && active) {
#pragma unroll
        for (int r = 0; r < RPL; ++r)
            if (brow[r] < p.B) {
                uint32_t* dst = p.out_bits + (size_t)opix * p.bits_pix_stride +
                                (size_t)brow[r] * p.bits_b_stride;
                dst[nt] = outword[r];
                if (nt == n_tiles - 1)  // zero the row's padding words
                    for (int w = n_tiles; w < p.bits_row_words; ++w) dst[w] = 0;
            }
    }
}

template <int RPL, int CH>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    const int n_tiles = (p.N + kNTile - 1) / kNTile;
    const int b_tiles = (p.B + 64 * RPL - 1) / (64 * RPL);
    const long long row_waves = (long long)p.OH * p.OW * b_tiles;
    const long long blocks = (row_waves + kWavesPerBlock - 1) / kWavesPerBlock * n_tiles;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return fail(TCBNN_EINVAL, "bgemm grid too large");
    hipLaunchKernelGGL((bgemm_popc_kernel<RPL, CH>), dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, p, n_tiles, (int)row_waves, b_tiles);
    TCBNN_LAUNCH_CHECK("bgemm_popc_kernel");
    return TCBNN_OK;
}

template <int CH>
int launch_r(const BgemmParams& p, hipStream_t stream) {
    // rows per lane: as many 64-image tiles of the batch as there are, up to 4
    if (p.B > 128) return launch_t<4, CH>(p, stream);
    if (p.B > 64) return launch_t<2, CH>(p, stream);
    return launch_t<1, CH>(p, stream);
}

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

int launch_bgemm_popc(const BgemmParams& p, hipStream_t stream) {
    if (int rc = validate_bgemm(p)) return rc;
    if (p.cw % 4 == 0) return launch_r<4>(p, stream);
    if (p.cw % 2 == 0) return launch_r<2>(p, stream);
    return launch_r<1>(p, stream);
}

}  // namespace tcbnn
