// Persistent FP4 matrix-core kernel for the 3x3 bit convolutions that carry almost all of a
// binarized ResNet / VGG / AlexNet (Conv128LayerFMT, kernel.cuh:676-827; Cin = 64, 128, 192, 256, 384
// or 512; un-pooled, or 2x2-pooled without residuals) and for the stand-alone 3x3 bit convolution
// with int32 output (BTC_Conv2d_balance, bmma_kernel.cu:101-165).
//
// Same operand mapping as bgemm_mfma.hip (MFMA "A" = 32 output channels, "B" = 32 images, a lane
// of the accumulator owns one image and 16 channels), plus what a short-K convolution needs to
// keep the matrix cores fed on a machine whose memory latency (~1 us) is longer than the whole
// K loop of one tile (9 taps x Cin = 576..4608 bits: 36..288 MFMAs):
//   - persistent workgroups: the FP4 weight fragments of a channel group (18..72 KiB, expanded from the
//     filter's words in fragment order) and its thresholds are staged in LDS ONCE, then every wave walks a
//     strided list of (pixel, 64-image) tiles; no barrier after the staging;
//   - whole-chunk register prefetch: all activation words a wave needs for the next chunk of
//     taps (the whole tile for Cin <= 128, one filter row above) are requested while the current
//     chunk is multiplied, across tile boundaries; for Cin <= 128 the requests are issued two per
//     k-step between the MFMAs of an interior tile (issued in one burst they hold the wave back);
//   - wave-uniform border handling: a tap outside the frame is a cleared bit in a scalar mask
//     (its loads and MFMAs are skipped), which is exactly the reference's "exclude" rule; pixel
//     columns are skewed by the row so that every wave gets its share of the slower border tiles;
//   - threshold folded into the accumulator: without a residual the accumulator starts from the
//     negated integer threshold (operand C of the tile's first MFMA, always the centre tap), so the
//     output bit is the sign of the finished accumulator;
//   - epilogue straight from the accumulator: one funnel shift per channel into a 16-channel half
//     word, one lane swap, 128-byte stores of the batch-innermost layouts; residual add / save as
//     contiguous 16-byte runs per lane.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <type_traits>

#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

using namespace mfma;

// Cache policy of the residual loads: the default one.  (With the stores below written through, a non-temporal
// hint on the loads costs 0.6 % of the ResNet-18 step at batch 256: 0.4641 -> 0.4611 ms over three runs each without
// it; before the stores were written through the hint had gained 2 %.)
constexpr int kResLoadAux = 0;
// Cache policy of the residual stores of full tiles with a narrow residual (the ResNet layers): written through
// (sc0 sc1).  The tensors are far larger than an XCD's L2 and are read one or two launches later, mostly by other
// XCDs: leaving them dirty in the writer's L2 only defers the write to the end of the launch.  Measured on ResNet-18
// at batch 256, three runs each: step 0.4640 -> 0.4590 ms (the residual launches 1-6 % shorter, the launches that
// read the tensors unchanged); non-temporal (nt) and agent scope (sc1) gave half of that.
constexpr int kResStoreAux = 0x11;
// ... and of the output words: written through as well (the next launch reads them from every XCD); another 0.5 % of
// that step (0.4633 -> 0.4610 ms, three runs each; non-temporal stores instead: 0.4693 ms).
constexpr int kBitsStoreAux = 0x11;
// Waves per workgroup: four, sharing the staged weights of their channel group; eight where the FP4 fragments of
// two channel tiles (18 KB per tile and 64 input channels) leave room for only one workgroup in a CU's 160 KB of
// LDS (Cin >= 384), and already at Cin = 256, where two four-wave workgroups would fit: the CU then still runs two
// waves per SIMD, each expanded activation fragment still feeds two MFMAs, the weights are staged once per CU
// instead of twice, and which waves share a SIMD is known (waves w and w + 4), which the numbering of the work
// items uses (ResNet-18 at batch 256: L3B2C1 14.6 -> 13.2 us, L3B1C2 17.1 -> 16.1 us).
constexpr int WIN_NONE = 0, WIN_ORPOOL = 1, WIN_MAXSAVE = 2;  // (see the kernel)
constexpr int waves_of(int spt, int nt, int win) {
    return win != WIN_MAXSAVE && 9 * spt * nt * 1024 > (nt == 2 ? 64 : 80) * 1024 ? 8 : 4;  // (WIN_MAXSAVE: a wave per pixel)
}
// WIN_MAXSAVE: where the four waves' sums of a window meet in LDS.  All channel tiles at once ([wave][NT][2][64]
// 128-bit words) where that leaves room for two workgroups per CU next to the staged weights; else one channel tile
// at a time ([3 other waves][2][64]: the wave that takes the tile's maximum keeps its own sums in registers), at the
// price of two more barriers per window.
constexpr bool win_two_phase(int spt, int nt) { return 9 * spt * nt * 1024 + nt * 128 + 4 * nt * 2 * 64 * 16 > 80 * 1024; }
constexpr int win_area_bytes(int spt, int nt) { return win_two_phase(spt, nt) ? 3 * 2 * 64 * 16 : 4 * nt * 2 * 64 * 16; }
// Residual mode of an instantiation.
constexpr int RM_NONE = 0;    // threshold only
constexpr int RM_PLAIN = 1;   // residual injected from a source of the same size and / or saved
constexpr int RM_POOLED = 2;  // residual injected as the 2x2 max of a source twice the size
constexpr int RM_RAW = 3;     // no threshold: the +-1 dot products are stored as int32 (tcbnn_bconv)

// RM_RAW: a wave's sums are transposed through a private LDS area of [32 images][32 NT + 4] words, so that every store
// writes whole contiguous channel runs, wherever that area leaves room for two workgroups in a CU's 160 KB of LDS
// next to the staged weights (9 SPT NT KB).  (The pitch, an odd multiple of 4 words, keeps both directions free of
// bank conflicts.)
constexpr int raw_pitch(int nt) { return 32 * nt + 4; }
constexpr bool raw_transposed(int spt, int rm, int nt, bool fullt) {
    return rm == RM_RAW && fullt && 9 * spt * nt * 1024 + 4 * 32 * raw_pitch(nt) * 4 <= 80 * 1024;
}

// Waves per SIMD the register allocator is asked to make room for (256 registers per lane: the plain layers
// use them for two image tiles and two channel tiles, the residual layers for operands in flight).
constexpr int kWavesPerSimd = 2;
// ... except where a fourth wave per SIMD is two registers away (one register spilled): Cin = 64 layers that save
// the window maximum
constexpr int waves_per_simd(int spt, int rm, int win) { return spt == 1 && rm == 1 && win == 2 ? 4 : kWavesPerSimd; }

// SPT = k-steps (64 bits) per filter tap = Cin / 64; MT = 32-image tiles per wave (2 for plain
// layers, 1 for residual layers); NT = 32-channel tiles per wave; RF = TCBNN_RES_* format of the
// injected residual (the narrower, the fewer registers hold it while it is in flight); WIN = what a wave does with
// the 2x2 windows of output pixels: WIN_NONE nothing (its work items are single pixels); WIN_ORPOOL = 2x2 OR-pooling
// of the output bits (kernel.cuh:797-816): a wave multiplies the four pixels of a window one after the other and
// stores the OR of their words once; WIN_MAXSAVE = the output bits are stored per pixel, but the saved residual is
// the element-wise maximum over the window, stored once per window: exactly what a consumer with residual_pool
// would compute from the full tensor (kernel.cuh:775-782), at a quarter of the bytes written and read.  A window is
// then the work item of a whole WORKGROUP: each of its four waves multiplies one of the window's pixels, the sums
// meet in LDS, and waves 0 .. NT-1 take the maximum of one channel tile each and store it (work items of one
// pixel tile instead of four: the layers that save such tensors have only one to four windows per wave).  FULLT = every 32-channel tile of the launch exists in full
// and, with an injected residual, lies entirely below or entirely above the channel limit: the per-channel
// tests of partial tiles are then not even compiled (they cost scalar registers and set-up instructions in
// every launch, and the networks' channel counts are multiples of 64).
template <int SPT, int RM, int MT, int NT, int RF, int WIN, bool FULLT>
__global__ __launch_bounds__(64 * waves_of(SPT, NT, WIN)) __attribute__((amdgpu_waves_per_eu(waves_per_simd(SPT, RM, WIN)))) void
conv3x3_mfma_f4_kernel(
    const BgemmParams p, const uint32_t* __restrict__ act, const uint32_t* __restrict__ wgt,
    const float* __restrict__ bnp, const int32_t* __restrict__ rin, int32_t* __restrict__ rout, int res_lim,
    int rout_fmt, unsigned act_bytes, unsigned rin_bytes, unsigned rout_bytes, unsigned bits_bytes,
    int n_groups, int b_groups, int pix_streams, int dy, int dx, int dxs) {
    constexpr bool kRes = RM == RM_PLAIN || RM == RM_POOLED;  // a residual is injected and / or saved
    constexpr bool POOL = WIN == WIN_ORPOOL, PSAVE = WIN == WIN_MAXSAVE, kWin = WIN != WIN_NONE;
    static_assert(RM == RM_NONE || !POOL, "residuals are defined for un-pooled layers only");
    static_assert(!PSAVE || (RM == RM_PLAIN && FULLT && (RF == TCBNN_RES_I16 || RF == TCBNN_RES_I12)),
                  "the window maximum is taken on 16-bit pairs in the epilogue of full tiles with a narrow injected residual");
    static_assert(!PSAVE || (MT == 1 && waves_of(SPT, NT, WIN) == 4), "one wave per pixel of the window, one image tile each");
    constexpr bool kTwoPhase = PSAVE && win_two_phase(SPT, NT);
    constexpr int TPC = SPT >= 3 ? 3 : 9;  // taps per prefetch chunk (a filter row, or all of it)
    constexpr int NCH = 9 / TPC;           // chunks per tile
    constexpr int NQ = 9 * SPT;            // k-steps per tile
    constexpr int kWaves = waves_of(SPT, NT, WIN);
    // A tile of one chunk is shorter than the memory latency: its residual operand is then
    // requested a whole tile ahead (double-buffered); otherwise with the tile's first chunk.
    constexpr bool kAhead = kRes && NCH == 1;
    extern __shared__ v4i lds_dyn[];
    v4i* lds_w = lds_dyn;  // [NQ][NT][64] fragments
    float* lds_thr = reinterpret_cast<float*>(lds_dyn + NQ * NT * 64);  // [NT*32]
    // RM_RAW with short K (the output-bound shapes): a wave's private [32 images][kRawPitch] int32 staging area, through
    // which a 32-image tile's sums are transposed so that every store writes whole contiguous channel runs
    constexpr bool kRawTranspose = raw_transposed(SPT, RM, NT, FULLT);
    constexpr int kRawPitch = raw_pitch(NT);
    int* lds_raw = reinterpret_cast<int*>(lds_thr + NT * 32);
    // WIN_MAXSAVE: where the four waves' sums of a window meet (pairs of int16; see win_two_phase)
    v4i* lds_win = reinterpret_cast<v4i*>(lds_thr + NT * 32);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int j = lane & 31;
    const int h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // The channel group is rotated by the workgroup's position, so that the workgroups an XCD receives
    // (every 8th) cover all channel groups, those that inject a residual and those that do not alike.
    // (grid = channel groups x image groups x pixel streams, launched in that order)
    const int bg = blockIdx.y;
    const int stream = blockIdx.z;
    const int ng = (blockIdx.x + bg + stream * b_groups) % n_groups;
    const int n0 = ng * (32 * NT);
    const int kw_tot = 9 * p.cw;

    // Kernel arguments that are only used further down are fetched now, together with the first ones: left to
    // the compiler, each is a scalar load placed right before its first use, i.e. one more exposed round trip
    // to memory in the set-up of every launch.
    auto fetch_now = [](auto v) __attribute__((always_inline)) { asm volatile("" ::"s"(v)); };
    fetch_now(p.out_bits);
    fetch_now(p.bits_pix_stride);
    fetch_now(p.bits_row_words);
    fetch_now(bnp);
    fetch_now(p.PH);
    fetch_now(p.OH);
    if constexpr (RM == RM_RAW) {
        fetch_now(p.raw_pix_stride);
        fetch_now(p.raw_b_stride);
    }

    // ---- the first requests of a workgroup: its channel group's thresholds and weight words.  The filter holds
    // the weight words in fragment order (64 consecutive words per fragment): all of a wave's words are requested
    // at once, here, before anything else is worked out, so that their latency runs during the set-up of the tile
    // loop; they are expanded to FP4 on the way into LDS further down (7 VALU instructions per fragment and lane,
    // once per workgroup; fetching fragments expanded at pack time moved four times the bytes and took longer).
    // (Thresholds requested after the weights had been stored were a second memory round trip in every launch.)
    constexpr int kStagePerWave = (9 * SPT * NT + kWaves - 1) / kWaves;
    float thr_stage = 0.0f;
    uint32_t wstage[kStagePerWave];
    {
        if (tid < NT * 32) thr_stage = RM != RM_RAW && (FULLT || n0 + tid < p.N) ? bnp[n0 + tid] : 0.0f;
        const uint32_t* __restrict__ fbits = wgt + (size_t)((p.N + 31) / 32) * 32 * kw_tot;
#pragma unroll
        for (int i = 0; i < kStagePerWave; ++i) {
            const int f = wave + i * kWaves;
            const int q = f / NT, nt = f % NT;
            // (the second channel tile of the last group may lie past the padded filter: nothing to read there)
            wstage[i] = f < 9 * SPT * NT && (FULLT || (ng * NT + nt) * 32 < p.N)
                            ? fbits[((size_t)(ng * NT + nt) * (9 * SPT) + q) * 64 + lane]
                            : 0u;
        }
    }

    // start values of a lane's 16 channels per channel tile (zeros when a residual is added first); filled once
    // the thresholds are staged
    v16f acc0[NT];

    // a wave's work items: output pixels, or 2x2 windows of them (row width `roww`)
    const int roww = kWin ? p.PW / 2 : p.PW;
    const int npix = kWin ? (p.PH / 2) * (p.PW / 2) : p.PH * p.PW;
    // First item of the wave (its later ones follow at stride dpi).  The items of the last, incomplete round go to
    // the waves with the lowest first item.  An eight-wave workgroup has a CU to itself, two waves per SIMD: its
    // waves 0-3 (one per SIMD) are numbered before the waves 4-7 of ANY workgroup, so that the left-over items fall
    // one to a SIMD over all CUs instead of two to a SIMD in the first CUs and none in the others.
    int pi = PSAVE ? stream  // (a window is taken by the whole workgroup)
                   : (kWaves == 8 ? (wave >> 2) * (pix_streams * 4) + stream * 4 + (wave & 3) : stream * kWaves + wave);
    const int dpi = PSAVE ? pix_streams : pix_streams * kWaves;
    // Item pi stands for row pi / roww and column (pi % roww + row) % roww.  The skew by the row keeps
    // a wave from staying in one column when its stride is a multiple of the row width (then the waves
    // that own a border column, whose tiles are slower, would finish long after the others).
    const int y = pi / roww, xr = pi % roww;
    // (dy = dpi / roww, dx = dpi % roww, dxs = (dx + dy) % roww come from the host)

    int bimg[MT], bload[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        bimg[mt] = (bg * MT + mt) * 32 + j;
        bload[mt] = min(bimg[mt], p.B - 1);
    }

    // Buffer addressing for every global access of the tile loop: a descriptor per tensor, one
    // per-lane byte offset (a constant of the lane) and a wave-uniform scalar offset per access, so
    // that addresses cost scalar adds only.  A lane that must not take part carries an offset beyond
    // every descriptor (the host checked the tensors are below 2 GiB): its load returns 0, its
    // store is dropped.
    constexpr unsigned kOutOfRange = 0x80000000u;
    auto make_rsrc = [](const void* ptr, unsigned bytes) __attribute__((always_inline)) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(ptr), 0, (int)bytes, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t r_act = make_rsrc(act, act_bytes), r_rin = make_rsrc(rin, rin_bytes),
                                 r_rout = make_rsrc(rout, rout_bytes), r_bits = make_rsrc(p.out_bits, bits_bytes);
    const unsigned row_b = (unsigned)p.B * 4u;  // bytes between consecutive words / channels of an image
    // RM_RAW: may a lane's 16 consecutive int32 outputs go out as 128-bit words?  (uniform)
    const bool raw_aligned = RM == RM_RAW && p.raw_pix_stride % 4 == 0 && p.raw_b_stride % 4 == 0 &&
                             (reinterpret_cast<uintptr_t>(rout) & 15) == 0;
    unsigned voff_act[MT], voff_bits[MT];  // activation loads; output words (stored by lanes 0-31)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        voff_act[mt] = ((unsigned)h * (unsigned)p.B + (unsigned)bload[mt]) * 4u;
        voff_bits[mt] = h == 0 && bimg[mt] < p.B ? (unsigned)bimg[mt] * 4u : kOutOfRange;
    }

    // The tile's first MFMA must belong to a tap that is never outside the frame (it brings in the
    // accumulator's start value): the centre tap.  Chunks of one filter row therefore come in the
    // order middle, top, bottom, and the taps of a chunk start with its middle one; the sums are
    // exact integers, so the order does not change them.
    auto chunk_row = [](int chunk) __attribute__((always_inline)) { return chunk == 0 ? 1 : (chunk == 1 ? 0 : 2); };
    // Requests the activation words of chunk `chunk` of the tile at pixel (yy, xx); returns the
    // wave-uniform mask of its in-frame taps.
    const unsigned pix_b = (unsigned)p.cw * row_b;        // bytes of one input pixel
    const unsigned pitch_b = (unsigned)p.W * pix_b;       // bytes of one input row
    constexpr uint32_t kAllTaps = (1u << TPC) - 1u;
    // Is every tap of the chunk inside the frame (the bulk of a layer)?  Then its loads need no
    // tests and one scalar add per tap: `soff` = offset of the chunk's first tap.
    auto chunk_interior = [&](int yy, int xx, int chunk, unsigned& soff) __attribute__((always_inline)) {
        const int ay0 = yy * p.stride_h - p.pad_h, ax0 = xx * p.stride_w - p.pad_w;
        const int r0 = TPC == 9 ? 0 : chunk_row(chunk), nr = TPC == 9 ? 3 : 1;  // filter rows of the chunk
        soff = (unsigned)((ay0 + r0) * p.W + ax0) * pix_b;  // uniform
        return ay0 + r0 >= 0 && ay0 + r0 + nr <= p.H && ax0 >= 0 && ax0 + 3 <= p.W;
    };
    // loads of k-step i (taps in raster order) of an interior chunk; moves `soff` on after a tap
    auto load_step = [&](uint32_t (*buf)[MT], int i, unsigned& soff) __attribute__((always_inline)) {
        const int tl = i / SPT, t = i % SPT;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            buf[i][mt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r_act, (int)voff_act[mt],
                                                                       (int)(soff + (unsigned)(2 * t) * row_b), 0);
        if (t == SPT - 1) soff += tl % 3 == 2 ? pitch_b - 2 * pix_b : pix_b;
    };
    auto load_chunk = [&](int yy, int xx, int chunk, uint32_t (*buf)[MT]) __attribute__((always_inline)) {
        const int ay0 = yy * p.stride_h - p.pad_h, ax0 = xx * p.stride_w - p.pad_w;
        const int r0 = TPC == 9 ? 0 : chunk_row(chunk);
        unsigned soff0;
        if (chunk_interior(yy, xx, chunk, soff0)) {
#pragma unroll
            for (int i = 0; i < TPC * SPT; ++i) load_step(buf, i, soff0);
            return kAllTaps;
        }
        uint32_t mask = 0;
#pragma unroll
        for (int tl = 0; tl < TPC; ++tl) {
            const int r = TPC == 9 ? tl / 3 : r0;
            const int s = tl % 3;
            const int ay = ay0 + r, ax = ax0 + s;
            if (ay >= 0 && ay < p.H && ax >= 0 && ax < p.W) {
                mask |= 1u << tl;
                const unsigned soff = (unsigned)(ay * p.W + ax) * pix_b;  // uniform
#pragma unroll
                for (int t = 0; t < SPT; ++t)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        buf[tl * SPT + t][mt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(
                            r_act, (int)voff_act[mt], (int)(soff + (unsigned)(2 * t) * row_b), 0);
            }
        }
        return mask;
    };

    v16f acc[MT][NT];

    // One k-step (64 input channels of one tap): the expanded activation words `bfrag` times the NT
    // weight fragments `a`.  FIRST: the accumulators start from acc0 instead of their old value.
    auto expand_step = [&](v4i* bfrag, const uint32_t* words) __attribute__((always_inline)) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) bfrag[mt] = expand_f4(words[mt]);
    };
    auto mma_frag = [&](auto first_tag, const v4i* a, const v4i* bfrag) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(first_tag)::value;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[mt][nt] = Acc<FMT_F4>::mma(a[nt], bfrag[mt], FIRST ? acc0[nt] : acc[mt][nt]);
    };
    auto mma_step = [&](auto first_tag, const v4i* a, const uint32_t* words) __attribute__((always_inline)) {
        v4i bfrag[MT];
        expand_step(bfrag, words);
        mma_frag(first_tag, a, bfrag);
    };
    auto load_a = [&](v4i* a, int q) __attribute__((always_inline)) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) a[nt] = lds_w[(q * NT + nt) * 64 + lane];
    };
    // Everything but LDS reads may be moved across this point by the instruction scheduler: the
    // fragment reads issued before it stay a whole k-step ahead of the MFMAs that use them.
    constexpr int kAllButDsRead = 0x07ff & ~0x0180;
    // order of the taps inside a chunk: the middle one first
    auto tap_of = [](int i) __attribute__((always_inline)) {
        return TPC == 9 ? (i == 0 ? 4 : (i <= 4 ? i - 1 : i)) : (i == 0 ? 1 : (i == 1 ? 0 : 2));
    };
    // For Cin <= 128, interior pixels (every tap of the chunk in the frame: the bulk of a layer) run one
    // straight-line block with the weight fragments of step i+1 read from LDS before step i is
    // multiplied; border pixels test each tap and read ahead inside a tap only.
    // LOADS: the words of the next chunk (interior as well) are requested two per step, in the shadow of
    // the MFMAs, instead of in one burst before the chunk.
    auto compute_chunk_as = [&](auto first_tag, auto loads_tag, int chunk, uint32_t (*buf)[MT], uint32_t mask,
                                uint32_t (*nbuf)[MT], unsigned nsoff) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(first_tag)::value;
        constexpr bool LOADS = decltype(loads_tag)::value;
        const int tap0 = TPC == 9 ? 0 : chunk_row(chunk) * 3;
        if (LOADS || (SPT <= 2 && mask == kAllTaps)) {
            constexpr int NS = TPC * SPT;
            auto q_of = [&](int i) __attribute__((always_inline)) { return (tap0 + tap_of(i / SPT)) * SPT + i % SPT; };
            // Software pipeline, one scheduling region per step (nothing moves across the region
            // boundaries): request the fragments and expand the activations of step i + 1, multiply
            // step i.
            auto words_of = [&](int i) __attribute__((always_inline)) { return buf[tap_of(i / SPT) * SPT + i % SPT]; };
            v4i a[2][NT], b[2][MT];
            load_a(a[0], q_of(0));
            expand_step(b[0], words_of(0));
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                if (i + 1 < NS) load_a(a[(i + 1) & 1], q_of(i + 1));
                if constexpr (LOADS) load_step(nbuf, i, nsoff);
                if (i + 1 < NS) expand_step(b[(i + 1) & 1], words_of(i + 1));
                const v4i* ai = a[i & 1];
                if (FIRST && i == 0)
                    mma_frag(std::true_type{}, ai, b[0]);
                else
                    mma_frag(std::false_type{}, ai, b[i & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < TPC; ++i) {
                const int tl = tap_of(i);
                if (!((mask >> tl) & 1u)) continue;  // wave-uniform; never the middle tap
                v4i a[2][NT];
                load_a(a[0], (tap0 + tl) * SPT);
#pragma unroll
                for (int t = 0; t < SPT; ++t) {
                    if (t + 1 < SPT) load_a(a[(t + 1) & 1], (tap0 + tl) * SPT + t + 1);
                    __builtin_amdgcn_sched_barrier(kAllButDsRead);
                    if (FIRST && i == 0 && t == 0)
                        mma_step(std::true_type{}, a[0], buf[tl * SPT + t]);
                    else
                        mma_step(std::false_type{}, a[t & 1], buf[tl * SPT + t]);
                }
            }
        }
    };
    auto compute_chunk = [&](int chunk, uint32_t (*buf)[MT], uint32_t mask, bool fused, uint32_t (*nbuf)[MT],
                             unsigned nsoff) __attribute__((always_inline)) {
        if constexpr (SPT <= 2) {
            if (fused) {  // uniform; NCH == 1: the chunk is a whole tile
                compute_chunk_as(std::true_type{}, std::true_type{}, chunk, buf, mask, nbuf, nsoff);
                return;
            }
        }
        if (NCH == 1 || chunk == 0)  // uniform: the tile starts here
            compute_chunk_as(std::true_type{}, std::false_type{}, chunk, buf, mask, nbuf, nsoff);
        else
            compute_chunk_as(std::false_type{}, std::false_type{}, chunk, buf, mask, nbuf, nsoff);
    };

    // ---- residual operand (kernel.cuh:770-794).  A lane owns channels n0 + 32 nt + 16 h + v of
    // images bload[mt] (slot mt * NT + nt); every load is a wave-uniform base plus a per-lane offset.
    // A lane's 16 values arrive as 16 (int32) or 8 (int16 pairs) words; a plain operand stays in
    // that raw form until its epilogue, a pooled one is reduced to 16 ints by finish_residual.
    constexpr int NRV = kRes ? MT * NT : 1;
    constexpr int NTMP = RM == RM_POOLED ? 3 : 1;
    constexpr bool R16 = RF == TCBNN_RES_I16, R12 = RF == TCBNN_RES_I12;  // format of the injected tensor
    // Narrow injected residual on full tiles: the sum, the residual and the threshold meet as floats that carry
    // small integers on top of 1.5 * 2^23 (kMagicBits), where the float's bit pattern IS 0x4B400000 + integer:
    //   the accumulators start from 1.5 * 2^23, so the finished one is such a float (exact: every partial sum is an
    //   integer below 2^24), and adding the residual is ONE integer add on its bit pattern (no conversions),
    //   its low 16 (or 12) bits are the two's complement value to store (no conversion, no subtraction),
    //   minus (1.5 * 2^23 + ceil(threshold)) has the sign the output bit needs.
    // The layers this serves are bound by instruction issue (the matrix pipeline and the VALU of a SIMD do not
    // overlap): 4.5 to 6.5 VALU instructions per value instead of 9.
    constexpr bool kMagic = kRes && FULLT && (R16 || R12);
    constexpr uint32_t kMagicBits = 0x4B400000u;  // 12582912.0f
    constexpr int NRAW = R12 ? 6 : (R16 ? 8 : 16);        // words loaded per channel tile
    constexpr bool kPackedMax = RM == RM_POOLED && R16 && kMagic;  // 2x2 maximum taken on the packed 16-bit pairs
    constexpr int NW = RM == RM_POOLED && !kPackedMax ? 16 : NRAW;  // words kept per channel tile
    int tmp[NTMP][NRV][NRAW];  // pooled: the other three pixels of the 2x2 window
    // A lane's 16 channels are 4 groups of 4 (int32) or 2 groups of 8 (int16), 16 bytes each, or one 12-bit group
    // of 24 bytes (a 16-byte piece in the group's first plane, an 8-byte piece in its second).
    unsigned lane_off[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        lane_off[mt] = R12 ? (unsigned)h * (unsigned)p.B * 24u + (unsigned)bload[mt] * 16u
                           : ((unsigned)((R16 ? 2 : 4) * h) * (unsigned)p.B + (unsigned)bload[mt]) * 16u;
    const unsigned grp_b = (unsigned)p.B * 16u;  // bytes between consecutive channel groups (32- and 16-bit formats)
    const unsigned g12_b = (unsigned)p.B * 24u;  // bytes of a 12-bit group of 16 channels

    auto request_residual = [&](int yy, int xx, int (*rv)[NW]) __attribute__((always_inline)) {
        if constexpr (kRes) {
            constexpr bool i16 = R16;
            // bytes per source pixel; per-lane offset; 128-bit loads per channel tile.  Groups past the
            // source's channels read the neighbouring pixel or (at the end of the tensor) zeros; their
            // values are cleared by finish_residual.
            const unsigned ch_b = (unsigned)(i16 ? (p.res_in_ch + 7) / 8 : (p.res_in_ch + 3) / 4) * grp_b;
            constexpr int nld = i16 ? 2 : 4;
            const unsigned pix = RM == RM_POOLED ? (unsigned)(2 * yy) * (unsigned)(2 * p.PW) + (unsigned)(2 * xx)
                                                 : (unsigned)yy * (unsigned)p.PW + (unsigned)xx;
            const unsigned ddy = (unsigned)(2 * p.PW) * ch_b;
#pragma unroll
            for (int sl = 0; sl < MT * NT; ++sl) {
                const int nt = sl % NT;
                const int cb = n0 + nt * 32;
                // a channel tile that receives no residual (uniform) reads zeros through an out-of-range
                // offset: no branch, no memory traffic
                const unsigned loff = cb < res_lim ? lane_off[sl / NT] : kOutOfRange;
                if constexpr (R12) {
                    // the lane's group: 16 bytes in its first plane, 8 in its second (B * 16 bytes further on, at half
                    // the per-image pitch); same out-of-range trick for tiles that receive nothing
                    const unsigned pb = (unsigned)((p.res_in_ch + 15) / 16) * g12_b;  // bytes per source pixel
                    const unsigned b0 = pix * pb + (unsigned)(cb / 16) * g12_b;       // uniform
                    const unsigned loff2 = cb < res_lim ? (unsigned)h * g12_b + grp_b + (unsigned)bload[sl / NT] * 8u : kOutOfRange;
                    auto fetch = [&](unsigned so, int* dst) __attribute__((always_inline)) {
                        const v4i a = __builtin_amdgcn_raw_buffer_load_b128(r_rin, (int)loff, (int)so, kResLoadAux);
                        const auto c2 = __builtin_amdgcn_raw_buffer_load_b64(r_rin, (int)loff2, (int)so, kResLoadAux);
                        dst[0] = a[0], dst[1] = a[1], dst[2] = a[2], dst[3] = a[3], dst[4] = c2[0], dst[5] = c2[1];
                    };
                    fetch(b0, rv[sl]);
                    if constexpr (RM == RM_POOLED) {
                        const unsigned dd = (unsigned)(2 * p.PW) * pb;
                        fetch(b0 + pb, tmp[0][sl]);
                        fetch(b0 + dd, tmp[1][sl]);
                        fetch(b0 + dd + pb, tmp[2][sl]);
                    }
                    continue;
                }
                const unsigned base = pix * ch_b + (unsigned)(i16 ? cb / 8 : cb / 4) * grp_b;  // uniform
#pragma unroll
                for (int g = 0; g < nld; ++g) {
                    const unsigned so = base + (unsigned)g * grp_b;
                    const v4i q0 = __builtin_amdgcn_raw_buffer_load_b128(r_rin, (int)loff, (int)so, kResLoadAux);
#pragma unroll
                    for (int k = 0; k < 4; ++k) rv[sl][4 * g + k] = q0[k];
                    if constexpr (RM == RM_POOLED) {
                        const v4i q1 = __builtin_amdgcn_raw_buffer_load_b128(r_rin, (int)loff, (int)(so + ch_b), kResLoadAux);
                        const v4i q2 = __builtin_amdgcn_raw_buffer_load_b128(r_rin, (int)loff, (int)(so + ddy), kResLoadAux);
                        const v4i q3 = __builtin_amdgcn_raw_buffer_load_b128(r_rin, (int)loff, (int)(so + ddy + ch_b), kResLoadAux);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            tmp[0][sl][4 * g + k] = q1[k];
                            tmp[1][sl][4 * g + k] = q2[k];
                            tmp[2][sl][4 * g + k] = q3[k];
                        }
                    }
                }
            }
        }
    };
    // Pooled source: 2x2 maximum of the four pixels, one int per channel (16-bit pairs unpacked).
    auto finish_residual = [&](int (*rv)[NW]) __attribute__((always_inline)) {
        if constexpr (RM == RM_POOLED) {
#pragma unroll
            for (int nt = 0; nt < MT * NT; ++nt) {  // every (image tile, channel tile) slot
                if constexpr (R12) {
                    int m[16], t[16];
                    i12_unpack8((uint32_t)rv[nt][0], (uint32_t)rv[nt][1], (uint32_t)rv[nt][2], m);
                    i12_unpack8((uint32_t)rv[nt][3], (uint32_t)rv[nt][4], (uint32_t)rv[nt][5], m + 8);
#pragma unroll
                    for (int k = 0; k < 3; ++k) {
                        i12_unpack8((uint32_t)tmp[k][nt][0], (uint32_t)tmp[k][nt][1], (uint32_t)tmp[k][nt][2], t);
                        i12_unpack8((uint32_t)tmp[k][nt][3], (uint32_t)tmp[k][nt][4], (uint32_t)tmp[k][nt][5], t + 8);
#pragma unroll
                        for (int v = 0; v < 16; ++v) m[v] = max(m[v], t[v]);
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) rv[nt][v] = m[v];
                } else if constexpr (kPackedMax) {
                    typedef short s2_t __attribute__((ext_vector_type(2)));
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        s2_t m = __builtin_bit_cast(s2_t, rv[nt][k]);
#pragma unroll
                        for (int t = 0; t < 3; ++t) m = __builtin_elementwise_max(m, __builtin_bit_cast(s2_t, tmp[t][nt][k]));
                        rv[nt][k] = __builtin_bit_cast(int, m);
                    }
                } else if constexpr (R16) {
#pragma unroll
                    for (int k = 7; k >= 0; --k) {  // downwards: slot k is read before 2k, 2k+1 are written
                        const int w = rv[nt][k];
                        int lo = (int)(short)(w & 0xffff), hi = w >> 16;
#pragma unroll
                        for (int t = 0; t < 3; ++t) {
                            const int wt = tmp[t][nt][k];
                            lo = max(lo, (int)(short)(wt & 0xffff));
                            hi = max(hi, wt >> 16);
                        }
                        rv[nt][2 * k] = lo;
                        rv[nt][2 * k + 1] = hi;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        rv[nt][v] = max(max(rv[nt][v], tmp[0][nt][v]), max(tmp[1][nt][v], tmp[2][nt][v]));
                }
            }
        }
    };

    // One channel tile of the epilogue.  FAST (wave-uniform choice): all 32 channels exist and, with a
    // residual, all of them receive it, so no per-channel condition is evaluated at all.
    uint32_t poolw[MT][NT];  // POOL: OR of the window's words so far
    uint32_t prw[kTwoPhase ? NT : 1][8];  // WIN_MAXSAVE, one channel tile at a time: this pixel's sums until their turn
    auto epilogue_tile = [&](auto fast_tag, int nt, unsigned pix, unsigned bits_pix, int (*rv)[NW],
                             int sub) __attribute__((always_inline)) {
        constexpr bool FAST = decltype(fast_tag)::value;
        const int cbase = n0 + nt * 32 + 16 * h;  // this lane's channels: cbase + v
        float thr[16];
        if constexpr (kRes) {
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
        if constexpr (RM == RM_RAW) {
            // int32 dot products, out_i32[pix * raw_pix_stride + b * raw_b_stride + channel]: a lane's 16
            // channels are consecutive, stored as four 128-bit words (single words for a partial tile or an
            // unaligned run); the kernel's `rout` descriptor covers this tensor
            const unsigned so = (pix * (unsigned)p.raw_pix_stride + (unsigned)(n0 + nt * 32)) * 4u;  // uniform
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const unsigned vo = bimg[mt] < p.B ? ((unsigned)bimg[mt] * (unsigned)p.raw_b_stride + 16u * (unsigned)h) * 4u
                                                   : kOutOfRange;
                if (FAST && raw_aligned) {
                    v4i q[4];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        q[g] = v4i{(int)acc[mt][nt][4 * g], (int)acc[mt][nt][4 * g + 1], (int)acc[mt][nt][4 * g + 2],
                                   (int)acc[mt][nt][4 * g + 3]};
                        __builtin_amdgcn_raw_buffer_store_b128(q[g], r_rout, (int)vo, (int)(so + 16u * (unsigned)g), 0);
                    }
                    asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]));  // see the residual stores
                    __builtin_amdgcn_sched_barrier(0);
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        __builtin_amdgcn_raw_buffer_store_b32((int)acc[mt][nt][v], r_rout,
                                                              (int)(cbase + v < p.N ? vo : kOutOfRange),
                                                              (int)(so + 4u * (unsigned)v), 0);
                }
            }
            return;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int b = bimg[mt];
            const bool b_ok = b < p.B;
            uint32_t hw = 0;
            if constexpr (kMagic && FAST) {
                // The accumulators started from 1.5 * 2^23 (acc0), so their bit patterns are 0x4B400000 + sum: the
                // residual is added to the PATTERN with an integer add, and the result is again such a float.
                uint32_t tb[16];
                const int* w = rv[mt * NT + nt];
                if constexpr (R12 && RM == RM_PLAIN) {  // still packed: six words
                    int un[16];
                    i12_unpack8((uint32_t)w[0], (uint32_t)w[1], (uint32_t)w[2], un);
                    i12_unpack8((uint32_t)w[3], (uint32_t)w[4], (uint32_t)w[5], un + 8);
#pragma unroll
                    for (int v = 0; v < 16; ++v) tb[v] = __float_as_uint(acc[mt][nt][v]) + (uint32_t)un[v];
                } else if constexpr (R12 || !kPackedMax && RM == RM_POOLED) {  // sixteen ints (2x2 maximum taken)
#pragma unroll
                    for (int v = 0; v < 16; ++v) tb[v] = __float_as_uint(acc[mt][nt][v]) + (uint32_t)w[v];
                } else {  // eight words of two int16 (plain, or the packed 2x2 maximum)
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        tb[2 * k] = __float_as_uint(acc[mt][nt][2 * k]) + (uint32_t)(int)(short)(w[k] & 0xffff);
                        tb[2 * k + 1] = __float_as_uint(acc[mt][nt][2 * k + 1]) + (uint32_t)(w[k] >> 16);
                    }
                }
                float t[16];  // 1.5 * 2^23 + (sum + residual)
#pragma unroll
                for (int v = 0; v < 16; ++v) t[v] = __uint_as_float(tb[v]);
                if constexpr (PSAVE) {
                    // Only the window's maximum is saved.  The low 16 bits of a bit pattern are the sum as int16 (the
                    // host admits this instantiation only for 12- and 16-bit outputs): two sums per word, handed to the
                    // wave that takes this channel tile's maximum (window_maximum below).
                    uint32_t pr[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        pr[k] = __builtin_amdgcn_perm(__float_as_uint(t[2 * k + 1]), __float_as_uint(t[2 * k]), 0x05040100u);
                    if constexpr (kTwoPhase) {
#pragma unroll
                        for (int k = 0; k < 8; ++k) prw[nt][k] = pr[k];
                    } else {
                        v4i* x = lds_win + ((wave * NT + nt) * 2) * 64 + lane;
                        x[0] = v4i{(int)pr[0], (int)pr[1], (int)pr[2], (int)pr[3]};
                        x[64] = v4i{(int)pr[4], (int)pr[5], (int)pr[6], (int)pr[7]};
                    }
                } else if (rout != nullptr) {
                    // the value to store is in the low bits of t's bit pattern (see the 128-bit store note below)
                    v4i q[4];
                    if (rout_fmt == TCBNN_RES_I12) {
                        int tb[16];
#pragma unroll
                        for (int v = 0; v < 16; ++v) tb[v] = (int)__float_as_uint(t[v]);
                        uint32_t d[6];
                        i12_pack8(tb, d[0], d[1], d[2]);
                        i12_pack8(tb + 8, d[3], d[4], d[5]);
                        const unsigned so = (pix * (unsigned)((p.N + 15) / 16) + (unsigned)((n0 + nt * 32) / 16)) * g12_b;
                        const unsigned vo = b_ok ? (unsigned)h * g12_b + (unsigned)b * 16u : kOutOfRange;
                        const unsigned vo2 = b_ok ? (unsigned)h * g12_b + grp_b + (unsigned)b * 8u : kOutOfRange;
                        q[0] = v4i{(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
                        typedef int v2i_t __attribute__((ext_vector_type(2)));
                        const v2i_t q2 = {(int)d[4], (int)d[5]};
                        __builtin_amdgcn_raw_buffer_store_b128(q[0], r_rout, (int)vo, (int)so, kResStoreAux);
                        __builtin_amdgcn_raw_buffer_store_b64(q2, r_rout, (int)vo2, (int)so, kResStoreAux);
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q2));
                    } else if (rout_fmt == TCBNN_RES_I16) {
                        const unsigned so = (pix * (unsigned)((p.N + 7) / 8) + (unsigned)((n0 + nt * 32) / 8)) * grp_b;
                        const unsigned vo = b_ok ? ((unsigned)(2 * h) * (unsigned)p.B + (unsigned)b) * 16u : kOutOfRange;
#pragma unroll
                        for (int g = 0; g < 2; ++g) {
#pragma unroll
                            for (int k = 0; k < 4; ++k)  // the low halves of two bit patterns: one byte permute
                                q[g][k] = (int)__builtin_amdgcn_perm(__float_as_uint(t[8 * g + 2 * k + 1]),
                                                                     __float_as_uint(t[8 * g + 2 * k]), 0x05040100u);
                            __builtin_amdgcn_raw_buffer_store_b128(q[g], r_rout, (int)vo, (int)(so + (unsigned)g * grp_b), kResStoreAux);
                        }
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]));
                    } else {
                        const unsigned so = (pix * (unsigned)((p.N + 3) / 4) + (unsigned)((n0 + nt * 32) / 4)) * grp_b;
                        const unsigned vo = b_ok ? ((unsigned)(4 * h) * (unsigned)p.B + (unsigned)b) * 16u : kOutOfRange;
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
#pragma unroll
                            for (int k = 0; k < 4; ++k) q[g][k] = (int)(__float_as_uint(t[4 * g + k]) - kMagicBits);
                            __builtin_amdgcn_raw_buffer_store_b128(q[g], r_rout, (int)vo, (int)(so + (unsigned)g * grp_b), kResStoreAux);
                        }
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]));
                    }
                }
                // bit = !(sum + residual < threshold): the inverted sign of t - (1.5 * 2^23 + ceil(threshold))
#pragma unroll
                for (int v = 0; v < 16; ++v) hw = __builtin_amdgcn_alignbit(hw, __float_as_uint(t[v] - thr[v]), 31);
                hw = ~hw & 0xffffu;
            } else if constexpr (kRes) {
                int res[16];
                int un[16];  // a plain 12-bit operand is still packed: six words -> sixteen values
                if constexpr (RM == RM_PLAIN && R12) {
                    const int* w = rv[mt * NT + nt];
                    i12_unpack8((uint32_t)w[0], (uint32_t)w[1], (uint32_t)w[2], un);
                    i12_unpack8((uint32_t)w[3], (uint32_t)w[4], (uint32_t)w[5], un + 8);
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int val;
                    if constexpr (RM == RM_PLAIN && R12) {
                        val = un[v];
                    } else if constexpr (RM == RM_PLAIN && R16) {
                        const int w = rv[mt * NT + nt][v >> 1];
                        val = (v & 1) ? (w >> 16) : (int)(short)(w & 0xffff);
                    } else {
                        val = rv[mt * NT + nt][v];
                    }
                    if constexpr (!FAST) {
                        if (cbase + v >= res_lim) val = 0;
                    }
                    res[v] = (int)acc[mt][nt][v] + val;
                }
                if (rout != nullptr) {
                    if constexpr (!FAST) {  // channels past N are stored as 0 inside a group
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (cbase + v >= p.N) res[v] = 0;
                    }
                    // 128-bit buffer stores.  On this hardware a buffer store of more than 64 bits still reads
                    // its data registers after issue even when its scalar offset comes from an SGPR; the
                    // compiler assumes that form is safe and lets the very next VALU instruction overwrite
                    // them (seen as rare wrong first words in lanes 12-15 of each 16).  The data vectors are
                    // therefore kept alive, by the empty-but-for-wait-states asm below, until well after the
                    // last store has issued.
                    v4i q[4];
                    if (rout_fmt == TCBNN_RES_I12) {  // the lane's 16 channels are one group: 16 + 8 bytes
                        uint32_t d[6];
                        i12_pack8(res, d[0], d[1], d[2]);
                        i12_pack8(res + 8, d[3], d[4], d[5]);
                        const unsigned so = (pix * (unsigned)((p.N + 15) / 16) + (unsigned)((n0 + nt * 32) / 16)) * g12_b;
                        const bool wr = b_ok && (FAST || cbase < p.N);  // a group that starts past N is not written
                        const unsigned vo = wr ? (unsigned)h * g12_b + (unsigned)b * 16u : kOutOfRange;
                        const unsigned vo2 = wr ? (unsigned)h * g12_b + grp_b + (unsigned)b * 8u : kOutOfRange;
                        q[0] = v4i{(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
                        typedef int v2i_t __attribute__((ext_vector_type(2)));
                        const v2i_t q2 = {(int)d[4], (int)d[5]};
                        __builtin_amdgcn_raw_buffer_store_b128(q[0], r_rout, (int)vo, (int)so, 0);
                        __builtin_amdgcn_raw_buffer_store_b64(q2, r_rout, (int)vo2, (int)so, 0);
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q2));
                    } else if (rout_fmt == TCBNN_RES_I16) {  // groups of 8 channels, two per word
                        const unsigned so = (pix * (unsigned)((p.N + 7) / 8) + (unsigned)((n0 + nt * 32) / 8)) * grp_b;
                        const unsigned vo = b_ok ? ((unsigned)(2 * h) * (unsigned)p.B + (unsigned)b) * 16u : kOutOfRange;
#pragma unroll
                        for (int g = 0; g < 2; ++g) {
#pragma unroll
                            for (int k = 0; k < 4; ++k)
                                q[g][k] = (res[8 * g + 2 * k] & 0xffff) | (res[8 * g + 2 * k + 1] << 16);
                            // a group that starts past N belongs to the next pixel: not written
                            __builtin_amdgcn_raw_buffer_store_b128(
                                q[g], r_rout, (int)(FAST || cbase + 8 * g < p.N ? vo : kOutOfRange),
                                (int)(so + (unsigned)g * grp_b), 0);
                        }
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]));
                    } else {
                        const unsigned so = (pix * (unsigned)((p.N + 3) / 4) + (unsigned)((n0 + nt * 32) / 4)) * grp_b;
                        const unsigned vo = b_ok ? ((unsigned)(4 * h) * (unsigned)p.B + (unsigned)b) * 16u : kOutOfRange;
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            q[g] = v4i{res[4 * g], res[4 * g + 1], res[4 * g + 2], res[4 * g + 3]};
                            __builtin_amdgcn_raw_buffer_store_b128(
                                q[g], r_rout, (int)(FAST || cbase + 4 * g < p.N ? vo : kOutOfRange),
                                (int)(so + (unsigned)g * grp_b), 0);
                        }
                        asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]));
                    }
                }
                if constexpr (FAST) {
                    // bit = !(res < thr) = inverted sign of res - thr (never -0: equal operands give +0);
                    // one subtract and one funnel shift per channel
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        hw = __builtin_amdgcn_alignbit(hw, __float_as_uint((float)res[v] - thr[v]), 31);
                    hw = ~hw & 0xffffu;
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const uint32_t bit = (cbase + v < p.N && !((float)res[v] < thr[v])) ? 1u : 0u;
                        hw = hw + hw + bit;
                    }
                }
            } else {
                // the accumulator is the exact integer sum minus the integer threshold (never -0):
                // its sign is the inverted bit
                if constexpr (FAST) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        hw = __builtin_amdgcn_alignbit(hw, __float_as_uint(acc[mt][nt][v]), 31);
                    hw = ~hw & 0xffffu;
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const uint32_t bit = (cbase + v < p.N && !(acc[mt][nt][v] < 0.0f)) ? 1u : 0u;
                        hw = hw + hw + bit;
                    }
                }
            }
            // the half word of lane + 32 (only the lower 32 lanes store a word): lanes 0-31 of the
            // second result are lanes 32-63 of the first operand; one VALU op, no LDS round trip
            const uint32_t other = __builtin_amdgcn_permlane32_swap(hw, hw, false, false)[1];
            uint32_t word = (hw << 16) | other;
            if constexpr (POOL) {
                word |= sub == 0 ? 0u : poolw[mt][nt];
                poolw[mt][nt] = word;
                if (sub != 3) continue;  // uniform: the window is not complete yet
            }
            const int w = ng * NT + nt;
            if (FULLT || w < p.bits_row_words)  // uniform; with full tiles every word of the group exists
                __builtin_amdgcn_raw_buffer_store_b32((int)word, r_bits, (int)voff_bits[mt],
                                                      (int)(bits_pix + (unsigned)w * row_b), kBitsStoreAux);
        }
    };

    // int32 output [N][P][Q][O] (bmma_kernel.cu:247-263): for one image and pixel the wave's 32 NT channels are one
    // contiguous run, but in the accumulator a lane holds 16 channels of ONE image, so a direct store scatters
    // 16-byte pieces over 64 different rows per instruction.  The sums of a 32-image tile go through the wave's LDS
    // area instead (row = image, conflict-free both ways) and leave as 128-bit stores in which 8 NT consecutive lanes
    // cover one image's whole run (4 runs of 256 bytes or 8 runs of 128 bytes per instruction).
    auto epilogue_raw_transposed = [&](unsigned pix) __attribute__((always_inline)) {
        if constexpr (kRawTranspose) {
            int* mine = lds_raw + wave * (32 * kRawPitch);
            constexpr int kCols = 8 * NT, kRows = 64 / kCols;  // 16-byte columns of a run; images per store instruction
            const int rl = lane / kCols, cl = lane % kCols;
            const unsigned so0 = (pix * (unsigned)p.raw_pix_stride + (unsigned)n0) * 4u;  // uniform
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        *reinterpret_cast<v4i*>(mine + j * kRawPitch + nt * 32 + 16 * h + 4 * g) =
                            v4i{(int)acc[mt][nt][4 * g], (int)acc[mt][nt][4 * g + 1], (int)acc[mt][nt][4 * g + 2],
                                (int)acc[mt][nt][4 * g + 3]};
                        __builtin_amdgcn_sched_barrier(0);  // convert and write four at a time (registers)
                    }
                // (same wave writes and reads: program order and the wait for LDS are all the synchronisation)
                const int img0 = (bg * MT + mt) * 32;
                // four store instructions at a time: eight would not fit the register file next to the activation buffers
#pragma unroll
                for (int part = 0; part < 32 / (4 * kRows); ++part) {
                    v4i q[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        q[k] = *reinterpret_cast<const v4i*>(mine + ((4 * part + k) * kRows + rl) * kRawPitch + 4 * cl);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int img = img0 + (4 * part + k) * kRows + rl;
                        const unsigned vo = img < p.B ? ((unsigned)img * (unsigned)p.raw_b_stride + 4u * (unsigned)cl) * 4u : kOutOfRange;
                        __builtin_amdgcn_raw_buffer_store_b128(q[k], r_rout, (int)vo, (int)so0, 0);
                    }
                    asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]));  // see the residual stores
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    // WIN_MAXSAVE, waves 0 .. NT-1 after the workgroup's barrier: the element-wise maximum of the four pixels' sums
    // of channel tile `nt` (packed 16-bit maxima on the pairs), stored in the tensor's 12- or 16-bit format at
    // window `pix` of the pooled tensor.  A lane reads what the same lane of each wave wrote: its own image and channels.
    auto window_maximum = [&](int nt, unsigned pix) __attribute__((always_inline)) {
        if constexpr (PSAVE) {
            typedef short s2_t __attribute__((ext_vector_type(2)));
            uint32_t wm[8];
            if constexpr (kTwoPhase) {
#pragma unroll
                for (int k = 0; k < 8; ++k) wm[k] = prw[nt][k];  // (this wave's own pixel)
            }
#pragma unroll
            for (int w = 0; w < (kTwoPhase ? 3 : 4); ++w) {
                const v4i* x = lds_win + (kTwoPhase ? w * 2 : (w * NT + nt) * 2) * 64 + lane;
                const v4i lo = x[0], hi = x[64];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const uint32_t pr = (uint32_t)(k < 4 ? lo[k] : hi[k - 4]);
                    wm[k] = !kTwoPhase && w == 0
                                ? pr
                                : __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s2_t, wm[k]),
                                                                                         __builtin_bit_cast(s2_t, pr)));
                }
            }
            const int b = bimg[0];
            const bool b_ok = b < p.B;
            v4i q[2];
            if (rout_fmt == TCBNN_RES_I12) {
                int un[16];
#pragma unroll
                for (int k = 0; k < 8; ++k) un[2 * k] = (int)wm[k], un[2 * k + 1] = (int)(wm[k] >> 16);
                uint32_t d[6];
                i12_pack8(un, d[0], d[1], d[2]);
                i12_pack8(un + 8, d[3], d[4], d[5]);
                const unsigned so = (pix * (unsigned)((p.N + 15) / 16) + (unsigned)((n0 + nt * 32) / 16)) * g12_b;
                const unsigned vo = b_ok ? (unsigned)h * g12_b + (unsigned)b * 16u : kOutOfRange;
                const unsigned vo2 = b_ok ? (unsigned)h * g12_b + grp_b + (unsigned)b * 8u : kOutOfRange;
                q[0] = v4i{(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
                typedef int v2i_t __attribute__((ext_vector_type(2)));
                const v2i_t q2 = {(int)d[4], (int)d[5]};
                __builtin_amdgcn_raw_buffer_store_b128(q[0], r_rout, (int)vo, (int)so, kResStoreAux);
                __builtin_amdgcn_raw_buffer_store_b64(q2, r_rout, (int)vo2, (int)so, kResStoreAux);
                asm volatile("s_nop 4" ::"v"(q[0]), "v"(q2));  // see the 128-bit store note in epilogue_tile
            } else {  // TCBNN_RES_I16
                const unsigned so = (pix * (unsigned)((p.N + 7) / 8) + (unsigned)((n0 + nt * 32) / 8)) * grp_b;
                const unsigned vo = b_ok ? ((unsigned)(2 * h) * (unsigned)p.B + (unsigned)b) * 16u : kOutOfRange;
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    q[g] = v4i{(int)wm[4 * g], (int)wm[4 * g + 1], (int)wm[4 * g + 2], (int)wm[4 * g + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(q[g], r_rout, (int)vo, (int)(so + (unsigned)g * grp_b), kResStoreAux);
                }
                asm volatile("s_nop 4" ::"v"(q[0]), "v"(q[1]));
            }
        }
    };

    // (yy, xx): the output pixel, or the window when pooled (sub = pixel of the window, 3 = last)
    // PSAVE: the bits belong to the window's pixel `sub` (this wave's), the saved residual to the window
    auto epilogue = [&](int yy, int xx, int sub, int (*rv)[NW]) __attribute__((always_inline)) {
        const unsigned pix = (unsigned)yy * (unsigned)roww + (unsigned)xx;
        // PSAVE: the previous window's maxima have been read (every wave of the workgroup runs the same sequence of
        // windows, so the barriers match; plain s_barrier: no wait for the global requests in flight)
        if constexpr (PSAVE) asm volatile("s_barrier" ::: "memory");
        const unsigned bpix = PSAVE ? (unsigned)(2 * yy + (sub >> 1)) * (unsigned)p.PW + (unsigned)(2 * xx + (sub & 1)) : pix;
        const unsigned bits_pix = bpix * (unsigned)p.bits_pix_stride * 4u;  // uniform
        if constexpr (kRawTranspose) {  // (the host only picks this instantiation for 16-byte aligned outputs)
            epilogue_raw_transposed(pix);
            return;
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int cb = n0 + nt * 32;
            // uniform: every channel of the tile exists, and gets a residual if any does (a tile that
            // gets none at all holds zeros and is fast as well)
            const bool fast = FULLT || (cb + 32 <= p.N && (!kRes || cb + 32 <= res_lim || cb >= res_lim));
            if (FULLT || fast)
                epilogue_tile(std::true_type{}, nt, pix, bits_pix, rv, sub);
            else
                epilogue_tile(std::false_type{}, nt, pix, bits_pix, rv, sub);
        }
        if constexpr (PSAVE && !kTwoPhase) {
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // the four pixels' sums are in LDS
            if (wave < NT) window_maximum(wave, pix);                       // (uniform per wave)
        }
        if constexpr (kTwoPhase) {  // one channel tile at a time: wave nt takes tile nt's maximum, the others hand in
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (nt > 0) asm volatile("s_barrier" ::: "memory");  // the previous tile's sums have been read
                if (wave != nt) {                                    // (uniform per wave)
                    v4i* x = lds_win + (((wave - nt - 1) & 3) * 2) * 64 + lane;
                    x[0] = v4i{(int)prw[nt][0], (int)prw[nt][1], (int)prw[nt][2], (int)prw[nt][3]};
                    x[64] = v4i{(int)prw[nt][4], (int)prw[nt][5], (int)prw[nt][6], (int)prw[nt][7]};
                }
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                if (wave == nt) window_maximum(nt, pix);
            }
        }
        if (RM != RM_RAW && ng == n_groups - 1 && (!POOL || sub == 3)) {  // zero the pixel's padding words
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                for (int w = max((p.N + 31) / 32, n_groups * NT); w < p.bits_row_words; ++w)
                    __builtin_amdgcn_raw_buffer_store_b32(0, r_bits, (int)voff_bits[mt],
                                                          (int)(bits_pix + (unsigned)w * row_b), 0);
        }
    };

    // ---- persistent loop over this wave's tiles.  The activation chunks rotate through NB register
    // buffers: the chunk that will be multiplied NB-1 steps from now is requested before the current
    // one is multiplied (two steps of lookahead for Cin >= 192, where one chunk of MFMAs is shorter
    // than the memory latency and few waves share a SIMD).
    // (Two tiles of lookahead for the short residual tiles, with a third buffer for words and operand, measured no
    // faster on ResNet-18's first two stages and cost the Cin = 128 layers their third wave per SIMD.)
    constexpr int NB = kAhead ? 2 : (SPT >= 3 && !(kRes && MT == 2 && SPT >= 6) ? 3 : 2);  // (registers)
    constexpr int LOOK = NB - 1;
    struct Cursor {
        int pi, y, x, chunk, sub;  // item index, row and (skewed) column, chunk of the tile, pixel of the window
        int xr;                    // pi % roww
    };
    auto advance = [&](Cursor& c) __attribute__((always_inline)) {
        if (++c.chunk == NCH) {
            c.chunk = 0;
            if constexpr (POOL) {  // (WIN_MAXSAVE: a wave stays on its pixel of the window)
                if (++c.sub < 4) return;
                c.sub = 0;
            }
            c.pi += dpi;
            c.xr += dx;
            c.y += dy;
            c.x += dxs;
            if (c.xr >= roww) {
                c.xr -= roww;
                ++c.y;
                ++c.x;
            }
            if (c.x >= roww) c.x -= roww;
        }
    };
    // output pixel a cursor stands on
    auto pix_y = [&](const Cursor& c) __attribute__((always_inline)) { return kWin ? 2 * c.y + (c.sub >> 1) : c.y; };
    auto pix_x = [&](const Cursor& c) __attribute__((always_inline)) { return kWin ? 2 * c.x + (c.sub & 1) : c.x; };
    uint32_t buf[NB][TPC * SPT][MT];
    uint32_t msk[NB];
    int rv[kAhead ? NB : 1][NRV][NW];
    Cursor cc = {pi, y, (xr + y) % roww, 0, PSAVE ? wave : 0, xr};  // chunk being multiplied
    Cursor lc = cc;             // chunk being requested (LOOK steps ahead)
#pragma unroll
    for (int i = 0; i < LOOK; ++i) {
        msk[i] = 0;
        if (lc.pi < npix) {
            msk[i] = load_chunk(pix_y(lc), pix_x(lc), lc.chunk, buf[i]);
            if constexpr (kAhead) request_residual(pix_y(lc), pix_x(lc), rv[i]);  // (a chunk is a whole tile here)
        }
        advance(lc);
    }

    // The first activation (and residual) requests are on their way as well.
    // ---- expand the weight words into LDS
    {
        constexpr int kPerWave = kStagePerWave;
        const uint32_t* tmp = wstage;
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) {
            const int f = wave + i * kWaves;
            const int nt = f % NT;
            if (f < NQ * NT) {
                if constexpr (FULLT) {
                    lds_w[f * 64 + lane] = expand_f4(tmp[i]);
                } else {
                    // channels past N multiply by FP4 zeros
                    const bool exists = (ng * NT + nt) * 32 + row_to_channel(j) < p.N;
                    lds_w[f * 64 + lane] = expand_f4_masked(tmp[i], exists ? 0xffffffffu : 0u);
                }
            }
        }
    }
    // A NaN threshold always yields bit 1 (!(x < NaN)), exactly like -inf: staged as such, so that
    // the epilogue can take the bit from the sign of x - threshold.
    // Without a residual the sum s is an integer with |s| <= 9 Cin <= 4608, so s < threshold is
    // the same as s < ceil(threshold), and thresholds beyond +-8192 decide like +-8192.  The
    // negated integer threshold is then what the accumulator STARTS from (operand C of the tile's
    // first MFMA): the finished accumulator is s - ceil(threshold), exact in fp32, and its sign is
    // the inverted output bit, with no per-value subtraction in the epilogue.
    if (tid < NT * 32) {
        float t = thr_stage;
        t = t != t ? -__builtin_huge_valf() : t;
        if constexpr (RM == RM_NONE) t = 0.0f - fminf(fmaxf(ceilf(t), -8192.0f), 8192.0f);
        // (narrow residuals: |sum + residual| < 2^16 + 4608, so thresholds beyond +-2^21 decide like +-2^21)
        if constexpr (kMagic) t = __uint_as_float(kMagicBits) + fminf(fmaxf(ceilf(t), -2097152.0f), 2097152.0f);
        lds_thr[tid] = t;
    }
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc0[nt][v] = RM == RM_NONE ? lds_thr[nt * 32 + 16 * h + v] : (kMagic ? __uint_as_float(kMagicBits) : 0.0f);
    if constexpr (kAhead && RM == RM_POOLED) {  // (one tile ahead: the first tile's operand)
        if (cc.pi < npix) finish_residual(rv[0]);
    }

    // one step with compile-time buffer indices: multiply buffer I, request into buffer (I + LOOK) % NB
    auto step = [&](auto slot) __attribute__((always_inline)) {
        constexpr int I = decltype(slot)::value;
        constexpr int J = (I + LOOK) % NB;
        // Both this chunk and the next one interior (Cin <= 128): the next one's loads ride along with
        // this one's MFMAs.
        bool fused = false;
        unsigned nsoff = 0;
        const bool ahead = lc.pi < npix;  // (uniform) there is a chunk LOOK steps ahead
        if (ahead) {
            if (SPT <= 2 && msk[I] == kAllTaps && chunk_interior(pix_y(lc), pix_x(lc), lc.chunk, nsoff)) {
                fused = true;
                msk[J] = kAllTaps;
            } else {
                msk[J] = load_chunk(pix_y(lc), pix_x(lc), lc.chunk, buf[J]);
            }
            // NCH == 1: that chunk is a whole tile, whose residual operand is requested with it
            if constexpr (kAhead) request_residual(pix_y(lc), pix_x(lc), rv[J]);
        }
        advance(lc);
        int (*rcur)[NW] = rv[kAhead ? I : 0];
        if constexpr (kAhead) {
            compute_chunk(cc.chunk, buf[I], msk[I], fused, buf[J], nsoff);
            // a pooled source is reduced as soon as its tile has been multiplied (frees the registers of
            // the window); otherwise the operand is left in flight until its own epilogue
            if constexpr (RM == RM_POOLED) {
                if (ahead) finish_residual(rv[J]);
            }
        } else {
            if constexpr (kRes) {
                if (cc.chunk == 0) request_residual(pix_y(cc), pix_x(cc), rcur);
            }
            compute_chunk(cc.chunk, buf[I], msk[I], fused, buf[J], nsoff);
        }
        if (cc.chunk == NCH - 1) {
            if constexpr (!kAhead) finish_residual(rcur);
            epilogue(cc.y, cc.x, cc.sub, rcur);
        }
        advance(cc);
    };

    while (cc.pi < npix) {
        step(std::integral_constant<int, 0>{});
        if (cc.pi >= npix) break;
        step(std::integral_constant<int, 1>{});
        if constexpr (NB >= 3) {
            if (cc.pi >= npix) break;
            step(std::integral_constant<int, 2>{});
        }
        if constexpr (NB >= 4) {
            if (cc.pi >= npix) break;
            step(std::integral_constant<int, 3>{});
        }
    }
}

// The current device and its number of compute units (looked up once per device).
constexpr int kMaxDevices = 64;
int device_info(int* dev, int* cus) {
    static std::atomic<int> cu_count[kMaxDevices];
    if (int rc = check_hip(hipGetDevice(dev), "hipGetDevice")) return rc;
    if (*dev < 0 || *dev >= kMaxDevices) return fail(TCBNN_EUNSUPPORTED, "conv3x3: device ordinal %d", *dev);
    int n = cu_count[*dev].load(std::memory_order_acquire);
    if (n == 0) {
        if (int rc = check_hip(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, *dev),
                               "hipDeviceGetAttribute(MultiprocessorCount)"))
            return rc;
        n = std::max(1, n);
        cu_count[*dev].store(n, std::memory_order_release);
    }
    *cus = n;
    return TCBNN_OK;
}

// Sizes in bytes of the tensors the kernel addresses through buffer descriptors.
struct TensorBytes {
    long long act, rin, rout, bits;
};
TensorBytes tensor_bytes(const BgemmParams& p) {
    auto res_words = [&](long long pixels, int channels, int fmt) {  // (32-bit words)
        const long long per = (long long)residual_group_channels(fmt);
        return pixels * ((channels + per - 1) / per) * p.B * (long long)(residual_group_bytes(fmt) / 4);
    };
    TensorBytes t;
    t.act = 4LL * p.H * p.W * p.cw * p.B;
    t.rin = p.res_in != nullptr ? 4 * res_words((long long)p.PH * p.PW * (p.res_pool ? 4 : 1), p.res_in_ch, p.res_in_fmt) : 0;
    t.rout = p.res_out != nullptr ? 4 * res_words((long long)p.PH * p.PW / (p.res_out_pool ? 4 : 1), p.N, p.res_out_fmt) : 0;
    t.bits = 4LL * p.OH * p.OW * p.bits_pix_stride;
    if (p.mode == EPI_RAW) {  // the int32 output takes the place of the saved residual
        const long long last = ((long long)p.PH * p.PW - 1) * p.raw_pix_stride + (long long)(p.B - 1) * p.raw_b_stride + p.N;
        t.rout = 4 * last;
        t.bits = 0;
    }
    return t;
}

template <int SPT, int RM, int MT, int NT, int RF, int WIN, bool FULLT>
int launch_f(const BgemmParams& p, hipStream_t stream) {
    constexpr int NQ = 9 * SPT;
    constexpr int kWaves = waves_of(SPT, NT, WIN), kThreads = 64 * kWaves;
    constexpr bool kRawTranspose = raw_transposed(SPT, RM, NT, FULLT);
    constexpr bool kWgItems = WIN == WIN_MAXSAVE;  // a work item (window) is taken by a whole workgroup
    const size_t lds_bytes = (size_t)NQ * NT * 64 * 16 + NT * 32 * sizeof(float) +
                             (kRawTranspose ? (size_t)kWaves * 32 * raw_pitch(NT) * sizeof(int) : 0) +
                             (kWgItems ? (size_t)win_area_bytes(SPT, NT) : 0);
    // Per instantiation and device, set up by the first launch there: the dynamic LDS limit, and how many of its
    // workgroups a CU holds at once (registers and LDS).  Atomics only so that two host threads that both find the
    // entry empty do no harm (both store the same value).
    static std::atomic<int> resident_on[kMaxDevices];
    int dev = 0, cus = 0;
    if (int rc = device_info(&dev, &cus)) return rc;
    int resident = resident_on[dev].load(std::memory_order_acquire);
    if (resident == 0) {
        const void* fn = reinterpret_cast<const void*>(&conv3x3_mfma_f4_kernel<SPT, RM, MT, NT, RF, WIN, FULLT>);
        if (int rc = check_hip(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes),
                               "hipFuncSetAttribute(MaxDynamicSharedMemorySize)"))
            return rc;
        int n = 0;
        if (int rc = check_hip(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, kThreads, lds_bytes),
                               "hipOccupancyMaxActiveBlocksPerMultiprocessor"))
            return rc;
        resident = std::max(1, n);
        resident_on[dev].store(resident, std::memory_order_release);
    }
    const int n_groups = (p.N + 32 * NT - 1) / (32 * NT);
    const int b_groups = (p.B + 32 * MT - 1) / (32 * MT);
    const int items = WIN != WIN_NONE ? (p.PH / 2) * (p.PW / 2) : p.PH * p.PW;  // pixels, or 2x2 windows of them
    // streams worth launching: one per item for workgroup-wide items; else one per kWaves items, or per 4 for
    // eight-wave workgroups, whose waves 0-3 (one per SIMD) are served first (see the kernel's first item)
    constexpr int kServedFirst = kWaves == 8 ? 4 : kWaves;
    const int quads = kWgItems ? items : (items + kServedFirst - 1) / kServedFirst;
    // Persistent workgroups, all resident at once: two per CU (three for residual layers), fewer
    // when registers or LDS hold fewer.  Measured on every layer of ResNet-18 at batch 256: more, shorter-lived
    // workgroups stage the weights more often and lose; and a grid even slightly larger than the resident slots
    // loses more (its last workgroups start, stage and ramp up only when the first ones have finished: the 14 x 14
    // and 7 x 7 layers ran 10-18 % longer with 1.5 rounds than with one round of workgroups that each take two
    // items per wave).  So: as many pixel streams as fit in one round, never more.
    static const int wg_env = getenv("TCBNN_WG_PER_CU") ? atoi(getenv("TCBNN_WG_PER_CU")) : 0;  // tuning switch
    // Residual layers with one image tile per wave are bound by memory and by their epilogue's latency chains: a third
    // workgroup per CU, where registers and LDS hold one (`resident`), keeps more requests in flight (stage-1 and
    // stage-2 layers of ResNet-18: -3 to -8 %); a fourth where the kernel was compiled for it (L1B2C2 at batch 256:
    // 28.0 -> 26.5 us).
    constexpr bool kResLayer = RM == RM_PLAIN || RM == RM_POOLED;
    const int wg_want = wg_env > 0 ? wg_env : (kResLayer && MT == 1 ? (waves_per_simd(SPT, RM, WIN) == 4 ? 4 : 3) : 2);
    const int wg_per_cu = std::max(1, std::min(wg_want, resident));
    const int best = std::max(1, std::min(cus * wg_per_cu / (n_groups * b_groups), quads));
    // channels that receive an injected residual: o < residual_channels, and only those the
    // source tensor holds (kernel.cuh:770)
    const int res_lim = p.res_in != nullptr ? std::min(std::min(p.res_limit, p.res_in_ch), p.N) : 0;
    const long long blocks = (long long)best * n_groups * b_groups;
    const TensorBytes tb = tensor_bytes(p);
    if (blocks > 0x7fffffffLL || b_groups > 65535 || best > 65535) return fail(TCBNN_EINVAL, "conv3x3: grid too large");
    // a wave's stride over the work items, split into rows and columns once here instead of in every wave
    const int roww = WIN != WIN_NONE ? p.PW / 2 : p.PW, dpi = kWgItems ? best : best * kWaves;
    const int dy = dpi / roww, dx = dpi % roww, dxs = (dx + dy) % roww;
    hipLaunchKernelGGL((conv3x3_mfma_f4_kernel<SPT, RM, MT, NT, RF, WIN, FULLT>),
                       dim3((unsigned)n_groups, (unsigned)b_groups, (unsigned)best), dim3(kThreads), lds_bytes,
                       stream, p, p.act, p.wgt, p.bn, p.res_in, RM == RM_RAW ? p.out_i32 : p.res_out, res_lim, p.res_out_fmt,
                       (unsigned)tb.act, (unsigned)tb.rin, (unsigned)tb.rout, (unsigned)tb.bits, n_groups, b_groups, best,
                       dy, dx, dxs);
    TCBNN_LAUNCH_CHECK("conv3x3_mfma_f4_kernel");
    return TCBNN_OK;
}

// Every channel tile of the launch full, and the residual limit on a tile boundary?  (see FULLT at the kernel)
template <int SPT, int RM, int MT, int NT, int RF, int WIN>
int launch_t(const BgemmParams& p, hipStream_t stream) {
    const int res_lim = p.res_in != nullptr ? std::min(std::min(p.res_limit, p.res_in_ch), p.N) : 0;
    // (with the int32 output, that instantiation also stores whole 128-bit words: the output must be aligned for them)
    const bool raw_ok = RM != RM_RAW || (p.raw_pix_stride % 4 == 0 && p.raw_b_stride % 4 == 0 &&
                                         (reinterpret_cast<uintptr_t>(p.out_i32) & 15) == 0);
    if (p.N % (32 * NT) == 0 && res_lim % 32 == 0 && raw_ok) return launch_f<SPT, RM, MT, NT, RF, WIN, true>(p, stream);
    if constexpr (WIN == WIN_MAXSAVE)  // (conv3x3_mfma_applicable admits the window maximum on full tiles only)
        return fail(TCBNN_EUNSUPPORTED, "conv3x3: pooled residual save needs full channel tiles");
    else
        return launch_f<SPT, RM, MT, NT, RF, WIN, false>(p, stream);
}

// Which instantiation serves a layer.  Measured on ResNet-18 and VGG-16 at batch 256 (10 launches back to back):
// two channel tiles per wave (each expanded activation fragment feeds two MFMAs) everywhere except on layers of
// Cin >= 384 that inject the 2 x 2 maximum of a larger tensor (the eight-wave workgroup below was 8 % slower
// there: four times the residual operands per tile) and on the int32-output kernel for Cin = 192..384 (its LDS
// staging area); from Cin = 384 on the weights of two channel tiles leave room for one workgroup per CU only, which
// then has eight waves (waves_of).  Two image tiles per wave (each weight fragment read from LDS feeds two MFMAs)
// on the plain and int32-output layers up to Cin = 256; one on residual layers (their operands fill the registers)
// and from Cin = 384 on (the activation ring of two image tiles no longer fits next to two channel tiles'
// accumulators).
struct Pick {
    int rm, mt, nt, r16, win;  // r16: TCBNN_RES_* format of the injected residual; win: WIN_*
};
constexpr int pick_nt(int spt, int rm) {
    return rm == RM_POOLED ? (spt >= 6 ? 1 : 2) : (rm == RM_RAW ? (spt >= 3 && spt < 8 ? 1 : 2) : 2);
}
// Channel tiles per wave when the saved residual is the window maximum (the four waves of a workgroup then share a
// window): two up to Cin = 128 (three or four workgroups per CU) and at Cin = 256 (two workgroups per CU with the
// one-tile-at-a-time exchange of win_two_phase: L3B2C2 of ResNet-18 at batch 256 20.8 -> 19.8 us), one otherwise.
constexpr int pick_nt_maxsave(int spt) { return spt <= 2 || spt == 4 ? 2 : 1; }
constexpr int pick_mt(int spt, int rm) {
    return rm == RM_RAW ? (spt >= 8 ? 1 : 2) : (rm == RM_NONE ? (spt >= 6 ? 1 : 2) : 1);
}
Pick pick(const BgemmParams& p) {
    const int rm = p.mode == EPI_RAW ? RM_RAW
                   : p.res_in == nullptr && p.res_out == nullptr
                       ? RM_NONE
                       : (p.res_in != nullptr && p.res_pool ? RM_POOLED : RM_PLAIN);
    const int fmt = p.res_in != nullptr ? p.res_in_fmt : TCBNN_RES_I32;
    // (a pooled int32 source keeps one channel tile per wave: four times sixteen words per tile and lane spilled)
    int nt = rm == RM_POOLED && fmt == TCBNN_RES_I32 ? 1 : pick_nt(p.cw / 2, rm);
    if (rm == RM_PLAIN && p.res_out_pool) nt = pick_nt_maxsave(p.cw / 2);
    int mt = pick_mt(p.cw / 2, rm);
    // A plain layer with fewer than four two-image tiles per SIMD takes one image tile per wave: twice the items, so
    // the last round leaves less of the machine idle, which outweighs the weight fragments then being read from LDS
    // for every MFMA (ResNet-18 at batch 256: the stride-2 layers L3B1C1 9.9 -> 9.3 us, L4B1C1 10.7 -> 10.0 us; with
    // more tiles the larger tile wins: L1B1C1 15.4 -> 17.5 us).
    if (rm == RM_NONE && p.pool_h == 1 && mt == 2) {
        int dev = 0, cus = 0;
        const long long tiles = (long long)p.PH * p.PW * ((p.B + 63) / 64) * ((p.N + 32 * nt - 1) / (32 * nt));
        if (device_info(&dev, &cus) == TCBNN_OK && tiles < 4LL * 4 * cus) mt = 1;
    }
    return {rm, mt, nt, fmt, p.pool_h == 2 ? WIN_ORPOOL : (p.res_out_pool ? WIN_MAXSAVE : WIN_NONE)};
}

template <int SPT>
int launch_m(const BgemmParams& p, hipStream_t stream) {
    const Pick k = pick(p);
    switch (k.rm) {
        case RM_NONE:
            return k.win == WIN_ORPOOL
                       ? launch_t<SPT, RM_NONE, pick_mt(SPT, RM_NONE), pick_nt(SPT, RM_NONE), TCBNN_RES_I32, WIN_ORPOOL>(p, stream)
                       : (k.mt == 1 ? launch_t<SPT, RM_NONE, 1, pick_nt(SPT, RM_NONE), TCBNN_RES_I32, WIN_NONE>(p, stream)
                                    : launch_t<SPT, RM_NONE, pick_mt(SPT, RM_NONE), pick_nt(SPT, RM_NONE), TCBNN_RES_I32, WIN_NONE>(p, stream));
        case RM_RAW:
            return launch_t<SPT, RM_RAW, pick_mt(SPT, RM_RAW), pick_nt(SPT, RM_RAW), TCBNN_RES_I32, WIN_NONE>(p, stream);
        case RM_PLAIN:
            if (k.win == WIN_MAXSAVE)  // (a narrow injected residual: conv3x3_mfma_applicable)
                return k.r16 == TCBNN_RES_I12
                           ? launch_t<SPT, RM_PLAIN, pick_mt(SPT, RM_PLAIN), pick_nt_maxsave(SPT), TCBNN_RES_I12, WIN_MAXSAVE>(p, stream)
                           : launch_t<SPT, RM_PLAIN, pick_mt(SPT, RM_PLAIN), pick_nt_maxsave(SPT), TCBNN_RES_I16, WIN_MAXSAVE>(p, stream);
            return k.r16 == TCBNN_RES_I12
                       ? launch_t<SPT, RM_PLAIN, pick_mt(SPT, RM_PLAIN), pick_nt(SPT, RM_PLAIN), TCBNN_RES_I12, WIN_NONE>(p, stream)
                       : (k.r16 == TCBNN_RES_I16
                              ? launch_t<SPT, RM_PLAIN, pick_mt(SPT, RM_PLAIN), pick_nt(SPT, RM_PLAIN), TCBNN_RES_I16, WIN_NONE>(p, stream)
                              : launch_t<SPT, RM_PLAIN, pick_mt(SPT, RM_PLAIN), pick_nt(SPT, RM_PLAIN), TCBNN_RES_I32, WIN_NONE>(p, stream));
        default:
            return k.r16 == TCBNN_RES_I12
                       ? launch_t<SPT, RM_POOLED, pick_mt(SPT, RM_POOLED), pick_nt(SPT, RM_POOLED), TCBNN_RES_I12, WIN_NONE>(p, stream)
                       : (k.r16 == TCBNN_RES_I16
                              ? launch_t<SPT, RM_POOLED, pick_mt(SPT, RM_POOLED), pick_nt(SPT, RM_POOLED), TCBNN_RES_I16, WIN_NONE>(p, stream)
                              : launch_t<SPT, RM_POOLED, pick_mt(SPT, RM_POOLED), 1, TCBNN_RES_I32, WIN_NONE>(p, stream));
    }
}

}  // namespace

// the kernel's 32-bit buffer offsets (and its "out of range" lane offset) need every tensor below 2 GiB
static bool within_2gib(const BgemmParams& p) {
    const TensorBytes t = tensor_bytes(p);
    const long long lim = 1LL << 31;
    return t.act < lim && t.rin < lim && t.rout < lim && t.bits < lim;
}

bool conv3x3_mfma_applicable(const BgemmParams& p) {
    // un-pooled, or 2x2 pooling of whole windows without residuals
    const bool pool_ok = (p.pool_h == 1 && p.pool_w == 1) ||
                         (p.pool_h == 2 && p.pool_w == 2 && p.PH % 2 == 0 && p.PW % 2 == 0 && p.res_in == nullptr &&
                          p.res_out == nullptr);
    // the centre tap of every output pixel lies inside the frame (the kernel starts each tile with it)
    const bool centre_ok = p.pad_h <= 1 && p.pad_w <= 1 && (p.PH - 1) * p.stride_h - p.pad_h + 1 < p.H &&
                           (p.PW - 1) * p.stride_w - p.pad_w + 1 < p.W;
    // threshold epilogue, or the int32 dot products of an un-pooled convolution without residuals
    const bool mode_ok = (p.mode == EPI_THRESH && p.nan_bit == 1) ||
                         (p.mode == EPI_RAW && p.pool_h == 1 && p.pool_w == 1 && p.res_in == nullptr &&
                          p.res_out == nullptr && p.raw_pix_stride >= 0 && p.raw_b_stride >= 0);
    // the saved residual as the maximum over 2x2 windows: whole windows, every channel tile full and entirely below or
    // above the injection limit, and sums that the epilogue handles as 16-bit pairs (a narrow injected residual, a
    // 12- or 16-bit output)
    const int res_lim = p.res_in != nullptr ? std::min(std::min(p.res_limit, p.res_in_ch), p.N) : 0;
    const bool psave_ok = !p.res_out_pool ||
                          (p.res_out != nullptr && p.res_in != nullptr && !p.res_pool && p.pool_h == 1 && p.pool_w == 1 &&
                           p.PH % 2 == 0 && p.PW % 2 == 0 && p.mode == EPI_THRESH && p.N % 64 == 0 && res_lim % 32 == 0 &&
                           (p.res_in_fmt == TCBNN_RES_I12 || p.res_in_fmt == TCBNN_RES_I16) &&
                           (p.res_out_fmt == TCBNN_RES_I12 || p.res_out_fmt == TCBNN_RES_I16));
    return p.R == 3 && p.S == 3 && pool_ok && centre_ok && mode_ok && psave_ok &&
           p.ksplit <= 1 && filter_has_fragments(3, 3, 32 * p.cw) && p.k_tap == 32 * p.cw &&
           (long long)p.PH * p.PW < (1 << 24) && within_2gib(p);
}

void conv3x3_mfma_kernel_name(const BgemmParams& p, char* buf, size_t len) {
    const Pick k = pick(p);
    const int res_lim = p.res_in != nullptr ? std::min(std::min(p.res_limit, p.res_in_ch), p.N) : 0;
    const bool raw_ok = k.rm != RM_RAW || (p.raw_pix_stride % 4 == 0 && p.raw_b_stride % 4 == 0 &&
                                           (reinterpret_cast<uintptr_t>(p.out_i32) & 15) == 0);
    const bool full = p.N % (32 * k.nt) == 0 && res_lim % 32 == 0 && raw_ok;
    snprintf(buf, len, "conv3x3_mfma_f4_kernel<%d, %d, %d, %d, %d, %d, %s>", p.cw / 2, k.rm, k.mt, k.nt, k.r16, k.win,
             full ? "true" : "false");
}

int launch_conv3x3_mfma(const BgemmParams& p, hipStream_t stream) {
    switch (p.cw) {
        case 2:
            return launch_m<1>(p, stream);
        case 4:
            return launch_m<2>(p, stream);
        case 6:
            return launch_m<3>(p, stream);
        case 8:
            return launch_m<4>(p, stream);
        case 12:
            return launch_m<6>(p, stream);
        default:
            return launch_m<8>(p, stream);
    }
}

}  // namespace tcbnn
