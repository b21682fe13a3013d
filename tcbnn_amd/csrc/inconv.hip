// First-layer convolution: fp32 3-channel NCHW input, +-1 filters, fp32
// accumulation in the reference's exact order (InConv128LayerFMT,
// kernel.cuh:578-672):
//     acc = 0; for r, for s (in-frame taps only): acc += ((+-f0) + (+-f1)) + (+-f2)
//     bit = !((float)acc < bn[o]);  OR over the pool window;  residual = (int)acc
// One ulp decides a threshold bit, so nothing here may be reassociated: there
// are no multiplies (the sign is applied by flipping the fp32 sign bit with a
// precomputed mask), hence no FMA contraction either.
//
// Two kernels:
//   inconv_tiled_kernel (pool 1x1): workgroup = one output row y, 4 consecutive output
//     columns, 64 images (lane = image); a wave owns two of the columns and 32 of the 64 output
//     channels of a pass.  For each filter row the needed
//     input row segment of the 64 images is read with lanes running along the image row
//     (contiguous runs) and transposed through LDS to image-innermost order, so the
//     compute phase reads LDS without bank conflicts, the filter sign masks are
//     wave-uniform scalar loads, and the packed words / int32 residuals are written as
//     contiguous 256-byte runs of the batch-innermost output layouts.
//   inconv_generic_kernel (any pooling): one lane per pooled output pixel.
#include <algorithm>
#include <stdlib.h>
#include <string.h>

#include <type_traits>

#include "common.h"

namespace tcbnn {
namespace {

constexpr int kThreads = 256;
constexpr int kXT = 4;        // output columns per workgroup (one per wave)
constexpr int kLB = 65;       // LDS row pitch in floats for 64 images (+1 against conflicts)
constexpr int kMaxCols = 32;  // (kXT-1)*stride + S must fit

struct InConvParams {
    const float* in;       // [B][3][H][W]
    const uint4* masks;    // [taps][opad32] {m0, m1, m2, 0}
    const float* bn;
    uint32_t* out;         // [OH][OW][ow][B]
    int32_t* res;          // residual tensor in format res_fmt, or null
    int res_fmt;           // TCBNN_RES_*
    int H, W, B, O, opad, ow;
    int R, S, stride_h, stride_w, pad_h, pad_w;
    int PH, PW, pool_h, pool_w, OH, OW;
};

__device__ __forceinline__ float flip(float f, uint32_t m) {
    return __uint_as_float(__float_as_uint(f) ^ m);
}

typedef float v8f __attribute__((ext_vector_type(8)));

// The eight possible values of ((+-f0) + (+-f1)) + (+-f2), indexed by the sign pattern
// 4*neg0 + 2*neg1 + neg2.  With t = f0 + f1 and u = f0 - f1 (round-to-nearest is symmetric
// under negation, so (-f0) + f1 == -(f0 - f1) bit for bit, up to the sign of a zero):
//   0: t + f2   1: t - f2   2: u + f2   3: u - f2   4: -(u - f2)   5: -(u + f2)   6: -(t - f2)   7: -(t + f2)
// A filter tap then costs 6 adds + 4 negations per lane once, and each output channel one
// register-indexed add (the pattern is wave-uniform), instead of 3 sign flips and 3 adds.
// A tap outside the frame reads zeros from the staged tile: all eight values are then +-0, and
// adding them leaves every accumulator as it was, which is the reference's "skip the tap".
__device__ __forceinline__ v8f sign_combos(float f0, float f1, float f2) {
    const float t = f0 + f1, u = f0 - f1;
    v8f c;
    c[0] = t + f2;
    c[1] = t - f2;
    c[2] = u + f2;
    c[3] = u - f2;
    c[4] = -c[3];
    c[5] = -c[2];
    c[6] = -c[1];
    c[7] = -c[0];
    return c;
}

// a[k] += ca[idx_k] and b[k] += cb[idx_k] for 8 output channels of two pixels with ONE switch
// into VGPR-index mode and one index write per channel: the combination vectors are pinned to
// v[120:127] and v[112:119], source 0 of each v_add_f32 is that base displaced by the index in
// M0 (s_set_gpr_idx_idx only rewrites the index, it does not touch the MODE register).  The
// scalar unit issues one instruction per cycle for the whole CU, so an index write per add
// would hold the four SIMDs back; shared by the two pixels it does not.
// Wait states between a write of the index (M0) and the VALU instruction that uses it: the
// hardware does not interlock this pair.  Without them an add can use a stale M0, i.e. a
// register far outside v[112:127].  Never remove them.
#define IDX_WAIT "s_nop 1\n\t"
__device__ __forceinline__ void add_indexed8x2(float* a, float* b, v8f ca, v8f cb, int i0, int i1, int i2, int i3,
                                               int i4, int i5, int i6, int i7) {
    asm volatile(
        "s_set_gpr_idx_on %16, gpr_idx(SRC0)\n\t" IDX_WAIT
        "v_add_f32_e32 %0, v120, %0\n\t"
        "v_add_f32_e32 %8, v112, %8\n\t"
        "s_set_gpr_idx_idx %17\n\t" IDX_WAIT
        "v_add_f32_e32 %1, v120, %1\n\t"
        "v_add_f32_e32 %9, v112, %9\n\t"
        "s_set_gpr_idx_idx %18\n\t" IDX_WAIT
        "v_add_f32_e32 %2, v120, %2\n\t"
        "v_add_f32_e32 %10, v112, %10\n\t"
        "s_set_gpr_idx_idx %19\n\t" IDX_WAIT
        "v_add_f32_e32 %3, v120, %3\n\t"
        "v_add_f32_e32 %11, v112, %11\n\t"
        "s_set_gpr_idx_idx %20\n\t" IDX_WAIT
        "v_add_f32_e32 %4, v120, %4\n\t"
        "v_add_f32_e32 %12, v112, %12\n\t"
        "s_set_gpr_idx_idx %21\n\t" IDX_WAIT
        "v_add_f32_e32 %5, v120, %5\n\t"
        "v_add_f32_e32 %13, v112, %13\n\t"
        "s_set_gpr_idx_idx %22\n\t" IDX_WAIT
        "v_add_f32_e32 %6, v120, %6\n\t"
        "v_add_f32_e32 %14, v112, %14\n\t"
        "s_set_gpr_idx_idx %23\n\t" IDX_WAIT
        "v_add_f32_e32 %7, v120, %7\n\t"
        "v_add_f32_e32 %15, v112, %15\n\t"
        "s_set_gpr_idx_off"
        : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
          "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7])
        : "s"(i0), "s"(i1), "s"(i2), "s"(i3), "s"(i4), "s"(i5), "s"(i6), "s"(i7), "{v[120:127]}"(ca),
          "{v[112:119]}"(cb)
        : "m0");
}

// Which (image tile, group of four output columns, output row) a workgroup takes; false for the padding of the grid.
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  When the number of image tiles divides 8
// (y_phases > 0 = column ranges per image tile), XCD slot = (image tile, range of column groups) and the workgroups
// of a slot walk along x and then down the rows, so that the input rows shared by consecutive output rows (7-row
// windows at stride 4 overlap by 3) and by neighbouring column groups are found in that XCD's L2 instead of being
// fetched from HBM again.
// Rows are dealt 0, k, 2k, ... then 1, k + 1, ... (k = row_il, chosen by the host): consecutive output rows share
// R - stride input rows, and the workgroup of row r + 1 needs a shared row stride/R of a workgroup's lifetime BEFORE
// the workgroup of row r does.  Dealt in natural order the two start almost together and the row has left the XCD's
// L2 by the time it is needed again; dealt k rows apart the later start of row r + 1 makes the two requests meet
// (fetched bytes of ResNet-18's first layer at batch 256: 286 -> 214 MB).
// In that order the grid is (8 slots, column groups per slot, rows): the workgroup's linear number, which the
// hardware deals to the XCDs, is slot + 8 (column group + groups per slot x row), and nothing has to be divided
// (b_tiles is a power of two there; row / row_g by the host's multiplier).  Every instruction of this kernel's set-up
// is paid 12544 times per launch on an instruction-issue-bound kernel.
__device__ __forceinline__ bool inconv_workgroup_position(int b_tiles, int x_groups, int y_phases, int row_il,
                                                          int rows_total, int row_g, unsigned row_g_magic, int& bt,
                                                          int& xg, int& y) {
    if (y_phases > 0) {
        const int slot = (int)blockIdx.x, xg_per = (int)gridDim.y;
        bt = slot & (b_tiles - 1);
        xg = (slot >> __builtin_ctz((unsigned)b_tiles)) * xg_per + (int)blockIdx.y;
        y = (int)blockIdx.z;
        if (row_il > 1) {
            const int q = (int)__umulhi((unsigned)y, row_g_magic);  // y / row_g
            y = (y - q * row_g) * row_il + q;
            if (y >= rows_total) return false;
        }
        return xg < x_groups;
    }
    const int block = (int)blockIdx.x;
    bt = block % b_tiles;
    xg = (block / b_tiles) % x_groups;
    y = block / (b_tiles * x_groups);
    return true;
}

// The read-only operands are separate __restrict__ kernel arguments so that the
// wave-uniform mask / threshold loads become scalar loads (s_load) feeding v_xor directly.
typedef uint32_t u16v __attribute__((ext_vector_type(16)));
typedef int v4i_t __attribute__((ext_vector_type(4)));

// The epilogue both first-layer kernels share, for a lane's 32 consecutive channels (word `wi`) of one image and pixel.
// Output word: bit n (MSB first) = !(acc[n] < bn[32 wi + n]), i.e. the inverted sign of acc - bn (equal operands give
// +0; a NaN threshold counts as -inf: the bit is 1 either way).
// FULL: the launch has full channel tiles only (O a multiple of 64): the partial-tile code is not even compiled.
template <bool FULL>
__device__ __forceinline__ uint32_t inconv_threshold_word(const float* acc, const float* __restrict__ bn, int wi, int O) {
    uint32_t word = 0;
    if (FULL || wi * 32 + 32 <= O) {  // uniform: full channel tile
#pragma unroll
        for (int n = 0; n < 32; ++n) {
            // (the NaN test on the threshold's bits: wave-uniform, so it stays on the scalar unit)
            const uint32_t tb = __float_as_uint(bn[wi * 32 + n]);
            const float t = __uint_as_float((tb & 0x7fffffffu) > 0x7f800000u ? 0xff800000u : tb);
            word = __builtin_amdgcn_alignbit(word, __float_as_uint(acc[n] - t), 31);
        }
        return ~word;
    }
#pragma unroll
    for (int n = 0; n < 32; ++n) {
        const int ch = wi * 32 + n;
        if (ch < O) word |= (acc[n] < bn[ch] ? 0u : 1u) << (31 - n);
    }
    return word;
}
// Saved residual: (int)acc of the 32 channels in the tensor's format; 16 bytes per (channel group, image) (4 int32 or
// 8 int16), or 24 per group of 16 channels at 12 bits; channels past O are stored as 0, groups past O not at all.
// Streaming stores: the tensor (77-103 MB for ResNet-18 at batch 256) is far larger than the caches and is read two
// launches later.
template <bool FULL>
__device__ __forceinline__ void inconv_store_residual(const float* acc, int32_t* __restrict__ res, int fmt, size_t pix,
                                                      int wi, int O, int B, int b) {
    int r32[32];
#pragma unroll
    for (int n = 0; n < 32; ++n) r32[n] = (int)acc[n];
    if (!FULL && wi * 32 + 32 > O) {  // uniform
#pragma unroll
        for (int n = 0; n < 32; ++n) r32[n] = wi * 32 + n < O ? r32[n] : 0;
    }
    v4i_t* __restrict__ dst = reinterpret_cast<v4i_t*>(res);
    if (fmt == TCBNN_RES_I12) {  // two groups of 16 channels: 16 + 8 bytes each
        typedef int v2i_t __attribute__((ext_vector_type(2)));
        uint32_t* __restrict__ w = reinterpret_cast<uint32_t*>(res);
        const size_t G = (size_t)((O + 15) / 16);
#pragma unroll
        for (int g = 0; g < 2; ++g)
            if (FULL || wi * 32 + 16 * g < O) {
                uint32_t d[6];
                i12_pack8(&r32[16 * g], d[0], d[1], d[2]);
                i12_pack8(&r32[16 * g + 8], d[3], d[4], d[5]);
                __builtin_nontemporal_store(v4i_t{(int)d[0], (int)d[1], (int)d[2], (int)d[3]},
                                            reinterpret_cast<v4i_t*>(w + i12_word_index(pix, G, wi * 2 + g, B, b, 0)));
                __builtin_nontemporal_store(v2i_t{(int)d[4], (int)d[5]},
                                            reinterpret_cast<v2i_t*>(w + i12_word_index(pix, G, wi * 2 + g, B, b, 4)));
            }
    } else if (fmt == TCBNN_RES_I16) {
        const size_t g0 = (pix * ((O + 7) / 8) + wi * 4) * B + b;
#pragma unroll
        for (int g = 0; g < 4; ++g)
            if (FULL || wi * 32 + 8 * g < O)
                __builtin_nontemporal_store(v4i_t{(r32[8 * g] & 0xffff) | (r32[8 * g + 1] << 16),
                                                  (r32[8 * g + 2] & 0xffff) | (r32[8 * g + 3] << 16),
                                                  (r32[8 * g + 4] & 0xffff) | (r32[8 * g + 5] << 16),
                                                  (r32[8 * g + 6] & 0xffff) | (r32[8 * g + 7] << 16)},
                                            dst + g0 + (size_t)g * B);
    } else {
        const size_t g0 = (pix * ((O + 3) / 4) + wi * 8) * B + b;
#pragma unroll
        for (int g = 0; g < 8; ++g)
            if (FULL || wi * 32 + 4 * g < O)
                __builtin_nontemporal_store(v4i_t{r32[4 * g], r32[4 * g + 1], r32[4 * g + 2], r32[4 * g + 3]},
                                            dst + g0 + (size_t)g * B);
    }
}

// Staging of one filter row: the 3 x 64 (channel, image) row segments of ncols floats each.
//   ROWS = true: a wave takes rpw segments at a time (a multiple of 3 for ncols <= 21, else 2), lanes
//     running along the segment; segments are numbered in memory order (image * 3 + channel),
//     so that the address of pass k is a wave-uniform base plus a per-lane constant and the
//     LDS slot a per-lane constant plus an immediate: no per-element address arithmetic.  NST =
//     passes = ceil(192 / (4 rpw)).  With rpw = 2 (NST = 24) the channel of a lane's segment
//     changes from pass to pass with period 3, so the LDS slot has three per-lane constants.
//   ROWS = false: the elements are dealt to the threads linearly, NST = ceil(3 * 64 * ncols / 256)
//     (only for images too large for 32-bit buffer offsets).
// POOLED: blockIdx selects a row of the POOLED output; the workgroup runs the pool_h convolution rows
// of it one after the other and ORs their words (kernel.cuh:646-664); with pool_w = 2 the two columns of
// a wave are one window.  pool_w is 1 or 2 (the host checks), no residual is saved.
// ALLIN (ROWS): the host found every staging pass of every lane inside the 192 segments, the batch a multiple of 64
// and the output channels a multiple of 64, so no pass, image or channel is tested (and none of those tests'
// invariants is computed or kept).
// DLDS (ALLIN): the row segments go from memory straight into LDS (buffer loads with the LDS flag: a wave's 64 lanes
// fill 64 consecutive words at a wave-uniform LDS address), into one of two buffers in turn: no staging registers, no
// LDS write instructions, and one barrier per filter row instead of two.  A lane's place in the 64 words is its
// segment times a fixed stride (kSegStride, odd) plus its column, so the layout is [image][channel][kSegStride]: the
// three channels of a tap are constant offsets apart and the 64 images of a wave's tap read fall into 64 different
// banks (3 kSegStride is odd).  The host selects it when a segment fits the stride.
constexpr int inconv_seg_stride(int nst) { return nst == 4 ? 5 : (nst == 8 ? 9 : (nst == 16 ? 21 : 31)); }
// Where it is used: 16 passes (segments of 11 to 21 columns: 7-wide filters at strides 2 to 4, three waves' worth of
// segments per pass), where it measured 2-4 % faster than staging through registers.  With 8 passes (3x3 filters at
// stride 1: three taps per row) it measured 3-5 % slower and with 24 (11-wide filters, three waves per SIMD) 20 %.
constexpr bool inconv_straight_to_lds(int nst, int ncols) { return nst == 16 && ncols <= inconv_seg_stride(nst); }
template <int NST, bool ROWS, bool POOLED, bool ALLIN, bool DLDS = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(ROWS && NST <= 16 ? 4 : 3))) void inconv_tiled_kernel(
    const InConvParams p, const float* __restrict__ in, const uint4* __restrict__ masks,
    const float* __restrict__ bn, uint32_t* __restrict__ out, int32_t* __restrict__ res, int b_tiles,
    int x_groups, int y_phases, int div_magic, int rpw_arg, int row_il, int rows_total, int row_g, unsigned row_g_magic) {
    // (ALLIN: NST passes of 4 rpw segments are exactly the 192 segments, so rpw is a constant of the instantiation and
    // the staging's LDS offsets are immediates)
    const int rpw = ALLIN ? 48 / NST : rpw_arg;
    static_assert(!DLDS || (ALLIN && ROWS), "direct-to-LDS staging is a variant of the full-tile row staging");
    constexpr int kSegStride = inconv_seg_stride(NST);
    constexpr int kBufWords = 3 * 64 * kSegStride;  // DLDS: one buffer = 192 segments
    __shared__ float tile[DLDS ? 2 * kBufWords : 3 * kMaxCols * kLB];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bt, xg, y;
    if (!inconv_workgroup_position(b_tiles, x_groups, y_phases, row_il, rows_total, row_g, row_g_magic, bt, xg, y))
        return;  // whole workgroup: grid padding
    const int x0 = xg * kXT;
    const int pp = wave & 1;    // which pair of the workgroup's four columns
    const int chh = wave >> 1;  // which 32 of the pass's 64 channels
    const int xa = x0 + 2 * pp, xb = xa + 1;
    // columns of the launch: the convolution's own, or all columns of the pool windows (pooled width rounded up)
    const int xcols = POOLED ? p.pool_w * p.OW : p.PW;
    const bool xa_ok = xa < xcols, xb_ok = xb < xcols;  // wave-uniform
    const int b0 = bt * 64;
    const int b = b0 + lane;
    const int ncols = (kXT - 1) * p.stride_w + p.S;
    const int ax_base = x0 * p.stride_w - p.pad_w;
    const size_t plane = (size_t)p.H * p.W;
    const int n_groups = (p.O + 63) / 64;
    const uint32_t* __restrict__ pats =
        reinterpret_cast<const uint32_t*>(masks) + (size_t)p.R * p.S * p.opad * 4;  // packed pattern table

    for (int g = 0; g < n_groups; ++g) {
      uint32_t pooled[2] = {0u, 0u};  // POOLED: OR of the rows so far, per pixel column of the wave
      const int wi = g * 2 + chh;                       // output word = channel tile of this wave
      const bool work = xa_ok && wi * 32 < p.opad;      // uniform
      for (int py = 0; py < (POOLED ? p.pool_h : 1); ++py) {
        const int yc = POOLED ? y * p.pool_h + py : y;  // convolution row (uniform)
        // (rows past the convolution's own output, when the pooled height is rounded up, are computed like any
        // other from the filter rows still inside the frame: kernel.cuh:587-596 walks pool * output rows)
        float acca[32], accb[32];  // this wave's 32 channels of pixels xa and xb
#pragma unroll
        for (int n = 0; n < 32; ++n) acca[n] = accb[n] = 0.0f;

        // Filter rows inside the frame: r_lo <= r < r_hi (uniform for the whole workgroup).
        const int ay0 = yc * p.stride_h - p.pad_h;
        const int r_lo = max(0, -ay0), r_hi = min(p.R, p.H - ay0);
        const int n_stage = 3 * 64 * ncols;

        // Software-pipelined staging: the input row segment of filter row r+1 is requested
        // from HBM into registers before row r is multiplied, and written to LDS afterwards.
        // Lanes run along the image row (contiguous runs of ncols floats per (channel, image)),
        // LDS is image-innermost; e / ncols by multiply-shift (the host checked the constant).
        float stg[NST];
        // ROWS scheme: per-lane constants
        const int rp = 4 * rpw;                      // segments per pass of the workgroup
        const int sub = DLDS ? lane / kSegStride : lane / ncols;  // segment of the wave's rpw this lane reads
        const int scol = lane - sub * (DLDS ? kSegStride : ncols);  // column in the segment
        const int seg0 = wave * rpw + sub;           // segment (image * 3 + channel) in pass 0
        const int sax = ax_base + scol;
        const bool lane_used = sub < rpw && scol < ncols;  // DLDS: the lane has a word of the segment at all
        const bool lane_ok = sub < rpw && sax >= 0 && sax < p.W && (!DLDS || scol < ncols);  // constant over passes and rows
        // Buffer addressing: descriptor = this workgroup's 64 images, per-lane byte offset (one
        // constant), wave-uniform scalar offset per (row, pass).  A lane outside the frame carries an
        // offset beyond the descriptor's range: the hardware returns 0 for it without touching memory.
        constexpr unsigned kOutOfRange = 0x80000000u;
        const unsigned imgs_here = (unsigned)min(64, p.B - b0);
        const unsigned tile_bytes = imgs_here * 3u * (unsigned)plane * 4u;  // host checked: below 2 GiB
        const unsigned voff = lane_ok ? ((unsigned)seg0 * (unsigned)plane + (unsigned)sax) * 4u : kOutOfRange;
        const int lds0 = (scol * 3 + seg0 % 3) * kLB + seg0 / 3;  // LDS: [column][channel][image]
        // rp not a multiple of 3 (NST = 24): pass k = 3m + i holds segment seg0 + rp i + 3 rp m, i.e. the channel
        // and image of segment seg0 + rp i, rp m images further on
        constexpr bool kThirds = ROWS && NST == 24;
        const int lds1 = (scol * 3 + (seg0 + rp) % 3) * kLB + (seg0 + rp) / 3;
        const int lds2 = (scol * 3 + (seg0 + 2 * rp) % 3) * kLB + (seg0 + 2 * rp) / 3;
        // every pass of every lane inside the 192 segments and the batch (wave-uniform)?
        constexpr bool all_in = ALLIN;
        __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(in + (size_t)b0 * 3 * plane), 0, (int)tile_bytes, 0x00020000);
        auto fetch_row = [&](int r) {
            if constexpr (ROWS) {
                const unsigned row_bytes = (unsigned)(ay0 + r) * (unsigned)p.W * 4u;       // uniform
                const unsigned pass_bytes = (unsigned)rp * (unsigned)plane * 4u;           // uniform
                if constexpr (all_in) {
#pragma unroll
                    for (int k = 0; k < NST; ++k)
                        stg[k] = __builtin_bit_cast(
                            float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff, (int)(row_bytes + k * pass_bytes), 0));
                } else {
#pragma unroll
                    for (int k = 0; k < NST; ++k) {
                        const int seg = seg0 + k * rp;
                        const bool ok = seg < 3 * 64 && b0 + seg / 3 < p.B;
                        stg[k] = __builtin_bit_cast(
                            float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(ok ? voff : kOutOfRange),
                                                                        (int)(row_bytes + k * pass_bytes), 0));
                    }
                }
            } else {
                const size_t row_off = (size_t)(ay0 + r) * p.W;
#pragma unroll
                for (int k = 0; k < NST; ++k) {
                    const int e = tid + k * kThreads;
                    const int bc = (int)(((unsigned)e * (unsigned)div_magic) >> 16);
                    const int col = e - bc * ncols;
                    const int ax = ax_base + col;
                    const int bb = min(b0 + (bc & 63), p.B - 1);
                    float v = 0.0f;
                    if (e < n_stage && ax >= 0 && ax < p.W)
                        v = in[((size_t)bb * 3 + (bc >> 6)) * plane + row_off + ax];
                    stg[k] = v;
                }
            }
        };
        // DLDS: the same requests with LDS as their destination: pass k of this wave fills the 64 words of its rpw
        // segments in buffer `sel` (lanes without a word are switched off; columns outside the frame arrive as zeros).
        auto fetch_row_lds = [&](int r, int sel) {
            typedef __attribute__((address_space(3))) void* lds_ptr_t;
            const unsigned row_bytes = (unsigned)(ay0 + r) * (unsigned)p.W * 4u;       // uniform
            const unsigned pass_bytes = (unsigned)rp * (unsigned)plane * 4u;           // uniform
            float* dst = tile + sel * kBufWords + wave * (48 / NST) * kSegStride;
            if (lane_used) {
#pragma unroll
                for (int k = 0; k < NST; ++k)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(dst + k * 4 * (48 / NST) * kSegStride), 4,
                                                             (int)voff, (int)(row_bytes + k * pass_bytes), 0, 0);
            }
        };
        auto store_row = [&]() {
            if constexpr (ROWS) {
                if (sub < rpw) {
#pragma unroll
                    for (int k = 0; k < NST; ++k)
                        if (all_in || seg0 + k * rp < 3 * 64) {
                            if constexpr (kThirds)
                                tile[(k % 3 == 0 ? lds0 : (k % 3 == 1 ? lds1 : lds2)) + (k / 3) * rp] = stg[k];
                            else
                                tile[lds0 + k * (rp / 3)] = stg[k];
                        }
                }
            } else {
#pragma unroll
                for (int k = 0; k < NST; ++k) {
                    const int e = tid + k * kThreads;
                    const int bc = (int)(((unsigned)e * (unsigned)div_magic) >> 16);
                    const int col = e - bc * ncols;
                    if (e < n_stage) tile[(col * 3 + (bc >> 6)) * kLB + (bc & 63)] = stg[k];
                }
            }
        };

        if constexpr (DLDS) {
            // (a slower wave may still be reading the previous row loop's last buffer)
            if (g > 0 || py > 0) __syncthreads();
            if (r_lo < r_hi) fetch_row_lds(r_lo, 0);
        } else {
            if (r_lo < r_hi) fetch_row(r_lo);
        }
        for (int r = r_lo; r < r_hi; ++r) {
            if constexpr (DLDS) {
                // this wave's words of row r have arrived; after the barrier everybody's have, and everybody has left
                // row r - 1, whose buffer the requests for row r + 1 overwrite
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (r + 1 < r_hi) fetch_row_lds(r + 1, (r + 1 - r_lo) & 1);
            } else {
                __syncthreads();
                store_row();
                __syncthreads();
                if (r + 1 < r_hi) fetch_row(r + 1);
            }
            if (!work) continue;
            // sign patterns of a tap's 32 channels, one per word (wide scalar loads); the pointer moves on by one tap
            // (formed anew per tap it was seven scalar instructions, a 64-bit multiplication among them)
            const uint32_t* __restrict__ ptap = pats + (size_t)(r * p.S) * p.opad + wi * 32;
            for (int s = 0; s < p.S; ++s, ptap += p.opad) {
                const int cola = 2 * pp * p.stride_w + s, colb = cola + p.stride_w;
                const u16v* pw = reinterpret_cast<const u16v*>(ptap);
                const u16v i0 = pw[0], i1 = pw[1];
                // the three channels of a column are kLB floats apart: one address per pixel, constant offsets
                // (DLDS: [image][channel][kSegStride] in the row's buffer)
                constexpr int kChan = DLDS ? kSegStride : kLB;
                const float* ta = DLDS ? tile + ((r - r_lo) & 1) * kBufWords + lane * 3 * kSegStride + cola
                                       : tile + cola * 3 * kLB + lane;
                const float* tb = DLDS ? ta + p.stride_w : tile + colb * 3 * kLB + lane;
                const v8f ca = sign_combos(ta[0], ta[kChan], ta[2 * kChan]);
                const v8f cb = sign_combos(tb[0], tb[kChan], tb[2 * kChan]);
                add_indexed8x2(&acca[0], &accb[0], ca, cb, i0[0], i0[1], i0[2], i0[3], i0[4], i0[5], i0[6], i0[7]);
                add_indexed8x2(&acca[8], &accb[8], ca, cb, i0[8], i0[9], i0[10], i0[11], i0[12], i0[13], i0[14],
                               i0[15]);
                add_indexed8x2(&acca[16], &accb[16], ca, cb, i1[0], i1[1], i1[2], i1[3], i1[4], i1[5], i1[6], i1[7]);
                add_indexed8x2(&acca[24], &accb[24], ca, cb, i1[8], i1[9], i1[10], i1[11], i1[12], i1[13], i1[14],
                               i1[15]);
            }
        }

        if (work && (ALLIN || (b < p.B && wi < p.ow))) {
            // The stores' addresses are worked out here, after the tap loops: formed ahead of them (the compiler hoists
            // what does not depend on the loops) they were live across the whole kernel and were spilled.
            // (the lane index comes from the hardware's lane count here, not from a register kept since the start)
            const int b = b0 + (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
#pragma unroll
            for (int px = 0; px < 2; ++px) {
                if (px == 1 && !xb_ok) continue;
                const float* acc = px == 0 ? acca : accb;
                const size_t pix = (size_t)yc * p.PW + xa + px;
                const uint32_t word = inconv_threshold_word<ALLIN>(acc, bn, wi, p.O);
                if constexpr (POOLED) {
                    pooled[px] |= word;
                    continue;
                }
                out[(pix * p.ow + wi) * p.B + b] = word;
                if (res != nullptr) inconv_store_residual<ALLIN>(acc, res, p.res_fmt, pix, wi, p.O, p.B, b);
            }
        }
      }
      if constexpr (POOLED) {
          if (work && (ALLIN || (b < p.B && wi < p.ow))) {
              if (p.pool_w == 2) {
                  out[(((size_t)y * p.OW + xa / 2) * p.ow + wi) * p.B + b] = pooled[0] | (xb_ok ? pooled[1] : 0u);
              } else {
                  out[(((size_t)y * p.OW + xa) * p.ow + wi) * p.B + b] = pooled[0];
                  if (xb_ok) out[(((size_t)y * p.OW + xb) * p.ow + wi) * p.B + b] = pooled[1];
              }
          }
      }
    }
}

// First layer on an input that is already batch-innermost and zero-padded: float [Hp][Wp][B][3] with
// Hp = (PH - 1) stride_h + R, Wp = (PW - 1) stride_w + S and the frame at (pad_h, pad_w) (tcbnn_inconv_pack_input
// writes it).  A lane's three channels of one input pixel are 12 contiguous bytes and a wave's 64 images 768, so a
// tap is ONE 96-bit buffer load per pixel, straight into registers: no staging through LDS, no barrier, no
// transposition, and no test for the frame (the border holds zeros, which add +-0 like the reference's skipped tap).
// Waves are independent; the four of a workgroup (two pixel pairs x two channel halves) only share cache lines.
// Same arithmetic, same order, same sign-combination and register-index scheme as inconv_tiled_kernel.
constexpr int kDirectAhead = 3;  // taps requested ahead of their use
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void inconv_direct_kernel(
    const InConvParams p, const float* __restrict__ in, const uint4* __restrict__ masks,
    const float* __restrict__ bn, uint32_t* __restrict__ out, int32_t* __restrict__ res, int b_tiles,
    int x_groups, int y_phases, int row_il, int Wp, unsigned in_bytes, int row_g, unsigned row_g_magic) {
    const int rows_total = p.PH;
    typedef float v3f __attribute__((ext_vector_type(3)));
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bt, xg, y;
    if (!inconv_workgroup_position(b_tiles, x_groups, y_phases, row_il, rows_total, row_g, row_g_magic, bt, xg, y)) return;
    const int pp = wave & 1, chh = wave >> 1;
    const int xa = xg * kXT + 2 * pp;
    const bool xa_ok = xa < p.PW, xb_ok = xa + 1 < p.PW;  // uniform
    if (!xa_ok) return;  // (no barrier in this kernel)
    const int b0 = bt * 64;
    const int b = b0 + lane;
    const int n_groups = (p.O + 63) / 64;
    const uint32_t* __restrict__ pats =
        reinterpret_cast<const uint32_t*>(masks) + (size_t)p.R * p.S * p.opad * 4;
    constexpr unsigned kOutOfRange = 0x80000000u;
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(in), 0, (int)in_bytes, 0x00020000);
    const unsigned voff = b < p.B ? (unsigned)b * 12u : kOutOfRange;
    const unsigned col_b = (unsigned)p.B * 12u;               // bytes per padded input column
    const unsigned row_b = (unsigned)Wp * col_b;              // ... per padded input row
    // from the wave's first pixel to its second (an odd width's last wave has none: it reads its first pixel twice)
    const unsigned pix_b = xb_ok ? (unsigned)p.stride_w * col_b : 0u;
    const int taps = p.R * p.S;

    for (int g = 0; g < n_groups; ++g) {
        const int wi = g * 2 + chh;
        if (wi * 32 >= p.opad) continue;  // uniform
        float acca[32], accb[32];
#pragma unroll
        for (int n = 0; n < 32; ++n) acca[n] = accb[n] = 0.0f;
        // cursor of the requests: tap (rr, rs) at byte offset roff
        const unsigned base = (unsigned)(y * p.stride_h) * row_b + (unsigned)(xa * p.stride_w) * col_b;
        unsigned roff = base;
        int rs = 0, rt = 0;
        v3f qa[kDirectAhead], qb[kDirectAhead];
        // (the cursor stops on the last tap: the requests issued past it ask for that tap again and are not used, so
        // nothing outside the packed input is ever addressed)
        auto request = [&](int slot) {
            qa[slot] = __builtin_bit_cast(v3f, __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)voff, (int)roff, 0));
            qb[slot] = __builtin_bit_cast(v3f, __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)voff, (int)(roff + pix_b), 0));
            if (++rt < taps) {
                roff += col_b;
                if (++rs == p.S) {
                    rs = 0;
                    roff += row_b - (unsigned)p.S * col_b;
                }
            }
        };
#pragma unroll
        for (int d = 0; d < kDirectAhead; ++d) request(d);
        for (int t0 = 0; t0 < taps; t0 += kDirectAhead) {
#pragma unroll
            for (int d = 0; d < kDirectAhead; ++d) {
                const int t = t0 + d;
                if (t < taps) {  // uniform
                    const u16v* pw = reinterpret_cast<const u16v*>(pats + (size_t)t * p.opad + wi * 32);
                    const u16v i0 = pw[0], i1 = pw[1];
                    const v8f ca = sign_combos(qa[d][0], qa[d][1], qa[d][2]);
                    const v8f cb = sign_combos(qb[d][0], qb[d][1], qb[d][2]);
                    request(d);
                    add_indexed8x2(&acca[0], &accb[0], ca, cb, i0[0], i0[1], i0[2], i0[3], i0[4], i0[5], i0[6], i0[7]);
                    add_indexed8x2(&acca[8], &accb[8], ca, cb, i0[8], i0[9], i0[10], i0[11], i0[12], i0[13], i0[14], i0[15]);
                    add_indexed8x2(&acca[16], &accb[16], ca, cb, i1[0], i1[1], i1[2], i1[3], i1[4], i1[5], i1[6], i1[7]);
                    add_indexed8x2(&acca[24], &accb[24], ca, cb, i1[8], i1[9], i1[10], i1[11], i1[12], i1[13], i1[14], i1[15]);
                }
            }
        }
        if (b < p.B && wi < p.ow) {
#pragma unroll
            for (int px = 0; px < 2; ++px) {
                if (px == 1 && !xb_ok) continue;
                const float* acc = px == 0 ? acca : accb;
                const size_t pix = (size_t)y * p.PW + xa + px;
                const uint32_t word = inconv_threshold_word<false>(acc, bn, wi, p.O);
                out[(pix * p.ow + wi) * p.B + b] = word;
                if (res != nullptr) inconv_store_residual<false>(acc, res, p.res_fmt, pix, wi, p.O, p.B, b);
            }
        }
    }
}

// fp32 [B][3][H][W] -> zero-padded, batch-innermost [Hp][Wp][B][3] (the frame at (pad_h, pad_w)).  One workgroup
// per (padded row, 64 images, 64 columns): the strip's 3 x 64 segments are read along the image row (lanes = columns) and
// written with lanes = (image, channel), through LDS.
__global__ __launch_bounds__(256) void inconv_pack_input_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                                int B, int H, int W, int Hp, int Wp, int pad_h,
                                                                int pad_w) {
    __shared__ float tile[64 * 3][65];  // [image * 3 + channel][column of a 64-column strip]
    const int yp = blockIdx.x, b0 = blockIdx.y * 64;
    const int y = yp - pad_h;
    const size_t plane = (size_t)H * W;
    {
        const int x0 = blockIdx.z * 64;
        const int cols = min(64, Wp - x0);
        const int c = threadIdx.x & 63, x = x0 + c - pad_w;  // lanes run along the row
        const bool in_frame = c < cols && y >= 0 && y < H && x >= 0 && x < W;
        for (int s0 = threadIdx.x >> 6; s0 < 192; s0 += 4 * 12) {  // 12 segments (= image * 3 + channel) in flight
            float v[12];
#pragma unroll
            for (int k = 0; k < 12; ++k) {
                const int seg = s0 + 4 * k, b = b0 + seg / 3;
                v[k] = in_frame && b < B ? in[((size_t)b * 3 + seg % 3) * plane + (size_t)y * W + x] : 0.0f;
            }
#pragma unroll
            for (int k = 0; k < 12; ++k) tile[s0 + 4 * k][c] = v[k];
        }
        __syncthreads();
        for (int e = threadIdx.x; e < cols * 192; e += 256) {
            const int c = e / 192, seg = e % 192;  // lanes run along (image, channel)
            if (b0 + seg / 3 < B) out[((size_t)yp * Wp + x0 + c) * B * 3 + (size_t)b0 * 3 + seg] = tile[seg][c];
        }
    }
}

__global__ __launch_bounds__(kThreads) void inconv_generic_kernel(const InConvParams p) {
    const long long m = (long long)blockIdx.x * kThreads + threadIdx.x;
    const long long total = (long long)p.B * p.OH * p.OW;
    if (m >= total) return;
    const int b = (int)(m % p.B);
    const int ox = (int)((m / p.B) % p.OW);
    const int oy = (int)(m / ((long long)p.B * p.OW));
    const size_t plane = (size_t)p.H * p.W;
    const float* img = p.in + (size_t)b * 3 * plane;

    for (int g = 0; g < p.ow; ++g) {
        uint32_t word = 0;
        for (int py = 0; py < p.pool_h; ++py) {
            for (int px = 0; px < p.pool_w; ++px) {
                const int y = oy * p.pool_h + py, x = ox * p.pool_w + px;
                // pixels of the window past the convolution's own output (pooled size rounded up) are computed
                // like any other, from the taps still inside the frame (kernel.cuh:587-596 walks pool * output
                // rows and columns); with no tap left the sum is 0
                const int ay0 = y * p.stride_h - p.pad_h, ax0 = x * p.stride_w - p.pad_w;
                float acc[32];
#pragma unroll
                for (int n = 0; n < 32; ++n) acc[n] = 0.0f;
                for (int r = 0; r < p.R; ++r) {
                    const int ay = ay0 + r;
                    if (ay < 0 || ay >= p.H) continue;
                    for (int s = 0; s < p.S; ++s) {
                        const int ax = ax0 + s;
                        if (ax < 0 || ax >= p.W) continue;
                        const size_t off = (size_t)ay * p.W + ax;
                        const float f0 = img[off];
                        const float f1 = img[plane + off];
                        const float f2 = img[2 * plane + off];
                        const uint4* mk = p.masks + (size_t)(r * p.S + s) * p.opad + g * 32;
#pragma unroll
                        for (int n = 0; n < 32; ++n) {
                            const uint4 mm = mk[n];
                            acc[n] += (flip(f0, mm.x) + flip(f1, mm.y)) + flip(f2, mm.z);
                        }
                    }
                }
#pragma unroll
                for (int n = 0; n < 32; ++n) {
                    const int ch = g * 32 + n;
                    if (ch < p.O) word |= (acc[n] < p.bn[ch] ? 0u : 1u) << (31 - n);
                }
                if (p.res != nullptr) {
                    int r32[32];
#pragma unroll
                    for (int n = 0; n < 32; ++n) r32[n] = g * 32 + n < p.O ? (int)acc[n] : 0;
#pragma unroll
                    for (int q = 0; q < 2; ++q)  // whole groups of 16 channels (12-bit values share words)
                        if (g * 32 + 16 * q < p.O)
                            residual_store_group16(p.res, p.res_fmt, (size_t)y * p.PW + x, p.O, g * 2 + q, p.B, b, &r32[16 * q]);
                }
            }
        }
        p.out[(((size_t)oy * p.OW + ox) * p.ow + g) * p.B + b] = word;
    }
}

}  // namespace
}  // namespace tcbnn

using namespace tcbnn;

// Row-wise staging: segments (image, channel) a wave takes per pass, ncols lanes each.  Whole segments only; a
// multiple of 3 where 3 fit the 64 lanes (the channel of a lane's segment is then the same in every pass), and among
// those the largest that divides 48, so that the workgroup's passes cover the 192 segments exactly and no pass needs a
// test (rpw = 9 for 6-column segments used more lanes per pass but left a ragged sixth pass); else 2.
static int inconv_segments_per_wave(int ncols) {
    const int fit = 64 / ncols;
    if (fit < 3) return 2;
    for (int r : {48, 24, 12, 6})
        if (r <= fit) return r;
    return 3;
}

// How the workgroups of the tiled and the direct kernel are dealt (see inconv_tiled_kernel): grid size and order.
struct InConvOrder {
    int b_tiles, x_groups, y_phases, row_il;
    long long blocks;
    dim3 grid;             // (8, column groups per slot, rows) in the XCD-aware order, else (blocks)
    int row_g;             // rows per interleave group (row_il > 1)
    unsigned row_g_magic;  // y / row_g == umulhi(y, row_g_magic) for every row of the grid
    bool ok;               // the grid fits the launch limits and the multiplier is exact
};
static InConvOrder inconv_order(const InConvParams& p, bool pooled, int rows_out) {
    InConvOrder o;
    o.b_tiles = (p.B + 63) / 64;
    o.x_groups = ((pooled ? p.pool_w * p.OW : p.PW) + kXT - 1) / kXT;
    // XCD-aware order when the image tiles divide the 8 XCD slots
    static const bool plain_order = getenv("TCBNN_INCONV_ORDER") != nullptr;  // tuning switch
    o.y_phases = (!plain_order && 8 % o.b_tiles == 0) ? 8 / o.b_tiles : 0;
    // Row interleave of the XCD-aware order: an XCD starts its resident workgroups (4 per CU x 32 CUs) once per
    // workgroup lifetime, xg_per of them per output row, and the start of row r + 1 should lag that of row r by
    // stride/R of a lifetime: k = stride/R x 128 / xg_per rows, taken at 0.7 of that (measured on the 7x7 stride-4
    // layer: 214-217 MB fetched for k = 7..10, 222 for 5, 241 for 14, 286 without).
    static const int il_env = getenv("TCBNN_INCONV_ROWIL") ? atoi(getenv("TCBNN_INCONV_ROWIL")) : -1;  // tuning switch
    o.row_il = 0;
    if (o.y_phases > 0 && !pooled) {
        const int xg_per = (o.x_groups + o.y_phases - 1) / o.y_phases;
        o.row_il = (int)(0.7 * p.stride_h * 128.0 / ((double)p.R * xg_per) + 0.5);
        if (il_env >= 0) o.row_il = il_env;
        o.row_il = std::min(o.row_il, rows_out / 2);
        if (il_env < 0 && o.row_il < 4) o.row_il = 0;  // (little to gain where rows already start close to the right lag)
    }
    const int rows_grid = o.row_il > 1 ? (rows_out + o.row_il - 1) / o.row_il * o.row_il : rows_out;
    const int xg_per = o.y_phases > 0 ? (o.x_groups + o.y_phases - 1) / o.y_phases : 0;
    o.blocks = o.y_phases > 0 ? 8LL * xg_per * rows_grid : (long long)o.b_tiles * o.x_groups * rows_out;
    o.row_g = o.row_il > 1 ? (rows_out + o.row_il - 1) / o.row_il : 1;
    o.row_g_magic = o.row_g > 1 ? 0xffffffffu / (unsigned)o.row_g + 1u : 0u;
    o.ok = o.blocks <= 0x7fffffffLL;
    if (o.y_phases > 0) {
        o.ok = o.ok && xg_per <= 65535 && rows_grid <= 65535;
        o.grid = dim3(8u, (unsigned)std::max(1, xg_per), (unsigned)std::max(1, rows_grid));
        if (o.row_il > 1 && o.ok)
            for (int y = 0; y < rows_grid; ++y)
                o.ok = o.ok && (int)(((unsigned long long)(unsigned)y * o.row_g_magic) >> 32) == y / o.row_g;
    } else {
        o.grid = dim3((unsigned)std::max(1LL, o.blocks));
    }
    return o;
}

static int inconv128_run(const tcbnn_inconv128_desc* d, void* stream, char* name_buf, size_t name_len) {
    TCBNN_NOTNULL(d);
    if (name_buf == nullptr) {
        TCBNN_NOTNULL(d->input);
        TCBNN_NOTNULL(d->filter);
        TCBNN_NOTNULL(d->bn);
        TCBNN_NOTNULL(d->output);
    }
    TCBNN_REQUIRE(d->input_channels == 3,
                  "inconv128: the first layer takes 3 input channels (kernel.cuh:620-625)");
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0 && d->batch > 0 &&
                      d->output_channels > 0 && d->filter_height > 0 && d->filter_width > 0 &&
                      d->stride_height > 0 && d->stride_width > 0 && d->pool_height > 0 &&
                      d->pool_width > 0,
                  "inconv128: bad shape");
    if (d->save_residual) {
        if (name_buf == nullptr) TCBNN_NOTNULL(d->output_residual);
        TCBNN_REQUIRE(d->pool_height == 1 && d->pool_width == 1,
                      "inconv128: save_residual requires pool 1x1");
    }
    InConvParams p;
    p.in = d->input;
    p.masks = reinterpret_cast<const uint4*>(d->filter);
    p.bn = d->bn;
    p.out = d->output;
    p.res = d->save_residual ? d->output_residual : nullptr;
    p.res_fmt = d->residual_format;
    TCBNN_REQUIRE(!d->save_residual || residual_format_known(p.res_fmt), "inconv128: unknown residual_format");
    TCBNN_REQUIRE(!d->save_residual || p.res_fmt != TCBNN_RES_I12 || d->batch % 2 == 0,
                  "inconv128: a 12-bit residual needs an even batch");
    p.H = d->input_height;
    p.W = d->input_width;
    p.B = d->batch;
    p.O = d->output_channels;
    p.opad = pad32(p.O);
    p.ow = step32(p.O);
    p.R = d->filter_height;
    p.S = d->filter_width;
    p.stride_h = d->stride_height;
    p.stride_w = d->stride_width;
    p.pad_h = tcbnn_conv_pad(p.H, p.R, p.stride_h, d->padding);
    p.pad_w = tcbnn_conv_pad(p.W, p.S, p.stride_w, d->padding);
    p.pool_h = d->pool_height;
    p.pool_w = d->pool_width;
    p.PH = tcbnn_conv_out(p.H, p.R, p.stride_h, d->padding, 1);
    p.PW = tcbnn_conv_out(p.W, p.S, p.stride_w, d->padding, 1);
    TCBNN_REQUIRE(p.PH > 0 && p.PW > 0, "inconv128: empty output");
    p.OH = (p.PH + p.pool_h - 1) / p.pool_h;
    p.OW = (p.PW + p.pool_w - 1) / p.pool_w;

    const bool pooled = p.pool_h != 1 || p.pool_w != 1;
    const bool tiled = (p.pool_w == 1 || p.pool_w == 2) && (kXT - 1) * p.stride_w + p.S <= kMaxCols;
    const int rows_out = pooled ? p.OH : p.PH;  // rows the workgroups are dealt
    // Row-wise staging needs 32-bit buffer offsets over a workgroup's 64 images; larger images (above 2.7 M pixels)
    // take the linear staging, which TCBNN_INCONV_STAGING=linear also selects (so that tests can reach it).
    static const bool force_linear = getenv("TCBNN_INCONV_STAGING") != nullptr &&
                                     strcmp(getenv("TCBNN_INCONV_STAGING"), "linear") == 0;
    const bool row_staging = !force_linear && 64LL * 3 * p.H * p.W * 4 < (1LL << 31);
    if (d->input_layout == TCBNN_INCONV_INPUT_PACKED) {
        // zero-padded, batch-innermost input (tcbnn_inconv_pack_input): the direct kernel, un-pooled layers only
        TCBNN_REQUIRE(!pooled, "inconv128: a packed input is for un-pooled first layers (pool 1x1)");
        const long long Hp = (long long)(p.PH - 1) * p.stride_h + p.R, Wp = (long long)(p.PW - 1) * p.stride_w + p.S;
        const long long in_bytes = Hp * Wp * p.B * 12;
        TCBNN_REQUIRE(in_bytes < (1LL << 31), "inconv128: packed input of 2 GiB or more");
        if (name_buf != nullptr) {
            snprintf(name_buf, name_len, "inconv_direct_kernel");
            return TCBNN_OK;
        }
        const InConvOrder o = inconv_order(p, false, p.PH);
        TCBNN_REQUIRE(o.ok, "inconv128: grid too large");
        hipLaunchKernelGGL(inconv_direct_kernel, o.grid, dim3(kThreads), 0, (hipStream_t)stream, p,
                           p.in, p.masks, p.bn, p.out, p.res, o.b_tiles, o.x_groups, o.y_phases, o.row_il, (int)Wp,
                           (unsigned)in_bytes, o.row_g, o.row_g_magic);
        TCBNN_LAUNCH_CHECK("inconv_direct_kernel");
        return TCBNN_OK;
    }
    TCBNN_REQUIRE(d->input_layout == TCBNN_INCONV_INPUT_NCHW, "inconv128: unknown input_layout");
    if (name_buf != nullptr) {  // report the kernel instead of launching it
        if (!tiled) {
            snprintf(name_buf, name_len, "inconv_generic_kernel");
            return TCBNN_OK;
        }
        const int ncols = (kXT - 1) * p.stride_w + p.S;
        const int rpw = inconv_segments_per_wave(ncols);
        if (row_staging) {
            const int passes = (3 * 64 + 4 * rpw - 1) / (4 * rpw);
            const int nst = passes <= 4 ? 4 : (passes <= 8 ? 8 : (passes <= 16 ? 16 : 24));
            const bool allin = nst * 4 * rpw == 3 * 64 && p.B % 64 == 0 && p.O % 64 == 0;
            snprintf(name_buf, name_len, "inconv_tiled_kernel<%d, true, %s, %s, %s>", nst, pooled ? "true" : "false",
                     allin ? "true" : "false", allin && inconv_straight_to_lds(nst, ncols) ? "true" : "false");
        } else {
            snprintf(name_buf, name_len, "inconv_tiled_kernel<%d, false, %s, false, false>",
                     (3 * 64 * ncols + kThreads - 1) / kThreads <= 15 ? 15 : 24, pooled ? "true" : "false");
        }
        return TCBNN_OK;
    }
    if (tiled) {
        // e / ncols == (e * magic) >> 16 for every e the staging loop uses
        const int ncols = (kXT - 1) * p.stride_w + p.S;
        const int div_magic = 65536 / ncols + 1;
        for (int e = 0; e < 3 * 64 * ncols; ++e)
            TCBNN_REQUIRE((int)(((unsigned)e * (unsigned)div_magic) >> 16) == e / ncols,
                          "inconv128: internal error (division constant)");
        const InConvOrder o = inconv_order(p, pooled, rows_out);
        TCBNN_REQUIRE(o.ok, "inconv128: grid too large");
        // staging scheme (see the kernel and inconv_segments_per_wave; ncols <= kMaxCols = 32)
        const int rpw = inconv_segments_per_wave(ncols);
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, o.grid, dim3(kThreads), 0, (hipStream_t)stream, p, p.in,
                               p.masks, p.bn, p.out, p.res, o.b_tiles, o.x_groups, o.y_phases, div_magic, rpw, o.row_il,
                               rows_out, o.row_g, o.row_g_magic);
        };
        auto launch_nst = [&](auto nst_tag, auto rows_tag) {
            constexpr int NST = decltype(nst_tag)::value;
            constexpr bool ROWS = decltype(rows_tag)::value;
            if constexpr (ROWS) {
                if (NST * 4 * rpw == 3 * 64 && p.B % 64 == 0 && p.O % 64 == 0) {
                    if constexpr (inconv_straight_to_lds(NST, 0)) {
                        if (inconv_straight_to_lds(NST, ncols)) {
                            if (pooled) return launch(inconv_tiled_kernel<NST, true, true, true, true>);
                            return launch(inconv_tiled_kernel<NST, true, false, true, true>);
                        }
                    }
                    if (pooled) return launch(inconv_tiled_kernel<NST, true, true, true>);
                    return launch(inconv_tiled_kernel<NST, true, false, true>);
                }
            }
            if (pooled)
                launch(inconv_tiled_kernel<NST, ROWS, true, false>);
            else
                launch(inconv_tiled_kernel<NST, ROWS, false, false>);
        };
        if (row_staging) {
            const int passes = (3 * 64 + 4 * rpw - 1) / (4 * rpw);
            if (passes <= 4)
                launch_nst(std::integral_constant<int, 4>{}, std::true_type{});
            else if (passes <= 8)
                launch_nst(std::integral_constant<int, 8>{}, std::true_type{});
            else if (passes <= 16)
                launch_nst(std::integral_constant<int, 16>{}, std::true_type{});
            else
                launch_nst(std::integral_constant<int, 24>{}, std::true_type{});
        } else {
            const int nst = (3 * 64 * ncols + kThreads - 1) / kThreads;
            if (nst <= 15)
                launch_nst(std::integral_constant<int, 15>{}, std::false_type{});
            else
                launch_nst(std::integral_constant<int, 24>{}, std::false_type{});
        }
        TCBNN_LAUNCH_CHECK("inconv_tiled_kernel");
        return TCBNN_OK;
    }
    const long long total = (long long)p.B * p.OH * p.OW;
    const long long blocks = (total + kThreads - 1) / kThreads;
    TCBNN_REQUIRE(blocks <= 0x7fffffffLL, "inconv128: grid too large");
    hipLaunchKernelGGL(inconv_generic_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                       (hipStream_t)stream, p);
    TCBNN_LAUNCH_CHECK("inconv_generic_kernel");
    return TCBNN_OK;
}

extern "C" size_t tcbnn_inconv_packed_input_floats(int batch, int height, int width, int filter_height,
                                                   int filter_width, int stride_height, int stride_width, int padding) {
    if (batch <= 0 || height <= 0 || width <= 0 || filter_height <= 0 || filter_width <= 0 || stride_height <= 0 ||
        stride_width <= 0)
        return 0;
    const long long ph = tcbnn_conv_out(height, filter_height, stride_height, padding, 1);
    const long long pw = tcbnn_conv_out(width, filter_width, stride_width, padding, 1);
    if (ph <= 0 || pw <= 0) return 0;
    return (size_t)(((ph - 1) * stride_height + filter_height) * ((pw - 1) * stride_width + filter_width)) *
           (size_t)batch * 3;
}

extern "C" int tcbnn_inconv_pack_input(const float* input, float* packed, int batch, int height, int width,
                                       int filter_height, int filter_width, int stride_height, int stride_width,
                                       int padding, void* stream) {
    TCBNN_NOTNULL(input);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(tcbnn_inconv_packed_input_floats(batch, height, width, filter_height, filter_width, stride_height,
                                                   stride_width, padding) > 0,
                  "inconv_pack_input: bad shape");
    const int ph = tcbnn_conv_out(height, filter_height, stride_height, padding, 1);
    const int pw = tcbnn_conv_out(width, filter_width, stride_width, padding, 1);
    const int Hp = (ph - 1) * stride_height + filter_height, Wp = (pw - 1) * stride_width + filter_width;
    const int pad_h = tcbnn_conv_pad(height, filter_height, stride_height, padding);
    const int pad_w = tcbnn_conv_pad(width, filter_width, stride_width, padding);
    const int b_tiles = (batch + 63) / 64;
    TCBNN_REQUIRE(b_tiles <= 65535 && (Wp + 63) / 64 <= 65535, "inconv_pack_input: batch or width too large");
    hipLaunchKernelGGL(inconv_pack_input_kernel, dim3((unsigned)Hp, (unsigned)b_tiles, (unsigned)((Wp + 63) / 64)), dim3(256), 0,
                       (hipStream_t)stream, input, packed, batch, height, width, Hp, Wp, pad_h, pad_w);
    TCBNN_LAUNCH_CHECK("inconv_pack_input_kernel");
    return TCBNN_OK;
}

extern "C" int tcbnn_inconv128_forward(const tcbnn_inconv128_desc* d, void* stream) {
    return inconv128_run(d, stream, nullptr, 0);
}

extern "C" int tcbnn_inconv128_kernel_name(const tcbnn_inconv128_desc* d, char* buf, size_t len) {
    TCBNN_NOTNULL(buf);
    TCBNN_REQUIRE(len > 0, "kernel_name: empty buffer");
    return inconv128_run(d, nullptr, buf, len);
}
