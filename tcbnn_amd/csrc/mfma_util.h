// Device helpers shared by the matrix-core kernels: +-1 bit expansion to FP4 / int8 MFMA
// operands, the MFMA wrappers, and the accumulator-row -> channel permutation.
#pragma once

#include "common.h"

namespace tcbnn {
namespace mfma {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int FMT_F4 = 0;
constexpr int FMT_I8 = 1;
enum MfmaMode : int { MM_THRESH = 0, MM_THRESH_RES = 1, MM_OTHER = 2 };

// ---- bit expansion ----------------------------------------------------------------
// FP4: bit value 1 -> nibble 0xA (-1.0), 0 -> 0x2 (+1.0): the sign is flipped for BOTH
// operands, so products are unchanged.  dword j takes bits {4p + (3-j)}.
// One v_bfi_b32 per dword: D = (M & shifted) | (~M & C) with M = 0x88888888 (sign bit of every
// nibble) and C = 0x22222222 (+1.0 in every nibble), plus the shift: 7 VALU ops per 32 values.
// Written as asm because two different 32-bit constants do not fit one VOP3 instruction otherwise
// (the compiler falls back to shift + and + or).
__device__ __forceinline__ int bfi_sign_nibbles(uint32_t shifted) {
    int d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(0x88888888u), "v"(shifted), "v"(0x22222222u));
    return d;
}
__device__ __forceinline__ v4i expand_f4(uint32_t x) {
    v4i r;
    r[0] = bfi_sign_nibbles(x << 3);
    r[1] = bfi_sign_nibbles(x << 2);
    r[2] = bfi_sign_nibbles(x << 1);
    r[3] = bfi_sign_nibbles(x);
    return r;
}
// nibbles whose bit is not `valid` become FP4 zero
__device__ __forceinline__ v4i expand_f4_masked(uint32_t x, uint32_t valid) {
    v4i r = expand_f4(x);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t t = ((valid << (3 - j)) & 0x88888888u) >> 3;  // 0x1 per valid nibble
        r[j] &= (int)(t * 15u);
    }
    return r;
}
// int8: lane half h of a 32-bit word takes bits {q + 4h + 8p}; bit 1 -> 0x01, bit 0 -> 0xFF
__device__ __forceinline__ v4i expand_i8(uint32_t x, int h) {
    v4i r;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t d = (x >> (q + 4 * h)) & 0x01010101u;
        const uint32_t m = (d << 8) - d;  // 0xFF in every byte whose bit is set
        r[q] = (int)(~m | 0x01010101u);
    }
    return r;
}
__device__ __forceinline__ v4i expand_i8_masked(uint32_t x, uint32_t valid, int h) {
    v4i r = expand_i8(x, h);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t d = (valid >> (q + 4 * h)) & 0x01010101u;
        r[q] &= (int)((d << 8) - d);
    }
    return r;
}

// ---- shift-free FP4 expansion of the activation ("row") operand ---------------------
// FP4 E2M1 has, for every bit position j of a nibble, a pair of values that differ in that bit alone and by exactly
// 2:  bit 3: +1.0 / -1.0 (0010 / 1010),  bit 2: 0 / 2 (0000 / 0100),  bit 1: 2 / 4 (0100 / 0110),  bit 0: 4 / 6
// (0110 / 0111).  So dword j of the operand is (x & 0x1111.. << j) | c_j: the word's bits of class j (positions
// 4p + j) stay where they are, one bit-field insert per dword, four instructions per word instead of seven (three
// shifts + four inserts).  The matrix pipeline and the VALU of a SIMD overlap little, so instructions saved here
// are matrix time.  With s = +-1 the value of the row bit, the operand holds -s (class 3) or a_j + s with a_2 = 1,
// a_1 = 3, a_0 = 5.  The weight side (expanded at pack time or once per block, off the critical path) holds -w for
// class 3 and +w for the others, so a product is  w s  (class 3)  or  w s + a_j w:  the accumulator ends as the dot
// product plus  C = sum over classes of a_j (sum of the column's w over the class), a per-column constant that the
// kernels take off again (the large-GEMM kernel counts it while staging, the 3x3 kernel reads a table written at
// pack time).  All products and partial sums are small integers: exact in fp32.
// (Pairs 0 / 0.5 and 0 / 1 with weights +-4 and +-2 need no constants in registers, but measured 8 % slower on the
// 8192^3 product than this choice, which keeps every weight at +-1.)
// One v_bfi_b32 each, D = (mask & x) | (~mask & c); written as asm because the compiler otherwise emits an AND and
// an OR (two 32-bit constants do not fit one VOP3 instruction unless one sits in a vector register).
__device__ __forceinline__ int bfi_keep(uint32_t mask, uint32_t x, uint32_t c) {
    int d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(mask), "v"(x), "v"(c));
    return d;
}
__device__ __forceinline__ v4i expand_rows_f4(uint32_t x) {
    v4i r;
    r[0] = bfi_keep(0x11111111u, x, 0x66666666u);
    r[1] = bfi_keep(0x22222222u, x, 0x44444444u);
    r[2] = (int)(x & 0x44444444u);
    r[3] = bfi_keep(0x88888888u, x, 0x22222222u);
    return r;
}
// weight word -> fragment dwords in the same class order: the sign code of bit 4p + j, flipped for class 3 only
__device__ __forceinline__ v4i expand_weights_f4(uint32_t x) {
    v4i r;
    r[0] = bfi_sign_nibbles(~x << 3);
    r[1] = bfi_sign_nibbles(~x << 2);
    r[2] = bfi_sign_nibbles(~x << 1);
    r[3] = bfi_sign_nibbles(x);
    return r;
}
// a_j-weighted sum of w = +-1 (bit set: +1) over the 24 class-0..2 positions of one weight word
__device__ __forceinline__ int class_sum(uint32_t x) {
    return 2 * (5 * __popc(x & 0x11111111u) + 3 * __popc(x & 0x22222222u) + __popc(x & 0x44444444u)) - 8 * (5 + 3 + 1);
}

template <int FMT>
struct Acc;
template <>
struct Acc<FMT_F4> {
    using type = v16f;
    static __device__ __forceinline__ type mma(v4i a, v4i b, type c) {
        const v8i a8 = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
        const v8i b8 = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
        // cbsz = blgp = 4: both operands FP4; scale operands 0 select the unscaled instruction
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c, 4, 4, 0, 0, 0, 0);
    }
    static __device__ __forceinline__ int to_int(float v) { return (int)v; }
};
template <>
struct Acc<FMT_I8> {
    using type = v16i;
    static __device__ __forceinline__ type mma(v4i a, v4i b, type c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int to_int(int v) { return v; }
};

__device__ __forceinline__ uint32_t thresh_bit(int res, float thr, int nan_bit) {
    const float rf = (float)res;
    return nan_bit ? (rf < thr ? 0u : 1u) : (rf >= thr ? 1u : 0u);
}

// MFMA row i of a channel tile holds channel perm(i), so that accumulator register v of
// lane half h (row 8*(v/4) + 4h + v%4) is channel 16h + v.
__device__ __forceinline__ int row_to_channel(int i) {
    return 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
}

}  // namespace mfma
}  // namespace tcbnn
