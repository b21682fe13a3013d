// Binarise / pack / unpack / layout-conversion kernels (HBM-bound byte work).
// Packing rule everywhere: bit = (value >= 0), element e of a 32-group is bit
// (31 - e) of its word, pad bits are 0 (kernel.cuh:165-170, param.h:58-61).
#include "common.h"
#include "mfma_util.h"

namespace tcbnn {
namespace {

constexpr int kThreads = 256;

inline unsigned blocks_for(long long n, int per_block = kThreads) {
    long long b = (n + per_block - 1) / per_block;
    if (b < 1) b = 1;
    return (unsigned)b;
}

// One wave binarises 64 consecutive elements of one row with a ballot:
// a fully coalesced 256-byte read yields two MSB-first words.
// src element (row, k) at src[row*row_stride + k*k_stride]; word (row, w) goes to
// dst[row*dst_row_stride + w*dst_word_stride].
__global__ __launch_bounds__(kThreads) void pack_rows_kernel(const float* __restrict__ src,
                                                             uint32_t* __restrict__ dst,
                                                             long long rows, int k,
                                                             long long row_stride,
                                                             long long k_stride, int k_words,
                                                             long long dst_row_stride,
                                                             long long dst_word_stride) {
    const int lane = threadIdx.x & 63;
    const long long wave = ((long long)blockIdx.x * kThreads + threadIdx.x) >> 6;
    const int segs = (k_words + 1) >> 1;  // 64-element segments per row
    if (wave >= rows * segs) return;
    const long long row = wave / segs;
    const int seg = (int)(wave - row * segs);
    const int kk = seg * 64 + lane;
    const float f = kk < k ? src[row * row_stride + kk * k_stride] : -1.0f;
    const unsigned long long m = __ballot(f >= 0.0f);
    if (lane == 0) {
        uint32_t* d = dst + row * dst_row_stride;
        d[(2 * seg) * dst_word_stride] = __brev((unsigned)(m & 0xffffffffull));
        if (2 * seg + 1 < k_words) d[(2 * seg + 1) * dst_word_stride] = __brev((unsigned)(m >> 32));
    }
}

// Clears n words.  A kernel rather than a memset call: memset nodes recorded into a captured HIP graph
// have misbehaved on replay, and a caller may capture its set-up.
__global__ __launch_bounds__(kThreads) void clear_words_kernel(uint32_t* __restrict__ dst, long long n) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx < n) dst[idx] = 0u;
}

// In128LayerFMT (kernel.cuh:153-172): fp32 [B][K] row major -> sign bits [KW128][B].  One thread per
// (word, image): consecutive lanes are consecutive images, so the packed words are written as
// contiguous runs, and each lane reads its own 128 contiguous bytes (one cache line) with four
// 128-bit loads when the rows are 16-byte aligned.
__global__ void in128_kernel(const float* __restrict__ x, uint32_t* __restrict__ out, int batch, int k, int kw) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= (long long)kw * batch) return;
    const int b = (int)(idx % batch);
    const int w = (int)(idx / batch);
    const float* row = x + (size_t)b * k + 32 * w;
    uint32_t word = 0;
    if (32 * w + 32 <= k && k % 4 == 0) {
        const float4* r4 = reinterpret_cast<const float4*>(row);
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const float4 v = r4[q];
            word = (word << 4) | (v.x >= 0.0f ? 8u : 0u) | (v.y >= 0.0f ? 4u : 0u) | (v.z >= 0.0f ? 2u : 0u) |
                   (v.w >= 0.0f ? 1u : 0u);
        }
    } else {
        for (int e = 0; e < 32; ++e)
            if (32 * w + e < k && row[e] >= 0.0f) word |= 1u << (31 - e);
    }
    out[idx] = word;
}

// HWIO fp32 filter -> [opad32][R*S][cw]; one thread per output word.
__global__ void pack_conv_filter_kernel(const float* __restrict__ f, uint32_t* __restrict__ dst,
                                        int taps, int in_ch, int out_ch, int cw, int opad) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= (long long)opad * taps * cw) return;
    const int w = (int)(idx % cw);
    const int t = (int)((idx / cw) % taps);
    const int o = (int)(idx / ((long long)cw * taps));
    uint32_t word = 0;
    if (o < out_ch) {
        for (int e = 0; e < 32; ++e) {
            const int c = w * 32 + e;
            if (c < in_ch && f[((size_t)t * in_ch + c) * out_ch + o] >= 0.0f) word |= 1u << (31 - e);
        }
    }
    dst[idx] = word;
}

// Sign-bit rows [opad32][9*cw] of a 3x3 filter -> the same words in the order the persistent kernel's lanes expand
// them into FP4 MFMA "A" fragments, uint32 [opad32/32][9*cw/2][64]: lane (j = lane % 32, h = lane / 32) of step
// q = tap * cw/2 + t holds word tap*cw + 2t + h of channel 32*tile + row_to_channel(j), so that a wave stages a
// fragment with one contiguous 256-byte load.
__global__ void permute_conv_filter_kernel(const uint32_t* __restrict__ bits, uint32_t* __restrict__ frag_bits,
                                           int cw, long long total) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int lane = (int)(idx & 63);
    const int nq = 9 * cw / 2;
    const int q = (int)((idx >> 6) % nq);
    const int tile = (int)((idx >> 6) / nq);
    const int j = lane & 31, h = lane >> 5;
    const int tap = q / (cw / 2), t = q % (cw / 2);
    const int c = tile * 32 + mfma::row_to_channel(j);
    frag_bits[idx] = bits[(size_t)c * 9 * cw + tap * cw + 2 * t + h];
}

// Re-orders packed FC weights (rows[neuron][kw], neurons padded to 32, written) into the lane order of the FP4 FC
// kernel: uint32 [npad/32][groups][64][4]; lane (j, h) of group g holds words 8g + 4h + i (i = 0..3) of neuron
// 32 tile + row_to_channel(j), zero past kw.
__global__ void permute_fc_weight_kernel(const uint32_t* __restrict__ rows, uint32_t* __restrict__ lanes, int kw,
                                         long long total) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= total) return;
    const int i = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
    const int groups = (kw + 7) / 8;
    const int g = (int)((idx >> 8) % groups);
    const long long tile = (idx >> 8) / groups;
    const int j = lane & 31, h = lane >> 5;
    const int w = 8 * g + 4 * h + i;
    lanes[idx] = w < kw ? rows[(size_t)(tile * 32 + mfma::row_to_channel(j)) * kw + w] : 0u;
}

// HWIO fp32 [R*S][3][O] -> two tables:
//   [R*S][opad32][4]  sign masks of the three input channels (0x80000000 where the weight is
//                     negative) and, in the 4th word, the sign pattern 4*neg0 + 2*neg1 + neg2;
//   [R*S][opad32]     the same patterns, one per word, contiguous (read with wide scalar loads).
__global__ void pack_inconv_filter_kernel(const float* __restrict__ f, uint32_t* __restrict__ dst,
                                          int taps, int in_ch, int out_ch, int opad) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    const long long n_mask = (long long)taps * opad * 4;
    if (idx >= n_mask + (long long)taps * opad) return;
    if (idx >= n_mask) {  // pattern table
        const long long j = idx - n_mask;
        const int t = (int)(j / opad);
        const int oo = (int)(j % opad);
        uint32_t pat = 0;
        for (int cc = 0; cc < 3; ++cc) {
            const float v = oo < out_ch ? f[((size_t)t * in_ch + cc) * out_ch + oo] : -1.0f;
            pat = pat * 2 + (v >= 0.0f ? 0u : 1u);
        }
        dst[idx] = pat;
        return;
    }
    const int c = (int)(idx & 3);
    const int o = (int)((idx >> 2) % opad);
    const int t = (int)((idx >> 2) / opad);
    // padded outputs behave like the reference's -1.0f fill (param.h:626-627)
    auto negative = [&](int cc) {
        const float v = o < out_ch ? f[((size_t)t * in_ch + cc) * out_ch + o] : -1.0f;
        return v >= 0.0f ? 0u : 1u;
    };
    uint32_t m;
    if (c < 3)
        m = negative(c) << 31;
    else
        m = 4u * negative(0) + 2u * negative(1) + negative(2);
    dst[idx] = m;
}

// NHWC fp32 -> [H][W][cw][B]; one thread per output word.
__global__ void pack_conv_input_nhwc_kernel(const float* __restrict__ src,
                                            uint32_t* __restrict__ dst, int batch, int height,
                                            int width, int ch, int cw) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    const long long total = (long long)height * width * batch * cw;
    if (idx >= total) return;
    const int b = (int)(idx % batch);
    const int w = (int)((idx / batch) % cw);
    const long long pix = idx / ((long long)cw * batch);
    const float* s = src + ((size_t)b * height * width + pix) * ch + w * 32;
    uint32_t word = 0;
    for (int e = 0; e < 32 && w * 32 + e < ch; ++e)
        if (s[e] >= 0.0f) word |= 1u << (31 - e);
    dst[idx] = word;
}

__global__ void unpack_fc_kernel(const uint32_t* __restrict__ packed, float* __restrict__ out,
                                 int batch, int features, int kw) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= (long long)batch * features) return;
    const int k = (int)(idx % features);
    const long long b = idx / features;
    const uint32_t w = packed[(long long)(k >> 5) * batch + b];
    out[idx] = 2.0f * (float)((w >> (31 - (k & 31))) & 1u) - 1.0f;
}

__global__ void unpack_conv_kernel(const uint32_t* __restrict__ packed, float* __restrict__ out,
                                   int height, int width, int ch, int batch, int cw) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;  // NHWC index
    const long long total = (long long)batch * height * width * ch;
    if (idx >= total) return;
    const int c = (int)(idx % ch);
    const long long pix = (idx / ch) % ((long long)height * width);
    const long long b = idx / ((long long)ch * height * width);
    const uint32_t w = packed[(pix * cw + (c >> 5)) * batch + b];
    out[idx] = 2.0f * (float)((w >> (31 - (c & 31))) & 1u) - 1.0f;
}

// engine [groups][row_words][rows] <-> reference tiles [groups][ceil(rows/8)][row128][8][4]
// where `groups` is the number of leading (pixel) blocks, each holding `rows` rows.
// to_fmt != 0: fmt is written (zero where the engine has no word); else packed is written.
__global__ void fmt_convert_kernel(uint32_t* __restrict__ packed, uint32_t* __restrict__ fmt,
                                   long long groups, int rows, int row_words, int row128,
                                   int to_fmt) {
    const int rows8 = (rows + 7) >> 3;
    const long long per_group = (long long)rows8 * row128 * 32;
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;  // fmt index
    if (idx >= groups * per_group) return;
    const long long g = idx / per_group;
    const int rem = (int)(idx - g * per_group);
    const int w = rem & 3;
    const int r = (rem >> 2) & 7;
    const int tile = rem >> 5;
    const int kc = tile % row128;
    const int rt = tile / row128;
    const int row = rt * 8 + r;
    const int word = kc * 4 + w;
    const bool has = row < rows && word < row_words;
    const long long pidx = (g * row_words + word) * rows + row;
    if (to_fmt)
        fmt[idx] = has ? packed[pidx] : 0u;
    else if (has)
        packed[pidx] = fmt[idx];
}

__global__ void residual_to_reference_kernel(const int32_t* __restrict__ res,
                                             int32_t* __restrict__ ref, long long pixels,
                                             int batch, int ch, int b8, int c128, int fmt) {
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= pixels * b8 * c128) return;
    const int c = (int)(idx % c128);
    const int b = (int)((idx / c128) % b8);
    const long long pix = idx / ((long long)c128 * b8);
    ref[idx] = (b < batch && c < ch) ? residual_load(res, fmt, (size_t)pix, ch, c, batch, b) : 0;
}

// One thread per 16-byte group of the engine's layouts (4 int32 or 8 int16 channels of one image and pixel);
// channels past `ch` are stored as 0, which is what the consumers of the padding lanes expect.
__global__ void residual_from_reference_kernel(const int32_t* __restrict__ ref, int32_t* __restrict__ res,
                                               long long pixels, int batch, int ch, int b8, int c128, int fmt) {
    const int per = (int)residual_group_channels(fmt);
    const int groups = (ch + per - 1) / per;
    const long long idx = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= pixels * groups * batch) return;
    const int b = (int)(idx % batch);
    const int g = (int)((idx / batch) % groups);
    const long long pix = idx / ((long long)batch * groups);
    const int32_t* src = ref + ((size_t)pix * b8 + b) * c128 + (size_t)g * per;
    if (fmt == TCBNN_RES_I12) {  // one thread per group of 16 channels
        int v16[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v16[i] = g * 16 + i < ch ? src[i] : 0;
        residual_store_group16(res, fmt, (size_t)pix, ch, g, batch, b, v16);
        return;
    }
    int v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (i < per && g * per + i < ch) ? src[i] : 0;
    int4 o;
    if (fmt == TCBNN_RES_I16)
        o = make_int4((v[0] & 0xffff) | (v[1] << 16), (v[2] & 0xffff) | (v[3] << 16), (v[4] & 0xffff) | (v[5] << 16),
                      (v[6] & 0xffff) | (v[7] << 16));
    else
        o = make_int4(v[0], v[1], v[2], v[3]);
    reinterpret_cast<int4*>(res)[idx] = o;  // [pix][group][b] is the linear order of both layouts
}

}  // namespace
}  // namespace tcbnn

using namespace tcbnn;

extern "C" {

int tcbnn_pack_rows(const float* src, uint32_t* packed, int rows, int k, int ld, int k_words,
                    void* stream) {
    TCBNN_NOTNULL(src);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(rows > 0 && k > 0 && ld >= k && k_words >= step32(k), "pack_rows: bad shape");
    const long long waves = (long long)rows * ((k_words + 1) / 2);
    hipLaunchKernelGGL(pack_rows_kernel, dim3(blocks_for(waves * 64)), dim3(kThreads), 0,
                       (hipStream_t)stream, src, packed, (long long)rows, k, (long long)ld, 1LL,
                       k_words, 1LL, (long long)rows);
    TCBNN_LAUNCH_CHECK("pack_rows_kernel");
    return TCBNN_OK;
}

int tcbnn_pack_cols(const float* src, uint32_t* packed, int k, int n, int k_words, void* stream) {
    TCBNN_NOTNULL(src);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(k > 0 && n > 0 && k_words >= step32(k), "pack_cols: bad shape");
    const long long waves = (long long)n * ((k_words + 1) / 2);
    hipLaunchKernelGGL(pack_rows_kernel, dim3(blocks_for(waves * 64)), dim3(kThreads), 0,
                       (hipStream_t)stream, src, packed, (long long)n, k, 1LL, (long long)n,
                       k_words, (long long)k_words, 1LL);
    TCBNN_LAUNCH_CHECK("pack_cols_kernel");
    return TCBNN_OK;
}

int tcbnn_pack_fc_weight(const float* weight_kn, uint32_t* packed, int in_features,
                         int out_features, void* stream) {
    TCBNN_NOTNULL(weight_kn);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(in_features > 0 && out_features > 0, "pack_fc_weight: bad shape");
    const int kw = kw128(in_features);
    const int npad = pad32(out_features);
    // rows of the padding neurons (the rest is written by the packing kernel)
    const long long pad_words = (long long)(npad - out_features) * kw;
    if (pad_words > 0) {
        hipLaunchKernelGGL(clear_words_kernel, dim3(blocks_for(pad_words)), dim3(kThreads), 0, (hipStream_t)stream,
                           packed + (size_t)out_features * kw, pad_words);
        TCBNN_LAUNCH_CHECK("clear_words_kernel");
    }
    if (int rc = tcbnn_pack_cols(weight_kn, packed, in_features, out_features, kw, stream)) return rc;
    const long long lane_words = (long long)fc_weight_lane_words(npad, kw);
    hipLaunchKernelGGL(permute_fc_weight_kernel, dim3(blocks_for(lane_words)), dim3(kThreads), 0, (hipStream_t)stream,
                       packed, packed + fc_weight_row_words(npad, kw), kw, lane_words);
    TCBNN_LAUNCH_CHECK("permute_fc_weight_kernel");
    return TCBNN_OK;
}

int tcbnn_pack_conv_filter(const float* filter_hwio, uint32_t* packed, int r, int s, int in_ch,
                           int out_ch, void* stream) {
    TCBNN_NOTNULL(filter_hwio);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(r > 0 && s > 0 && in_ch > 0 && out_ch > 0, "pack_conv_filter: bad shape");
    const int cw = step32(in_ch), opad = pad32(out_ch);
    const long long total = (long long)opad * r * s * cw;
    hipLaunchKernelGGL(pack_conv_filter_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, filter_hwio, packed, r * s, in_ch, out_ch, cw, opad);
    TCBNN_LAUNCH_CHECK("pack_conv_filter_kernel");
    if (filter_has_fragments(r, s, in_ch)) {
        const long long frags = (long long)(opad / 32) * (9 * cw / 2) * 64;  // == total
        hipLaunchKernelGGL(permute_conv_filter_kernel, dim3(blocks_for(frags)), dim3(kThreads), 0, (hipStream_t)stream,
                           packed, packed + total, cw, frags);
        TCBNN_LAUNCH_CHECK("permute_conv_filter_kernel");
    }
    return TCBNN_OK;
}

int tcbnn_pack_inconv_filter(const float* filter_hwio, uint32_t* packed, int r, int s, int in_ch,
                             int out_ch, void* stream) {
    TCBNN_NOTNULL(filter_hwio);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(r > 0 && s > 0 && out_ch > 0, "pack_inconv_filter: bad shape");
    TCBNN_REQUIRE(in_ch == 3, "first-layer convolution has 3 input channels (kernel.cuh:620-625)");
    const int opad = pad32(out_ch);
    const long long total = (long long)r * s * opad * 5;
    hipLaunchKernelGGL(pack_inconv_filter_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, filter_hwio, packed, r * s, in_ch, out_ch, opad);
    TCBNN_LAUNCH_CHECK("pack_inconv_filter_kernel");
    return TCBNN_OK;
}

int tcbnn_pack_conv_input_nhwc(const float* src, uint32_t* packed, int batch, int height,
                               int width, int ch, void* stream) {
    TCBNN_NOTNULL(src);
    TCBNN_NOTNULL(packed);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0, "pack_conv_input: bad shape");
    const int cw = step32(ch);
    const long long total = (long long)height * width * batch * cw;
    hipLaunchKernelGGL(pack_conv_input_nhwc_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, src, packed, batch, height, width, ch, cw);
    TCBNN_LAUNCH_CHECK("pack_conv_input_nhwc_kernel");
    return TCBNN_OK;
}

int tcbnn_in128_forward(const tcbnn_in128_desc* d, void* stream) {
    TCBNN_NOTNULL(d);
    TCBNN_NOTNULL(d->input);
    TCBNN_NOTNULL(d->output);
    TCBNN_REQUIRE(d->input_height > 0 && d->input_width > 0, "in128: bad shape");
    const int kw = kw128(d->input_width);
    const long long total = (long long)kw * d->input_height;
    hipLaunchKernelGGL(in128_kernel, dim3(blocks_for(total)), dim3(kThreads), 0, (hipStream_t)stream, d->input,
                       d->output, d->input_height, d->input_width, kw);
    TCBNN_LAUNCH_CHECK("in128_kernel");
    return TCBNN_OK;
}

int tcbnn_unpack_fc_output(const uint32_t* packed, float* out, int batch, int features,
                           void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(out);
    TCBNN_REQUIRE(batch > 0 && features > 0, "unpack_fc: bad shape");
    hipLaunchKernelGGL(unpack_fc_kernel, dim3(blocks_for((long long)batch * features)),
                       dim3(kThreads), 0, (hipStream_t)stream, packed, out, batch, features,
                       kw128(features));
    TCBNN_LAUNCH_CHECK("unpack_fc_kernel");
    return TCBNN_OK;
}

int tcbnn_unpack_conv_output(const uint32_t* packed, float* out, int height, int width, int ch,
                             int batch, void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(out);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0, "unpack_conv: bad shape");
    const long long total = (long long)batch * height * width * ch;
    hipLaunchKernelGGL(unpack_conv_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, packed, out, height, width, ch, batch, step32(ch));
    TCBNN_LAUNCH_CHECK("unpack_conv_kernel");
    return TCBNN_OK;
}

static int fmt_convert(uint32_t* packed, uint32_t* fmt, long long groups, int rows, int row_words,
                       int row128, int to_fmt, void* stream) {
    const long long total = groups * ((rows + 7) / 8) * row128 * 32;
    hipLaunchKernelGGL(fmt_convert_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, packed, fmt, groups, rows, row_words, row128, to_fmt);
    TCBNN_LAUNCH_CHECK("fmt_convert_kernel");
    return TCBNN_OK;
}

int tcbnn_fc_to_reference_fmt(const uint32_t* packed, uint32_t* fmt, int batch, int features,
                              void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(fmt);
    TCBNN_REQUIRE(batch > 0 && features > 0, "fc_to_reference_fmt: bad shape");
    return fmt_convert(const_cast<uint32_t*>(packed), fmt, 1, batch, kw128(features),
                       step128(features), 1, stream);
}
int tcbnn_fc_from_reference_fmt(const uint32_t* fmt, uint32_t* packed, int batch, int features,
                                void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(fmt);
    TCBNN_REQUIRE(batch > 0 && features > 0, "fc_from_reference_fmt: bad shape");
    return fmt_convert(packed, const_cast<uint32_t*>(fmt), 1, batch, kw128(features),
                       step128(features), 0, stream);
}
int tcbnn_conv_to_reference_fmt(const uint32_t* packed, uint32_t* fmt, int height, int width,
                                int batch, int ch, void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(fmt);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0, "conv_to_reference_fmt: bad shape");
    return fmt_convert(const_cast<uint32_t*>(packed), fmt, (long long)height * width, batch,
                       step32(ch), step128(ch), 1, stream);
}
int tcbnn_conv_from_reference_fmt(const uint32_t* fmt, uint32_t* packed, int height, int width,
                                  int batch, int ch, void* stream) {
    TCBNN_NOTNULL(packed);
    TCBNN_NOTNULL(fmt);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0,
                  "conv_from_reference_fmt: bad shape");
    return fmt_convert(packed, const_cast<uint32_t*>(fmt), (long long)height * width, batch,
                       step32(ch), step128(ch), 0, stream);
}

int tcbnn_residual_to_reference(const int32_t* res, int32_t* ref, int height, int width, int batch,
                                int ch, int format, void* stream) {
    TCBNN_NOTNULL(res);
    TCBNN_NOTNULL(ref);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0, "residual_to_reference: bad shape");
    TCBNN_REQUIRE(residual_format_known(format), "residual_to_reference: unknown format");
    TCBNN_REQUIRE(format != TCBNN_RES_I12 || batch % 2 == 0, "residual_to_reference: a 12-bit residual needs an even batch");
    const long long pixels = (long long)height * width;
    const long long total = pixels * pad8(batch) * pad128(ch);
    hipLaunchKernelGGL(residual_to_reference_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, res, ref, pixels, batch, ch, pad8(batch), pad128(ch), format);
    TCBNN_LAUNCH_CHECK("residual_to_reference_kernel");
    return TCBNN_OK;
}

int tcbnn_residual_from_reference(const int32_t* ref, int32_t* res, int height, int width, int batch,
                                  int ch, int format, void* stream) {
    TCBNN_NOTNULL(ref);
    TCBNN_NOTNULL(res);
    TCBNN_REQUIRE(batch > 0 && height > 0 && width > 0 && ch > 0, "residual_from_reference: bad shape");
    TCBNN_REQUIRE(residual_format_known(format), "residual_from_reference: unknown format");
    TCBNN_REQUIRE(format != TCBNN_RES_I12 || batch % 2 == 0, "residual_from_reference: a 12-bit residual needs an even batch");
    const long long pixels = (long long)height * width;
    const int per = (int)residual_group_channels(format);
    const long long total = pixels * ((ch + per - 1) / per) * batch;
    hipLaunchKernelGGL(residual_from_reference_kernel, dim3(blocks_for(total)), dim3(kThreads), 0,
                       (hipStream_t)stream, ref, res, pixels, batch, ch, pad8(batch), pad128(ch), format);
    TCBNN_LAUNCH_CHECK("residual_from_reference_kernel");
    return TCBNN_OK;
}

}  // extern "C"
