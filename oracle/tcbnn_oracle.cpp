// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// CPU restatement (C++17 + OpenMP, XOR / popcount on 64-bit words) of the
// reference's bit-matmul / bit-convolution inference path.  It is the parity
// oracle of the test-suite and the timed CPU baseline of the benchmark; the
// GPU library never links, loads or calls it.
//
// Every function names the reference lines it restates (paths relative to the
// reference checkout).  Nothing here was obtained by running the reference
// (it is CUDA for sm_75 bit tensor cores and cannot be built in this image);
// the test-suite pins each function against mathematics instead:
//   orc_bmm / orc_fc128 / orc_out128   integer matmul on unpacked +-1 (numpy)
//   orc_bconv / orc_conv128            zero-padded cross-correlation on +-1
//                                      (torch.nn.functional.conv2d) + brute force
//   orc_conv_geometry                  closed forms, brute force over (H, s, R)
//   pack / threshold / pool / residual unpack(pack(x)) == sign(x), OR == max,
//                                      invariants of the residual rules
//   orc_inconv128                      fp64 convolution (tolerance on non-tie
//                                      elements) and exact integer sums for
//                                      pre-signed inputs
//   reference "FMT" layout maps        round trip through independently written
//                                      numpy versions of the reference unpack kernels
// Parity unpinned: logits of the reference's *trained* checkpoints (the weight
// files are not shipped with the reference).
//
// Logical layouts (host memory), all MSB first (element e of a 32-group is bit
// 31-e; bit = 1 <=> value >= 0; pad bits 0):
//   FC activations    uint32 [B][KW128]       KW128 = 4*ceil(K/128)
//   conv activations  uint32 [H][W][B][CW]    CW = ceil(C/32)
//   FC weights        uint32 [N][KW128]       row n = column n of the fp32 [K][N] matrix
//   conv filters      uint32 [O][R*S][CW]
//   residuals         int32  [P][Q][B][O]
#include <limits.h>
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <vector>

namespace {

inline int step32(int x) { return (x + 31) >> 5; }    // utility.h:36
inline int step128(int x) { return (x + 127) >> 7; }  // utility.h:38
inline int pad8(int x) { return ((x + 7) >> 3) << 3; }      // utility.h:41
inline int pad128(int x) { return step128(x) << 7; }  // utility.h:45
inline int kw128(int k) { return 4 * step128(k); }

inline int popc32(uint32_t v) { return __builtin_popcount(v); }

// popcount of (a xor w) over n 32-bit words, 64 bits at a time.
inline int xor_popc(const uint32_t* a, const uint32_t* w, int n) {
    int c = 0, i = 0;
    for (; i + 2 <= n; i += 2) {
        uint64_t x, y;
        memcpy(&x, a + i, 8);
        memcpy(&y, w + i, 8);
        c += __builtin_popcountll(x ^ y);
    }
    if (i < n) c += popc32(a[i] ^ w[i]);
    return c;
}

// float -> int as the device does it for `int = float` (cvt, round toward zero,
// saturating, NaN -> 0); kernel.cuh:666-668 stores the fp32 sum into an int array.
inline int32_t f2i_rz_sat(float f) {
    if (f != f) return 0;
    if (f >= 2147483648.0f) return INT_MAX;
    if (f <= -2147483648.0f) return INT_MIN;
    return (int32_t)f;
}

}  // namespace

extern "C" {

int orc_num_threads(void) { return omp_get_max_threads(); }

// param.h:719-728 / 897-906: pad, pre-pool size and pooled output size.
void orc_conv_geometry(int in_size, int filter, int stride, int padding, int pool, int* pad,
                       int* buf, int* out) {
    *pad = padding
               ? ((((in_size + stride - (in_size % stride)) / stride - 1) * stride + filter - in_size) / 2)
               : 0;
    *buf = padding ? (in_size + stride - 1) / stride : ((in_size - filter) / stride + 1);
    *out = (*buf + pool - 1) / pool;
}

// Binarise rows: bit = (x >= 0), MSB first, zero padded to kwords per row
// (kernel.cuh:165-170: out-of-range elements are -1.0f, i.e. bit 0;
// __brev(__ballot) puts element 0 in bit 31).
void orc_pack_rows(const float* x, uint32_t* out, long rows, int k, long ld, int kwords) {
#pragma omp parallel for
    for (long r = 0; r < rows; ++r) {
        for (int w = 0; w < kwords; ++w) {
            uint32_t word = 0;
            for (int e = 0; e < 32; ++e) {
                const int kk = w * 32 + e;
                if (kk < k && x[r * ld + kk] >= 0.0f) word |= 1u << (31 - e);
            }
            out[r * kwords + w] = word;
        }
    }
}

// In128LayerFMT, kernel.cuh:153-172 (logical row-major result).
void orc_in128(const float* x, uint32_t* out, int batch, int k) {
    orc_pack_rows(x, out, batch, k, k, kw128(k));
}

// PackFcWeight128FMT, param.h:44-63: fp32 [K][N] -> one packed row per output n.
void orc_pack_fc_weight(const float* w_kn, uint32_t* out, int k, int n) {
    const int kw = kw128(k);
#pragma omp parallel for
    for (int j = 0; j < n; ++j) {
        for (int w = 0; w < kw; ++w) {
            uint32_t word = 0;
            for (int e = 0; e < 32; ++e) {
                const int kk = w * 32 + e;
                if (kk < k && w_kn[(size_t)kk * n + j] >= 0.0f) word |= 1u << (31 - e);
            }
            out[(size_t)j * kw + w] = word;
        }
    }
}

// PackFiltersByInChannels128FMT, param.h:560-581: HWIO fp32 -> [O][R*S][CW].
void orc_pack_conv_filter(const float* hwio, uint32_t* out, int r, int s, int c, int o) {
    const int cw = step32(c), taps = r * s;
#pragma omp parallel for
    for (int oc = 0; oc < o; ++oc)
        for (int t = 0; t < taps; ++t)
            for (int w = 0; w < cw; ++w) {
                uint32_t word = 0;
                for (int e = 0; e < 32; ++e) {
                    const int ch = w * 32 + e;
                    if (ch < c && hwio[((size_t)t * c + ch) * o + oc] >= 0.0f) word |= 1u << (31 - e);
                }
                out[((size_t)oc * taps + t) * cw + w] = word;
            }
}

// BTC_bin_input, bmma_kernel.cu:73-98: NHWC fp32 -> [H][W][B][CW].
void orc_pack_conv_input_nhwc(const float* x, uint32_t* out, int batch, int h, int w, int c) {
    const int cw = step32(c);
#pragma omp parallel for
    for (long pix = 0; pix < (long)h * w; ++pix)
        for (int b = 0; b < batch; ++b)
            orc_pack_rows(x + ((size_t)b * h * w + pix) * c, out + ((size_t)pix * batch + b) * cw, 1, c,
                          c, cw);
}

// BMMAS / BMMAcpu, tensorcore_kernel.cu:38-57, 305-356: C = K - 2*popc(A xor B).
void orc_bmm(const uint32_t* a, const uint32_t* b, int32_t* c, int m, int n, int k) {
    const int kw = k / 32;
#pragma omp parallel for
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j)
            c[(size_t)i * n + j] = k - 2 * xor_popc(a + (size_t)i * kw, b + (size_t)j * kw, kw);
}

// Fc128LayerFMT, kernel.cuh:174-226.  acc (optional) receives popc sums.
//   bit = ((float)K - 2*(float)c >= bn[n])   (l.210-213), rows>=B / cols>=N are 0.
void orc_fc128(const uint32_t* in, const uint32_t* w, const float* bn, uint32_t* out, int32_t* acc,
               int batch, int k, int n) {
    const int kw = kw128(k), nw = kw128(n);
#pragma omp parallel for
    for (int b = 0; b < batch; ++b) {
        uint32_t* orow = out + (size_t)b * nw;
        for (int i = 0; i < nw; ++i) orow[i] = 0;
        for (int j = 0; j < n; ++j) {
            const int c = xor_popc(in + (size_t)b * kw, w + (size_t)j * kw, kw);
            if (acc) acc[(size_t)b * n + j] = c;
            if ((float)k - 2 * (float)c >= bn[j]) orow[j >> 5] |= 1u << (31 - (j & 31));
        }
    }
}

// Out128LayerFMT, kernel.cuh:230-280:
//   y = ((float)K - (float)c*2.0f)*bn_scale[n] + bn_bias[n]   (l.270-273)
// Built with -ffp-contract=off: multiply and add are separate roundings.
void orc_out128(const uint32_t* in, const uint32_t* w, const float* scale, const float* bias,
                float* out, int batch, int k, int n) {
    const int kw = kw128(k);
#pragma omp parallel for
    for (int b = 0; b < batch; ++b)
        for (int j = 0; j < n; ++j) {
            const int c = xor_popc(in + (size_t)b * kw, w + (size_t)j * kw, kw);
            const float d = (float)k - (float)c * 2.0f;
            const float prod = d * scale[j];
            out[(size_t)b * n + j] = prod + bias[j];
        }
}

// BTC_Conv2d_balance + BTC_trans_output, bmma_kernel.cu:101-165, 247-263:
//   out[b][p][q][o] = Cin*R*S - exclude*Cin - 2*popc over in-frame taps.
void orc_bconv(const uint32_t* in, const uint32_t* filt, int32_t* out, int batch, int h, int w,
               int cin, int cout, int r, int s, int stride_h, int stride_w, int pad_h, int pad_w,
               int oh, int ow) {
    const int cw = step32(cin), taps = r * s;
#pragma omp parallel for collapse(2)
    for (int y = 0; y < oh; ++y)
        for (int x = 0; x < ow; ++x) {
            const int ay0 = y * stride_h - pad_h, ax0 = x * stride_w - pad_w;
            for (int b = 0; b < batch; ++b)
                for (int o = 0; o < cout; ++o) {
                    int exclude = 0, c = 0;
                    for (int rr = 0; rr < r; ++rr)
                        for (int ss = 0; ss < s; ++ss) {
                            const int ay = ay0 + rr, ax = ax0 + ss;
                            if (ay >= 0 && ay < h && ax >= 0 && ax < w)
                                c += xor_popc(in + (((size_t)ay * w + ax) * batch + b) * cw,
                                              filt + ((size_t)o * taps + rr * s + ss) * cw, cw);
                            else
                                ++exclude;
                        }
                    out[(((size_t)b * oh + y) * ow + x) * cout + o] =
                        cin * r * s - exclude * cin - 2 * c;
                }
        }
}

// Conv128LayerFMT, kernel.cuh:676-827.
//   res = Cin*R*S - exclude*Cin - 2*popc                                   l.766-768
//   inject (o < residual_channels): + Rin[y][x][b][o], or the max over the
//     2x2 block (2y+i, 2x+j) of a source twice as large (residual_pool)    l.770-794
//     source channels >= res_in_ch read 0 (zero-filled padding, param.h:979-980)
//   bit = (float)res < bn[o] ? 0 : 1                                        l.795-796
//   OR into pooled pixel (y/pool_h, x/pool_w)                               l.811-815
//   the pixels walked are pool_h*output_height x pool_w*output_width          l.685-690
//     (NOT the pre-pool size): when the pooled size is rounded up, the last windows hold pixels past
//     the convolution's own output; those are computed like any other, from the taps that still lie
//     inside the frame (l.720-757), and their bits are ORed in.  With no tap left the sum is 0.
//     Residuals on such pixels: the reference indexes buffers of output_height*output_width pixels
//     (param.h:925-927) with pre-pool coordinates, i.e. out of bounds whenever pool > 1; here they
//     neither receive nor save a residual (the GPU library rejects residuals on pooled layers).
//   ahead_fc: FC feature index ((y/ph)*OW + x/pw)*PAD128(O) + o             l.798-808
//   save_residual: Rout[y][x][b][o] = res                                   l.818-824
void orc_conv128(const uint32_t* in, const uint32_t* filt, const float* bn, uint32_t* out,
                 const int32_t* res_in, int32_t* res_out, int h, int w, int cin, int cout,
                 int batch, int r, int s, int stride_h, int stride_w, int padding, int pool_h,
                 int pool_w, int ahead_fc, int inject_residual, int residual_channels,
                 int residual_pool, int res_in_ch) {
    int pad_h, pad_w, ph, pw, oh, ow;
    orc_conv_geometry(h, r, stride_h, padding, pool_h, &pad_h, &ph, &oh);
    orc_conv_geometry(w, s, stride_w, padding, pool_w, &pad_w, &pw, &ow);
    const int cw = step32(cin), taps = r * s;
    const int ocw = step32(cout), ocw128 = kw128(cout);
    const size_t out_words =
        ahead_fc ? (size_t)batch * oh * ow * ocw128 : (size_t)oh * ow * batch * ocw;
    memset(out, 0, out_words * 4);
#pragma omp parallel for collapse(2)
    for (int oy = 0; oy < oh; ++oy)
        for (int ox = 0; ox < ow; ++ox)
            for (int py = 0; py < pool_h; ++py)
                for (int px = 0; px < pool_w; ++px) {
                    const int y = oy * pool_h + py, x = ox * pool_w + px;
                    const bool past = y >= ph || x >= pw;  // beyond the convolution's own output
                    const int ay0 = y * stride_h - pad_h, ax0 = x * stride_w - pad_w;
                    for (int b = 0; b < batch; ++b)
                        for (int o = 0; o < cout; ++o) {
                            int exclude = 0, c = 0;
                            for (int rr = 0; rr < r; ++rr)
                                for (int ss = 0; ss < s; ++ss) {
                                    const int ay = ay0 + rr, ax = ax0 + ss;
                                    if (ay >= 0 && ay < h && ax >= 0 && ax < w)
                                        c += xor_popc(in + (((size_t)ay * w + ax) * batch + b) * cw,
                                                      filt + ((size_t)o * taps + rr * s + ss) * cw, cw);
                                    else
                                        ++exclude;
                                }
                            int res = cin * r * s - exclude * cin - 2 * c;
                            if (inject_residual && o < residual_channels && !past) {
                                int v = 0;
                                if (o < res_in_ch) {
                                    if (residual_pool) {
                                        v = INT_MIN;
                                        for (int i = 0; i < 2; ++i)
                                            for (int j = 0; j < 2; ++j)
                                                v = std::max(
                                                    v, res_in[(((size_t)(2 * y + i) * (2 * pw) + (2 * x + j)) * batch + b) * res_in_ch + o]);
                                    } else {
                                        v = res_in[(((size_t)y * pw + x) * batch + b) * res_in_ch + o];
                                    }
                                }
                                res += v;
                            }
                            const uint32_t bit = ((float)res < bn[o]) ? 0u : 1u;
                            uint32_t* word =
                                ahead_fc ? out + (size_t)b * oh * ow * ocw128 + ((size_t)oy * ow + ox) * ocw128 + (o >> 5)
                                         : out + (((size_t)oy * ow + ox) * batch + b) * ocw + (o >> 5);
                            *word |= bit << (31 - (o & 31));
                            if (res_out && !past) res_out[(((size_t)y * pw + x) * batch + b) * cout + o] = res;
                        }
                }
}

// InConv128LayerFMT, kernel.cuh:578-672.  x: fp32 [B][3][H][W]; filter fp32 HWIO.
//   acc = 0; for r, s in-frame: acc += ((+-f0) + (+-f1)) + (+-f2)           l.609-643
//     sign = filter bit (weight >= 0 -> +f, else -f)    param.h:626-628, kernel.cuh:636-638
//   bit = (float)acc < bn[o] ? 0 : 1; OR-pool                                l.646-661
//   pixels walked: pool_h*output_height x pool_w*output_width (l.587-596), so windows of a rounded-up
//     pooled size include pixels past the convolution's own output: computed from the taps still in
//     the frame (acc stays 0 when none is), bit ORed in; no residual is saved for them
//   residual[y][x][b][o] = (int)acc                                          l.662-669
// The three-term sum and the running sum are separate fp32 roundings in this order.
void orc_inconv128(const float* x, const float* hwio, const float* bn, uint32_t* out,
                   int32_t* res_out, int h, int w, int cout, int batch, int r, int s, int stride_h,
                   int stride_w, int padding, int pool_h, int pool_w) {
    int pad_h, pad_w, ph, pw, oh, ow;
    orc_conv_geometry(h, r, stride_h, padding, pool_h, &pad_h, &ph, &oh);
    orc_conv_geometry(w, s, stride_w, padding, pool_w, &pad_w, &pw, &ow);
    const int ocw = step32(cout);
    memset(out, 0, (size_t)oh * ow * batch * ocw * 4);
    const size_t plane = (size_t)h * w;
    std::vector<unsigned char> pos((size_t)r * s * 3 * cout);
    for (size_t i = 0; i < pos.size(); ++i) pos[i] = hwio[i] >= 0.0f;
#pragma omp parallel for collapse(2)
    for (int oy = 0; oy < oh; ++oy)
        for (int ox = 0; ox < ow; ++ox) {
            std::vector<float> acc(cout);
            for (int py = 0; py < pool_h; ++py)
                for (int px = 0; px < pool_w; ++px) {
                    const int y = oy * pool_h + py, xx = ox * pool_w + px;
                    const bool past = y >= ph || xx >= pw;
                    const int ay0 = y * stride_h - pad_h, ax0 = xx * stride_w - pad_w;
                    for (int b = 0; b < batch; ++b) {
                        const float* img = x + (size_t)b * 3 * plane;
                        std::fill(acc.begin(), acc.end(), 0.0f);
                        for (int rr = 0; rr < r; ++rr) {
                            const int ay = ay0 + rr;
                            if (ay < 0 || ay >= h) continue;
                            for (int ss = 0; ss < s; ++ss) {
                                const int ax = ax0 + ss;
                                if (ax < 0 || ax >= w) continue;
                                const float f0 = img[(size_t)ay * w + ax];
                                const float f1 = img[plane + (size_t)ay * w + ax];
                                const float f2 = img[2 * plane + (size_t)ay * w + ax];
                                const unsigned char* pp = &pos[(size_t)(rr * s + ss) * 3 * cout];
                                for (int o = 0; o < cout; ++o) {
                                    const float t0 = pp[o] ? f0 : -f0;
                                    const float t1 = pp[cout + o] ? f1 : -f1;
                                    const float t2 = pp[2 * cout + o] ? f2 : -f2;
                                    const float t01 = t0 + t1;
                                    const float t012 = t01 + t2;
                                    acc[o] = acc[o] + t012;
                                }
                            }
                        }
                        for (int o = 0; o < cout; ++o) {
                            const uint32_t bit = (acc[o] < bn[o]) ? 0u : 1u;
                            out[(((size_t)oy * ow + ox) * batch + b) * ocw + (o >> 5)] |= bit << (31 - (o & 31));
                            if (res_out && !past)
                                res_out[(((size_t)y * pw + xx) * batch + b) * cout + o] = f2i_rz_sat(acc[o]);
                        }
                    }
                }
        }
}

// ------------------------------------------------------------------------
// Reference tile-contiguous ("FMT") layouts.
// ------------------------------------------------------------------------
// FC activations / FC-ready conv output: word (b, kw) lives at
//   ((b/8)*ceil(K/128) + kw/4)*32 + (b%8)*4 + kw%4
// (In128LayerFMT store, kernel.cuh:170 with warpid = row*4 + word; Fc128LayerFMT byte
//  store l.222-223; UnPackFcOutput128FMT, param.h:100).  fmt: PAD8(B)*ceil(K/128)*4 words.
void orc_fc_to_fmt(const uint32_t* logical, uint32_t* fmt, int batch, int k) {
    const int k128 = step128(k), kw = kw128(k);
    memset(fmt, 0, (size_t)pad8(batch) * k128 * 4 * 4);
    for (int b = 0; b < batch; ++b)
        for (int w = 0; w < kw; ++w)
            fmt[((size_t)(b / 8) * k128 + w / 4) * 32 + (b % 8) * 4 + w % 4] = logical[(size_t)b * kw + w];
}
// Conv activations: word (y, x, b, k) lives at
//   (y*W + x)*PAD8(B)*ceil(C/128)*4 + ((b/8)*ceil(C/128) + k/4)*32 + (b%8)*4 + k%4
// (kernel.cuh:650-660, 811-815; UnpackConvOutput32FMT, param.h:678-679).
void orc_conv_to_fmt(const uint32_t* logical, uint32_t* fmt, int h, int w, int batch, int c) {
    const int c128 = step128(c), cw = step32(c);
    const size_t per_pix = (size_t)pad8(batch) * c128 * 4;
    memset(fmt, 0, (size_t)h * w * per_pix * 4);
    for (size_t pix = 0; pix < (size_t)h * w; ++pix)
        for (int b = 0; b < batch; ++b)
            for (int k = 0; k < cw; ++k)
                fmt[pix * per_pix + ((size_t)(b / 8) * c128 + k / 4) * 32 + (b % 8) * 4 + k % 4] =
                    logical[(pix * batch + b) * cw + k];
}
// FC weights: row n, word kw at ((n/8)*ceil(K/128) + kw/4)*32 + (n%8)*4 + kw%4
// (PackFcWeight128FMT, param.h:61 with warpid = (n%8)*4 + word); PAD128(N) rows (param.h:246).
void orc_fc_weight_to_fmt(const uint32_t* logical, uint32_t* fmt, int k, int n) {
    const int k128 = step128(k), kw = kw128(k);
    memset(fmt, 0, (size_t)pad128(n) * k128 * 4 * 4);
    for (int j = 0; j < n; ++j)
        for (int w = 0; w < kw; ++w)
            fmt[((size_t)(j / 8) * k128 + w / 4) * 32 + (j % 8) * 4 + w % 4] = logical[(size_t)j * kw + w];
}
// Conv filters: (tap, o, c-word) at tap*PAD32(O)*ins + ((o/8)*(ins/4) + c/4)*32 + (o%8)*4 + c%4,
// ins = 4*ceil(C/128) (PackFiltersByInChannels128FMT, param.h:568-579).
void orc_conv_filter_to_fmt(const uint32_t* logical, uint32_t* fmt, int r, int s, int c, int o) {
    const int ins = 4 * step128(c), cw = step32(c), taps = r * s;
    const int opad = ((o + 31) >> 5) << 5;
    memset(fmt, 0, (size_t)taps * opad * ins * 4);
    for (int t = 0; t < taps; ++t)
        for (int oc = 0; oc < o; ++oc)
            for (int k = 0; k < cw; ++k)
                fmt[(size_t)t * opad * ins + ((size_t)(oc / 8) * (ins / 4) + k / 4) * 32 + (oc % 8) * 4 + k % 4] =
                    logical[((size_t)oc * taps + t) * cw + k];
}
// Residual tensors: [P][Q][PAD8(B)][PAD128(O)], zero filled (kernel.cuh:666-668, 820-823;
// param.h:925-927, 979-980).
void orc_residual_to_reference(const int32_t* res, int32_t* ref, int h, int w, int batch, int c) {
    const int b8 = pad8(batch), c128 = pad128(c);
    memset(ref, 0, (size_t)h * w * b8 * c128 * 4);
    for (size_t pix = 0; pix < (size_t)h * w; ++pix)
        for (int b = 0; b < batch; ++b)
            for (int o = 0; o < c; ++o)
                ref[(pix * b8 + b) * c128 + o] = res[(pix * batch + b) * c + o];
}


// ---- layers of the textbook ResNet wiring: NO counterpart in the reference (its ResNet has no
// pooling layer, no convolutional shortcut and no average-pooling head, imagenet_resnet.cu:223-325).
// Defined here as plain loops; pinned in the tests against torch.nn.functional.max_pool2d on the
// unpacked +-1 values / the integer residual, and against fp64 mean + matmul.
// Overlapping pooling: bit = OR over the window's in-frame taps, residual = their maximum.
void orc_pool128(const uint32_t* in, uint32_t* out, const int32_t* res_in, int32_t* res_out, int h, int w,
                 int c, int batch, int window, int stride, int padding) {
    const int oh = (h + 2 * padding - window) / stride + 1, ow = (w + 2 * padding - window) / stride + 1;
    const int cw = step32(c);
#pragma omp parallel for collapse(2)
    for (int oy = 0; oy < oh; ++oy)
        for (int ox = 0; ox < ow; ++ox)
            for (int b = 0; b < batch; ++b) {
                for (int k = 0; k < cw; ++k) {
                    uint32_t acc = 0;
                    for (int r = 0; r < window; ++r)
                        for (int s = 0; s < window; ++s) {
                            const int y = oy * stride - padding + r, x = ox * stride - padding + s;
                            if (y >= 0 && y < h && x >= 0 && x < w) acc |= in[(((size_t)y * w + x) * batch + b) * cw + k];
                        }
                    out[(((size_t)oy * ow + ox) * batch + b) * cw + k] = acc;
                }
                if (res_in == nullptr) continue;
                for (int o = 0; o < c; ++o) {
                    int m = INT_MIN;
                    for (int r = 0; r < window; ++r)
                        for (int s = 0; s < window; ++s) {
                            const int y = oy * stride - padding + r, x = ox * stride - padding + s;
                            if (y >= 0 && y < h && x >= 0 && x < w)
                                m = std::max(m, res_in[(((size_t)y * w + x) * batch + b) * c + o]);
                        }
                    res_out[(((size_t)oy * ow + ox) * batch + b) * c + o] = m;
                }
            }
}
// Global average pool of an integer residual tensor + fp32 fully connected layer: the pixel sum is an
// exact integer, mean = (float)sum / (float)pixels, out = bias + fma chain over the channels in
// ascending order.
void orc_avgpool_fc(const int32_t* res, const float* weight, const float* bias, float* out, int h, int w, int c,
                    int batch, int n) {
    const int pixels = h * w;
#pragma omp parallel for
    for (int b = 0; b < batch; ++b) {
        std::vector<float> mean(c);
        for (int o = 0; o < c; ++o) {
            long long sum = 0;
            for (int p = 0; p < pixels; ++p) sum += res[((size_t)p * batch + b) * c + o];
            mean[o] = (float)(int)sum / (float)pixels;
        }
        for (int j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (int o = 0; o < c; ++o) acc = fmaf(mean[o], weight[(size_t)o * n + j], acc);
            out[(size_t)b * n + j] = acc + bias[j];
        }
    }
}

}  // extern "C"
