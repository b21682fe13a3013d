/*
 * tcbnn_hip.h — C ABI of the MI355X (gfx950) binarized-network inference path.
 *
 * Every entry point replaces one piece of the CUDA reference's bit-matmul /
 * bit-convolution inference path (pnnl/TCBNN).  The citation on each
 * declaration names the reference function or method whose behaviour the
 * entry point reproduces.  The reference fuses its layers into one persistent
 * cooperative kernel (imagenet_resnet.cu:34-125); here every layer is one
 * stream-ordered launch, so a network is a host loop over *_forward calls on
 * one stream.
 *
 * Conventions
 *   - All data pointers are DEVICE pointers unless the name ends in _host.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *   - Return value: 0 on success, a negative TCBNN_E* code otherwise.  No
 *     entry point ever calls exit(); tcbnn_last_error() returns a message for
 *     the calling thread.  (The reference prints and exits, utility.h:57-92;
 *     the C++ layer classes layered above this ABI keep that behaviour.)
 *   - Bit convention (kernel.cuh:168, param.h:60): bit = 1 <=> value >= 0
 *     (resp. >= threshold) <=> "+1"; element e of a group of 32 is bit (31-e)
 *     of its uint32 ("MSB first"); pad bits are 0 in both operands and the
 *     true K / Cin enters  K - 2*popc(a xor w).
 *
 * Engine layouts (device memory).  The batch index is innermost everywhere, so a
 * wavefront whose lanes are 64 consecutive images reads and writes contiguous runs:
 *   FC activations   : uint32 [KW128][B]          KW128 = 4*ceil(K/128) words per image
 *   conv activations : uint32 [H][W][CW][B]       CW    = ceil(C/32) words per (pixel,image)
 *   FC-ready conv out: uint32 [OH*OW*CW128][B]    feature order (y, x, c), c padded to 128
 *                                                 (kernel.cuh:798-808): an FC activation
 *   packed weights   : uint32 [NPAD32][KWTOT]     one row per output neuron/channel,
 *                                                 FC: KWTOT = KW128; conv: KWTOT = R*S*CW,
 *                                                 K index = (r*S+s)*32*CW + c; rows >= N are 0;
 *                                                 FC weights and 3x3 filters are followed by the
 *                                                 same words in the order the matrix-core kernels'
 *                                                 lanes load them (tcbnn_fc_weight_words,
 *                                                 tcbnn_conv_filter_words give the total)
 *   residual tensors : TCBNN_RES_I32: int32 [P][Q][ceil(O/4)][B][4]; TCBNN_RES_I16: int16
 *                      [P][Q][ceil(O/8)][B][8] for tensors whose values provably fit 16 bits;
 *                      TCBNN_RES_I12: per pixel and group of 16 channels uint32 [B][4] then
 *                      uint32 [B][2] (12 bits per value, 24 bytes per image) for tensors whose
 *                      values provably fit 12 bits (see "residual formats" below).  In every
 *                      format an image's group of 4 / 8 / 16 consecutive channels is one or two
 *                      contiguous pieces of 16 (or 16 + 8) bytes and consecutive images follow
 *                      each other; channels are padded to the group, not to 128
 *   fp32 stem input  : float  [B][3][H][W]        (kernel.cuh:620-625)
 * The reference's own tile-contiguous "FMT" layouts ([.../8][.../128][8][4],
 * kernel.cuh:170,222,650-660,798-815) are produced / consumed by the
 * *_to_reference_fmt / *_from_reference_fmt converters below.
 */
#ifndef TCBNN_HIP_H
#define TCBNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TCBNN_OK 0
#define TCBNN_EINVAL (-1)   /* bad shape / flag combination                  */
#define TCBNN_ENULL (-2)    /* required pointer is NULL (utility.h:84-92)    */
#define TCBNN_EHIP (-3)     /* HIP runtime error (utility.h:57-81)           */
#define TCBNN_EUNSUPPORTED (-4)

/* Inner-product engines.  AUTO is the process-wide default (FP4 matrix cores unless
 * changed by tcbnn_set_default_variant or the environment). */
#define TCBNN_VARIANT_AUTO 0
#define TCBNN_VARIANT_POPC 1      /* v_xor_b32 + v_bcnt_u32_b32 on the VALU   */
#define TCBNN_VARIANT_MFMA_I8 2   /* +-1 unpacked to int8, v_mfma_i32_32x32x32_i8 */
#define TCBNN_VARIANT_MFMA_F4 3   /* +-1 unpacked to FP4 E2M1, v_mfma_f32_32x32x64_f8f6f4 (exact: |sum| < 2^24) */

/* Residual storage formats.  The reference keeps residuals (pre-threshold sums, kernel.cuh:
 * 662-669, 818-824) as int32.  They are this path's dominant HBM traffic, and their magnitude
 * is bounded by construction: |first-layer sum| <= R*S*3*max|input|, and every bit
 * convolution adds at most Cin*R*S.  A tensor whose bound is <= 32767 may be stored as
 * int16 without changing a single value; the caller states the format per tensor and is
 * responsible for the bound (tcbnn_*_residual_bound compute it, the layer classes above
 * this ABI track it from the actual input data).  Producer and consumer must agree. */
#define TCBNN_RES_I32 0
#define TCBNN_RES_I16 1
/* 12 bits per value, for tensors whose bound is <= 2047 (the first layer's and the first stage's of a ResNet on
 * normalised images: they are the largest tensors of the path).  Groups of 16 channels: the 192-bit string that
 * holds value e (two's complement) at bits 12e..12e+11 is stored as words w0..w5, laid out per pixel and group as
 * uint32 [B][4] (w0..w3 of every image) followed by uint32 [B][2] (w4, w5): 24 bytes per image, pixel and group. */
#define TCBNN_RES_I12 2

/* ------------------------------------------------------------------ misc */
int tcbnn_abi_version(void);
/* Message of the last failing call on this thread ("" if none). */
const char* tcbnn_last_error(void);
/* Process-wide default for TCBNN_VARIANT_AUTO (also read once from the
 * environment variable TCBNN_VARIANT = popc | mfma_i8 | mfma_f4). */
int tcbnn_set_default_variant(int variant);
int tcbnn_get_default_variant(void);

/* ------------------------------------------------------------ geometry */
/* Derived conv geometry, identical in both reference conv constructors
 * (param.h:719-728, 897-906):
 *   pad = padding ? ((((H + s - H%s)/s - 1)*s + R - H)/2) : 0
 *   buf = padding ? ceil(H/s) : (H-R)/s + 1 ;  out = ceil(buf/pool)          */
int tcbnn_conv_pad(int in_size, int filter, int stride, int padding);
int tcbnn_conv_out(int in_size, int filter, int stride, int padding, int pool);

/* Word counts of the engine layouts above. */
size_t tcbnn_fc_act_words(int batch, int features);                    /* B*KW128          */
size_t tcbnn_conv_act_words(int height, int width, int batch, int ch); /* H*W*B*CW         */
size_t tcbnn_fc_weight_words(int in_features, int out_features);       /* NPAD32*KW128 rows + the lane-order copy, NPAD32*8*ceil(KW128/8) */
size_t tcbnn_conv_filter_words(int r, int s, int in_ch, int out_ch);   /* NPAD32*R*S*CW, x2 for 3x3 filters with
                                                                           Cin = 64/128/192/256/384/512: they carry a
                                                                           copy in MFMA lane order after the bit rows */
size_t tcbnn_inconv_filter_words(int r, int s, int in_ch, int out_ch); /* R*S*OPAD32*5     */
/* bytes of a residual tensor of `channels` channels in the given TCBNN_RES_* format */
size_t tcbnn_residual_bytes(int height, int width, int channels, int batch, int format);
/* Upper bound of |residual| of a first layer whose input satisfies |x| <= input_abs_max
 * (R*S*3 terms plus rounding slack), and of a bit convolution that adds its own
 * Cin*R*S to an injected residual bounded by injected_bound (0 if none).  INT32_MAX
 * when unknown (non-finite input_abs_max, overflow).  tcbnn_residual_format_for_bound:
 * TCBNN_RES_I16 when 0 <= bound <= 32767, else TCBNN_RES_I32.  tcbnn_residual_format_narrowest also
 * considers TCBNN_RES_I12: 0 <= bound <= 2047 and an even batch (its 128-bit pieces are then aligned).
 * tcbnn_inconv_residual_bound_of_input is the first layer's bound from the actual batch (HOST pointer,
 * float [batch][3][height][width]): the largest sum of |x| over any filter window, plus rounding slack;
 * far tighter than R*S*3*max|x| on real images, which is what lets the first stage use 12 bits. */
int tcbnn_inconv_residual_bound(int filter_height, int filter_width, float input_abs_max);
int tcbnn_inconv_residual_bound_of_input(const float* input_host, int batch, int height, int width,
                                         int filter_height, int filter_width, int stride_height,
                                         int stride_width, int padding);
/* max |x| over a HOST array (on a few host threads; +infinity if any value is NaN or infinite): the cheap first test of
 * a new first-layer batch against the recorded bound, before the window scan above. */
float tcbnn_host_abs_max(const float* values_host, size_t count);
int tcbnn_conv_residual_bound(int input_channels, int filter_height, int filter_width, int injected_bound);
int tcbnn_residual_format_for_bound(int bound);
int tcbnn_residual_format_narrowest(int bound, int batch);

/* ------------------------------------------------- one-time weight packing */
/* fp32 [K][N] (param.h:58-59) -> packed [NPAD32][KW128], followed by the same words in the FP4 FC kernel's lane
 * order, uint32 [NPAD32/32][ceil(KW128/8)][64][4].  `packed` holds tcbnn_fc_weight_words(...) words; the FC and
 * output layers take only buffers written by this function.  Replaces PackFcWeight128FMT (param.h:44-63). */
int tcbnn_pack_fc_weight(const float* weight_kn, uint32_t* packed, int in_features,
                         int out_features, void* stream);
/* fp32 HWIO [R][S][C][O] (param.h:573-574) -> packed [OPAD32][R*S][CW] (+ the FP4 fragment copy
 * for the 3x3 shapes named at tcbnn_conv_filter_words).  `packed` holds
 * tcbnn_conv_filter_words(...) words.  Replaces PackFiltersByInChannels128FMT (param.h:560-581). */
int tcbnn_pack_conv_filter(const float* filter_hwio, uint32_t* packed, int r, int s, int in_ch,
                           int out_ch, void* stream);
/* fp32 HWIO [R][S][3][O] -> sign table uint32 [R*S][OPAD32][4]: entry c<3 is 0 if the
 * weight of input channel c is >= 0 and 0x80000000 otherwise (the bit the first layer
 * flips on the fp32 input, kernel.cuh:636-638); entry 3 is the sign pattern index
 * 4*neg0 + 2*neg1 + neg2.  A second table [R*S][OPAD32] follows with the patterns alone,
 * one per word.  Replaces PackFiltersByOutChannels32 (param.h:613-632). */
int tcbnn_pack_inconv_filter(const float* filter_hwio, uint32_t* packed, int r, int s, int in_ch,
                             int out_ch, void* stream);
/* fp32 +-1 matrix rows -> packed activation matrix, MSB first, batch (row) innermost:
 * out[k/32][row].  `rows` x `k` row-major input with leading dimension `ld`; k_words
 * words are written per row (zero padded).  Replaces BMMA_toBit32Row
 * (tensorcore_kernel.cu:87-97). */
int tcbnn_pack_rows(const float* src, uint32_t* packed, int rows, int k, int ld, int k_words,
                    void* stream);
/* fp32 [K][N] -> packed [N][k_words] (each column contiguous along K).  Replaces
 * BMMA_toBit32Col (tensorcore_kernel.cu:74-84). */
int tcbnn_pack_cols(const float* src, uint32_t* packed, int k, int n, int k_words, void* stream);
/* fp32 +-1 NHWC [B][H][W][C] -> packed [H][W][CW][B].  Replaces BTC_bin_input
 * (bmma_kernel.cu:73-98). */
int tcbnn_pack_conv_input_nhwc(const float* src, uint32_t* packed, int batch, int height,
                               int width, int ch, void* stream);

/* ------------------------------------------------------------ layer forward */
/* In128LayerFMT (kernel.cuh:153-172), descriptor fields of In128LayerParam
 * (param.h:210-218): fp32 [B][K] -> sign bits, FC activation layout. */
typedef struct tcbnn_in128_desc {
    const float* input;   /* [input_height][input_width] */
    uint32_t* output;     /* [KW128][B] */
    int input_height;     /* batch */
    int input_width;      /* features */
} tcbnn_in128_desc;
int tcbnn_in128_forward(const tcbnn_in128_desc* d, void* stream);

/* Fc128LayerFMT (kernel.cuh:174-226), fields of Fc128LayerParam (param.h:362-384):
 * bit[b][n] = ((float)K - 2*(float)popc(a_b xor w_n) >= bn[n]). */
typedef struct tcbnn_fc128_desc {
    const uint32_t* input;   /* [KW128(input_width)][B] */
    const uint32_t* weight;  /* tcbnn_pack_fc_weight output */
    const float* bn;         /* [weight_width] thresholds */
    uint32_t* output;        /* [KW128(weight_width)][B] */
    int input_height;        /* batch */
    int input_width;         /* K */
    int weight_width;        /* N */
    int variant;             /* TCBNN_VARIANT_* */
    int32_t* workspace;      /* optional int32 [NPAD32][B] scratch: lets small-batch layers
                                split K over workgroups; NULL = never split */
    size_t workspace_words;
} tcbnn_fc128_desc;
int tcbnn_fc128_forward(const tcbnn_fc128_desc* d, void* stream);
/* The same layer for callers that can neither allocate device memory nor hand over a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  NO counterpart in the
 * reference.  The split-K partial sums go to a buffer built into the library's code object (4 MiB of device
 * memory per GPU, held until the process ends); d->workspace and d->workspace_words are ignored.  The call
 * allocates and frees nothing, clears what it accumulates into with a fill kernel (no memset node), and gives
 * the same bits as tcbnn_fc128_forward.  Limits: PAD32(weight_width) * input_height <= 1048576 words, else
 * TCBNN_EINVAL; all calls on one GPU share the one buffer, so calls that overlap in time on one GPU (different
 * streams or threads) race - serialise them.  The buffer's device address is looked up on the first call per
 * device (hipGetSymbolAddress, which allocates nothing): make that first call outside a stream capture. */
int tcbnn_fc128_forward_static_scratch(const tcbnn_fc128_desc* d, void* stream);

/* Out128LayerFMT (kernel.cuh:230-280), fields of Out128LayerParam (param.h:506-530):
 * y[b][n] = ((float)K - (float)popc*2.0f)*bn_scale[n] + bn_bias[n], fp32 row major. */
typedef struct tcbnn_out128_desc {
    const uint32_t* input;
    const uint32_t* weight;
    const float* bn_scale;
    const float* bn_bias;
    float* output;           /* [B][weight_width] */
    int input_height, input_width, weight_width;
    int variant;
} tcbnn_out128_desc;
int tcbnn_out128_forward(const tcbnn_out128_desc* d, void* stream);

/* InConv128LayerFMT (kernel.cuh:578-672), fields of InConv128LayerParam
 * (param.h:841-869).  fp32 NCHW 3-channel input, +-1 filters, fp32 adds in the
 * reference order  acc += ((+-f0) + (+-f1)) + (+-f2)  per in-frame tap in (r,s)
 * raster order; bit = !((float)acc < bn[o]); OR-pool; residual = (int)acc.
 * save_residual requires pool 1x1 (the reference index by*output_width+bx,
 * kernel.cuh:666, is only meaningful then). */
#define TCBNN_INCONV_INPUT_NCHW 0   /* float [batch][3][H][W], the reference's device layout (kernel.cuh:620-625) */
#define TCBNN_INCONV_INPUT_PACKED 1 /* float [Hp][Wp][batch][3], zero-padded: see tcbnn_inconv_pack_input */
typedef struct tcbnn_inconv128_desc {
    const float* input;        /* device, in the layout `input_layout` names */
    const uint32_t* filter;    /* tcbnn_pack_inconv_filter output */
    const float* bn;           /* [output_channels] */
    uint32_t* output;          /* [OH][OW][CW(output_channels)][B] */
    int32_t* output_residual;  /* residual tensor in `residual_format`, or NULL */
    int input_height, input_width, input_channels;
    int filter_height, filter_width;
    int output_channels, batch;
    int stride_height, stride_width;
    int padding;               /* bool */
    int pool_height, pool_width;
    int save_residual;         /* bool */
    int residual_format;       /* TCBNN_RES_* of output_residual */
    int input_layout;          /* TCBNN_INCONV_INPUT_*; PACKED needs pool 1x1 */
} tcbnn_inconv128_desc;
int tcbnn_inconv128_forward(const tcbnn_inconv128_desc* d, void* stream);
/* The engine's own layout of the first layer's input: batch innermost like every other tensor, and zero-padded, so
 * that a lane (= image) reads the three channels of an input pixel as 12 contiguous bytes, a wavefront 768, and no
 * tap needs a test for the frame: float [Hp][Wp][batch][3] with Hp = (P - 1) * stride_height + filter_height,
 * Wp = (Q - 1) * stride_width + filter_width (P x Q = tcbnn_conv_out of the two dimensions, pool 1) and the frame's
 * pixel (0, 0) at (tcbnn_conv_pad(height...), tcbnn_conv_pad(width...)).  The reference reads [batch][3][H][W]
 * directly (kernel.cuh:620-625) and has no such step; here it belongs to the upload of an input
 * (InConv128LayerParam::initialize / set_input), not to the forward pass.  Both pointers are device pointers. */
size_t tcbnn_inconv_packed_input_floats(int batch, int height, int width, int filter_height, int filter_width,
                                        int stride_height, int stride_width, int padding);
int tcbnn_inconv_pack_input(const float* input, float* packed, int batch, int height, int width, int filter_height,
                            int filter_width, int stride_height, int stride_width, int padding, void* stream);

/* Conv128LayerFMT (kernel.cuh:676-827), fields of Conv128LayerParam (param.h:1028-1064).
 *   res = Cin*R*S - exclude*Cin - 2*popc                      (kernel.cuh:766-768)
 *   if inject_residual && o < residual_channels:
 *        res += residual_pool ? max_{i,j in {0,1}} Rin[2y+i][2x+j][b][o] : Rin[y][x][b][o]
 *                                                              (kernel.cuh:770-794)
 *   bit = !((float)res < bn[o]); OR over the pool window      (kernel.cuh:795-816)
 *   if save_residual: Rout[y][x][b][o] = res                  (kernel.cuh:818-824)
 * Channels o >= input_residual_channels of the source read as 0 (the reference
 * gets the same effect from its zero-filled 128-channel padding, param.h:979-980).
 * save_residual / inject_residual require pool 1x1, residual_pool requires the
 * source to be exactly twice the output size (as the reference indexing assumes).
 * output_residual_pool = 2 (no counterpart in the reference): Rout holds, per 2x2 window of output
 * pixels, the element-wise maximum of `res`: a P/2 x Q/2 x O tensor, i.e. exactly what a consumer
 * with residual_pool computes from the full tensor before it adds it (kernel.cuh:775-782), so that
 * consumer then injects it with residual_pool = 0.  A quarter of the bytes are written and read;
 * meant for a tensor whose every consumer pools.  Available where
 * tcbnn_conv128_pooled_save_supported says so (TCBNN_EUNSUPPORTED otherwise). */
typedef struct tcbnn_conv128_desc {
    const uint32_t* input;         /* [H][W][CW(input_channels)][B] */
    const uint32_t* filter;        /* tcbnn_pack_conv_filter output */
    const float* bn;               /* [output_channels] */
    uint32_t* output;              /* [OH][OW][CW(O)][B]; ahead_fc: [OH][OW][CW128(O)][B] */
    const int32_t* input_residual; /* source tensor (Hr x Wr x input_residual_channels) or NULL */
    int32_t* output_residual;      /* P x Q x O tensor or NULL */
    int input_height, input_width, input_channels;
    int filter_height, filter_width;
    int output_channels, batch;
    int stride_height, stride_width;
    int padding;
    int pool_height, pool_width;
    int ahead_fc, save_residual, inject_residual;
    int residual_channels;         /* inject only into o < residual_channels */
    int residual_pool;
    int input_residual_channels;   /* channel count of the source tensor */
    int variant;
    int input_residual_format;     /* TCBNN_RES_* of input_residual */
    int output_residual_format;    /* TCBNN_RES_* of output_residual */
    int output_residual_pool;      /* 0: P x Q x O tensor; 2: its 2x2 maximum, P/2 x Q/2 x O */
} tcbnn_conv128_desc;
int tcbnn_conv128_forward(const tcbnn_conv128_desc* d, void* stream);
/* 1 if the layer `d` describes can be run with output_residual_pool = 2 (whatever d->output_residual_pool says; no
 * pointer is dereferenced): the FP4 engine's 3x3 kernel on an un-pooled layer with even P and Q, output channels a
 * multiple of 64, a 12- or 16-bit injected residual whose channel limit is a multiple of 32, and a 12- or 16-bit
 * output format.  0 otherwise.  No counterpart in the reference. */
int tcbnn_conv128_pooled_save_supported(const tcbnn_conv128_desc* d);

/* Name of the device kernel (as a profiler lists it, template arguments included) that
 * the corresponding *_forward call would launch for this descriptor; no
 * launch happens and no pointer is dereferenced.  No counterpart in the reference
 * (its layers are inlined device functions of one network kernel); used to match
 * per-launch timings with profiler output. */
int tcbnn_conv128_kernel_name(const tcbnn_conv128_desc* d, char* buf, size_t len);
int tcbnn_fc128_kernel_name(const tcbnn_fc128_desc* d, char* buf, size_t len);
int tcbnn_out128_kernel_name(const tcbnn_out128_desc* d, char* buf, size_t len);
int tcbnn_inconv128_kernel_name(const tcbnn_inconv128_desc* d, char* buf, size_t len);

/* Measurement aid (no counterpart in the reference): one wavefront counts shader clock cycles over `microseconds` of
 * the device's constant-rate wall clock, on `stream`, while whatever else is queued on other streams runs beside it.
 * After the stream has been synchronised, counts[0] = shader cycles, counts[1] = wall-clock ticks (DEVICE pointer to
 * two 64-bit words); *wall_clock_khz = ticks per millisecond.  Shader MHz = counts[0] / counts[1] * khz / 1000. */
int tcbnn_shader_clock_probe(unsigned long long* counts, int microseconds, int* wall_clock_khz, void* stream);

/* ------------------------------------------------ layers of the textbook ResNet wiring */
/* The reference wires ResNet-18 without a pooling layer after the first convolution, without
 * convolutional shortcuts and without an average-pooling head (imagenet_resnet.cu:223-325).  The two
 * layers below have NO counterpart in the reference; together with a Conv128 layer of filter 1x1,
 * stride 2 and save_residual (the downsample shortcut) they let the same engine run the textbook wiring
 * (7x7/2 first layer + 3x3/2 max-pool, 1x1/2 shortcut convolutions, global average pool + fp32 FC).
 *
 * Overlapping pooling on a packed activation tensor and, optionally, its residual: every output bit is
 * the OR of the bits of its window (the maximum of the +-1 values), every output residual value the
 * maximum of the window's values; taps outside the frame are ignored.  Output size per dimension:
 * (in + 2*padding - window) / stride + 1.  The output residual has the input's format. */
typedef struct tcbnn_pool128_desc {
    const uint32_t* input;          /* device, conv activation layout [H][W][CW][B]                 */
    uint32_t* output;               /* device, [OH][OW][CW][B]                                      */
    const int32_t* input_residual;  /* device, residual layout with `channels` channels, or NULL    */
    int32_t* output_residual;       /* device, residual layout [OH][OW]..., or NULL                 */
    int input_height, input_width, channels, batch;
    int window, stride, padding;    /* square window; padding < window                              */
    int residual_format;            /* TCBNN_RES_* of both residual tensors                         */
} tcbnn_pool128_desc;
int tcbnn_pool_out(int in_size, int window, int stride, int padding);
int tcbnn_pool128_forward(const tcbnn_pool128_desc* d, void* stream);

/* Global average pool over the pixels of a residual tensor, then an fp32 fully connected layer:
 * mean[b][c] = (float)(sum over pixels of residual[p][c][b]) / (float)(height*width) (the sum is an exact
 * integer), out[b][n] = bias[n] + sum over c, in ascending order with fused multiply-add, of
 * mean[b][c] * weight[c][n].  channels <= 512. */
typedef struct tcbnn_avgpool_fc_desc {
    const int32_t* input_residual;  /* device, residual layout [H][W]... with `channels` channels   */
    const float* weight;            /* device, fp32 [channels][out_features] row major              */
    const float* bias;              /* device, fp32 [out_features]                                  */
    float* output;                  /* device, fp32 [batch][out_features] row major                 */
    int input_height, input_width, channels, batch, out_features;
    int residual_format;            /* TCBNN_RES_* of input_residual                                */
} tcbnn_avgpool_fc_desc;
int tcbnn_avgpool_fc_forward(const tcbnn_avgpool_fc_desc* d, void* stream);

/* ------------------------------------------------ standalone GEMM / conv */
/* C[m][n] = K - 2*popc(A[m,:] xor B[n,:]), int32 row major [M][N].  A: [K/32][M]
 * (tcbnn_pack_rows output), B: [N][K/32] (tcbnn_pack_cols output: each column of the
 * logical K x N matrix contiguous along K); K % 32 == 0, N % 32 == 0.  Replaces
 * BMMAS / BMMAS_new (tensorcore_kernel.cu:305-356). */
int tcbnn_bmm(const uint32_t* a, const uint32_t* b, int32_t* c, int m, int n, int k, int variant,
              void* stream);
/* out[b][p][q][o] = Cin*R*S - exclude*Cin - 2*popc  (bmma_kernel.cu:154-159), int32
 * [N][P][Q][O] (the layout BTC_trans_output produces, bmma_kernel.cu:247-263).
 * input: [H][W][CW][B]; filter: tcbnn_pack_conv_filter output.  Replaces
 * BTC_Conv2d_balance[_128] (bmma_kernel.cu:101-165, 326-392). */
int tcbnn_bconv(const uint32_t* input, const uint32_t* filter, int32_t* output, int batch,
                int height, int width, int in_ch, int out_ch, int r, int s, int stride_h,
                int stride_w, int pad_h, int pad_w, int out_h, int out_w, int variant,
                void* stream);

/* -------------------------------------------------- unpack / interop */
/* bits -> +-1.0f, [B][N] row major.  Replaces UnPackFcOutput128FMT (param.h:87-104). */
int tcbnn_unpack_fc_output(const uint32_t* packed, float* out, int batch, int features,
                           void* stream);
/* bits -> +-1.0f, NHWC [B][H][W][C].  Replaces UnpackConvOutput32FMT (param.h:661-688). */
int tcbnn_unpack_conv_output(const uint32_t* packed, float* out, int height, int width, int ch,
                             int batch, void* stream);
/* Engine FC activation layout <-> reference [ceil(B/8)][ceil(K/128)][8][4] tiles
 * (kernel.cuh:170,222-223).  fmt holds PAD8(B)*ceil(K/128)*4 words. */
int tcbnn_fc_to_reference_fmt(const uint32_t* packed, uint32_t* fmt, int batch, int features,
                              void* stream);
int tcbnn_fc_from_reference_fmt(const uint32_t* fmt, uint32_t* packed, int batch, int features,
                                void* stream);
/* Engine conv activation layout <-> reference [H][W][PAD8(B)/8][ceil(C/128)][8][4]
 * (kernel.cuh:650-660, 811-815). */
int tcbnn_conv_to_reference_fmt(const uint32_t* packed, uint32_t* fmt, int height, int width,
                                int batch, int ch, void* stream);
int tcbnn_conv_from_reference_fmt(const uint32_t* fmt, uint32_t* packed, int height, int width,
                                  int batch, int ch, void* stream);
/* Engine residual (either format) -> reference int32 [P][Q][PAD8(B)][PAD128(O)] with
 * zero fill (kernel.cuh:666-668, 820-823). */
int tcbnn_residual_to_reference(const int32_t* res, int32_t* ref, int height, int width,
                                int batch, int ch, int format, void* stream);
/* The reverse: a residual in the reference layout -> the engine layout `format`
 * (tcbnn_residual_bytes(...) bytes), for a Conv128 layer that injects a residual a
 * reference-layout producer saved (read at kernel.cuh:760-791).  TCBNN_RES_I16 keeps the low
 * 16 bits: only for values the caller knows to fit. */
int tcbnn_residual_from_reference(const int32_t* ref, int32_t* res, int height, int width,
                                  int batch, int ch, int format, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TCBNN_HIP_H */
