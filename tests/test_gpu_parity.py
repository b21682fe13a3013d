"""Parity of the HIP path (through the C ABI) with the CPU oracle: bit-exact for popcount
accumulators, packed activations and int32 residuals; fp32 logits to 1e-5 relative (they are in
fact bit-identical: multiply and add are separately rounded on both sides)."""
import numpy as np
import pytest

from oracle import orc
from oracle import nets as orc_nets
from tests import gpuops, refmath as rm

pytestmark = pytest.mark.gpu

VARIANTS = ["popc", "mfma_f4", "mfma_i8"]


def rng(seed):
    return np.random.default_rng(seed)


def _variant(gpu, name):
    return gpu.VARIANTS[name]


# --------------------------------------------------------------------------- standalone GEMM
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (8, 32, 32), (100, 64, 96), (77, 160, 1056),
                                   (300, 32, 4096), (64, 32, 64),
                                   # large products (the FP4 engine's large-GEMM kernel): ragged rows and columns,
                                   # K of 3, 8 and 24 k-steps (groups of 8, weight blocks of 16)
                                   (4100, 992, 192), (4100, 992, 512), (9000, 2048, 1536), (8192, 1024, 1024),
                                   # a last column group of 32 (its rows leave element-wise, the others through LDS)
                                   (4100, 1056, 192)])
def test_bmm(gpu, variant, m, n, k):
    r = rng(m + n + k)
    a = r.integers(0, 2 ** 32, size=(m, k // 32), dtype=np.uint64).astype(np.uint32)
    b = r.integers(0, 2 ** 32, size=(n, k // 32), dtype=np.uint64).astype(np.uint32)
    got = gpuops.bmm(a, b, m, n, k, _variant(gpu, variant))
    np.testing.assert_array_equal(got, orc.bmm(a, b, k))


# --------------------------------------------------------------------------- In / Fc / Out layers
@pytest.mark.parametrize("b,k", [(8, 784), (100, 128), (8192, 784), (3, 1000)])
def test_in128(gpu, b, k):
    x = rng(b + k).standard_normal((b, k)).astype(np.float32)
    x[0, :3] = [0.0, -0.0, 1e-30]
    layer = gpu.In128LayerParam("Fin", b, k).initialize(x)
    layer.forward()
    want = orc.in128(x)
    np.testing.assert_array_equal(layer.download_packed(), want)
    np.testing.assert_array_equal(layer.download_output(), orc.fc_to_fmt(want, b, k))
    np.testing.assert_array_equal(layer.download_full_output(), np.where(x >= 0, 1.0, -1.0))
    layer.release()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,k,n", [(8, 128, 128), (64, 784, 1024), (100, 1024, 1024), (13, 300, 100),
                                   (256, 2048, 160), (130, 25088, 64), (1000, 1024, 32), (1, 512, 64), (3, 96, 40),
                                   # large batches: the large-GEMM kernel with the threshold epilogue
                                   (8192, 1024, 1024), (4100, 512, 1000), (4100, 300, 1000)])
def test_fc128(gpu, variant, b, k, n):
    r = rng(b + k + n)
    x = r.standard_normal((b, k)).astype(np.float32)
    w = rm.pm1(r, (k, n))
    bn = r.normal(0, np.sqrt(k), n).astype(np.float32)
    wl = orc.pack_fc_weight(w)
    _, acc = orc.fc128(orc.in128(x), wl, bn, k, n, want_acc=True)
    bn[: min(n, 8)] = (k - 2 * acc)[0, : min(n, 8)]  # exact ties
    want = orc.fc128(orc.in128(x), wl, bn, k, n)
    inp = gpuops.in128(x)
    wbuf = gpuops.pack_fc_weight(w)
    got = gpuops.fc128(inp, wbuf, bn, b, k, n, _variant(gpu, variant))
    np.testing.assert_array_equal(got, want)
    got = gpuops.fc128(inp, wbuf, bn, b, k, n, _variant(gpu, variant), workspace=False)  # no split-K
    np.testing.assert_array_equal(got, want)
    # packed weights agree with the oracle's packing (rows >= N are zero)
    wg = wbuf.to_numpy(np.uint32, (((n + 31) // 32) * 32, orc.kw128(k)))
    np.testing.assert_array_equal(wg[:n], wl)
    assert not wg[n:].any()


@pytest.mark.parametrize("variant", VARIANTS)
def test_fc128_nan_threshold(gpu, variant):
    r = rng(3)
    x = r.standard_normal((8, 128)).astype(np.float32)
    w = rm.pm1(r, (128, 32))
    bn = np.full(32, np.nan, np.float32)
    out = gpuops.fc128(gpuops.in128(x), gpuops.pack_fc_weight(w), bn, 8, 128, 32, _variant(gpu, variant))
    assert out.shape == (8, 4) and not out.any()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,k,n", [(8, 1024, 10), (256, 512, 1000), (70, 300, 33), (1, 512, 1000), (8192, 1024, 10),
                                   (4100, 1536, 1000), (4100, 1000, 72)])
def test_out128(gpu, variant, b, k, n):
    r = rng(b + k + n)
    x = r.standard_normal((b, k)).astype(np.float32)
    w = rm.pm1(r, (k, n))
    scale = r.normal(1, 0.1, n).astype(np.float32)
    bias = r.normal(0, 1, n).astype(np.float32)
    want = orc.out128(orc.in128(x), orc.pack_fc_weight(w), scale, bias, k, n)
    got = gpuops.out128(gpuops.in128(x), gpuops.pack_fc_weight(w), scale, bias, b, k, n, _variant(gpu, variant))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)  # tolerance stated by the target
    np.testing.assert_array_equal(got, want)  # and in fact bit-identical


# --------------------------------------------------------------------------- standalone conv
SWEEP = [(32, 128), (16, 256), (8, 512), (56, 64), (28, 128), (14, 256), (7, 512)]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("h,c", SWEEP)
def test_bconv_sweep_shapes(gpu, variant, h, c):
    """The 3x3 stride-1 pad-1 sweep shapes at a batch the CPU oracle finishes in seconds."""
    b = 8 if h > 16 else 24
    r = rng(h + c)
    x = rm.pm1(r, (b, h, h, c))
    f = rm.pm1(r, (3, 3, c, c))
    pad, buf, _ = orc.conv_geometry(h, 3, 1)
    want = orc.bconv(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), c, c, 3, 3, 1, pad, buf, buf)
    inp, filt = gpuops.pack_conv_input(x), gpuops.pack_conv_filter(f)
    np.testing.assert_array_equal(inp.to_numpy(np.uint32, (h, h, c // 32, b)).transpose(0, 1, 3, 2),
                                  orc.pack_conv_input_nhwc(x))
    got = gpuops.bconv(inp, filt, b, h, h, c, c, 3, 3, 1, pad, buf, buf, _variant(gpu, variant))
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("h,c", SWEEP)
def test_bconv_sweep_shapes_batch256(gpu, h, c):
    """The sweep at its configured batch of 256 on the default engine (the persistent kernel's int32 epilogue
    with every image group, pixel stream and channel group of the full-size launch), bit for bit."""
    b = 256
    r = rng(1000 + h + c)
    x = rm.pm1(r, (b, h, h, c))
    f = rm.pm1(r, (3, 3, c, c))
    pad, buf, _ = orc.conv_geometry(h, 3, 1)
    want = orc.bconv(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), c, c, 3, 3, 1, pad, buf, buf)
    got = gpuops.bconv(gpuops.pack_conv_input(x), gpuops.pack_conv_filter(f), b, h, h, c, c, 3, 3, 1, pad, buf, buf,
                       _variant(gpu, "mfma_f4"))
    np.testing.assert_array_equal(got, want)
    # the zero-padded cross-correlation it must equal (benchmark-bconv.cu:126-135), on a few images
    np.testing.assert_array_equal(got[:3], rm.xcorr_pm1(x[:3], f, 1, pad, pad, buf, buf))


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,h,cin,cout,R,stride", [(70, 9, 32, 16, 3, 2), (3, 12, 160, 40, 5, 2),
                                                   (130, 6, 96, 24, 1, 2), (5, 16, 64, 8, 7, 4),
                                                   (260, 5, 256, 64, 3, 1),
                                                   # 3x3 shapes of the persistent kernel's int32 epilogue: partial
                                                   # channel tile, partial image tile, stride 2, one-pixel frame
                                                   (70, 9, 64, 48, 3, 2), (33, 7, 192, 100, 3, 1), (8, 1, 128, 64, 3, 1),
                                                   (40, 2, 384, 32, 3, 1), (9, 6, 64, 33, 3, 1),
                                                   # whole channel tiles at Cin = 192 / 256 (one channel tile per wave through LDS)
                                                   (64, 4, 192, 64, 3, 1), (48, 3, 256, 96, 3, 1)])
def test_bconv_odd_shapes(gpu, variant, b, h, cin, cout, R, stride):
    r = rng(b + h + cin)
    x = rm.pm1(r, (b, h, h, cin))
    f = rm.pm1(r, (R, R, cin, cout))
    pad, buf, _ = orc.conv_geometry(h, R, stride)
    want = orc.bconv(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), cin, cout, R, R, stride, pad, buf, buf)
    got = gpuops.bconv(gpuops.pack_conv_input(x), gpuops.pack_conv_filter(f), b, h, h, cin, cout, R, R, stride,
                       pad, buf, buf, _variant(gpu, variant))
    np.testing.assert_array_equal(got, want)


def test_fc_out_bmm_bconv_random_shapes(gpu):
    """Seeded random FC / output layers and stand-alone bit-GEMMs / bit-convolutions on all three engines: ragged
    batches, K from one word to 25088, N from 8 to 1024, exact ties on FC thresholds, with and without split-K."""
    r = rng(4242)
    for it in range(60):
        variant = str(r.choice(["mfma_f4"] * 4 + ["popc", "mfma_i8"]))
        V = _variant(gpu, variant)
        kind = it % 4
        if kind == 0:
            b = int(r.choice([1, 3, 8, 13, 64, 100, 130, 256, 1000, 4100]))
            k = int(r.choice([32, 96, 128, 300, 512, 784, 1000, 1024, 2048, 4096, 25088]))
            n = int(r.choice([8, 32, 40, 64, 100, 160, 512, 1000, 1024]))
            b = min(b, max(1, int(1e7 // k)))
            case = ("fc", b, k, n, variant)
            x, w = r.standard_normal((b, k)).astype(np.float32), rm.pm1(r, (k, n))
            bn = r.normal(0, np.sqrt(k), n).astype(np.float32)
            wl = orc.pack_fc_weight(w)
            _, acc = orc.fc128(orc.in128(x), wl, bn, k, n, want_acc=True)
            bn[: min(n, 8)] = (k - 2 * acc)[0, : min(n, 8)]
            want = orc.fc128(orc.in128(x), wl, bn, k, n)
            inp, wbuf = gpuops.in128(x), gpuops.pack_fc_weight(w)
            np.testing.assert_array_equal(gpuops.fc128(inp, wbuf, bn, b, k, n, V), want, err_msg=str(case))
            np.testing.assert_array_equal(gpuops.fc128(inp, wbuf, bn, b, k, n, V, workspace=False), want,
                                          err_msg=str(case))
        elif kind == 1:
            b, k = int(r.choice([1, 8, 70, 256, 1000, 4100])), int(r.choice([32, 300, 512, 1000, 1024, 1536, 4096]))
            n = int(r.choice([10, 33, 72, 100, 1000]))
            case = ("out", b, k, n, variant)
            x, w = r.standard_normal((b, k)).astype(np.float32), rm.pm1(r, (k, n))
            scale, bias = r.normal(1, 0.1, n).astype(np.float32), r.normal(0, 1, n).astype(np.float32)
            want = orc.out128(orc.in128(x), orc.pack_fc_weight(w), scale, bias, k, n)
            got = gpuops.out128(gpuops.in128(x), gpuops.pack_fc_weight(w), scale, bias, b, k, n, V)
            np.testing.assert_array_equal(got, want, err_msg=str(case))
        elif kind == 2:
            m, n = int(r.choice([8, 77, 100, 300, 1024, 4100, 5000])), 32 * int(r.integers(1, 40))
            k = 32 * int(r.choice([1, 2, 3, 6, 16, 33, 48, 64]))
            a = r.integers(0, 2 ** 32, size=(m, k // 32), dtype=np.uint64).astype(np.uint32)
            bb = r.integers(0, 2 ** 32, size=(n, k // 32), dtype=np.uint64).astype(np.uint32)
            np.testing.assert_array_equal(gpuops.bmm(a, bb, m, n, k, V), orc.bmm(a, bb, k),
                                          err_msg=str(("bmm", m, n, k, variant)))
        else:
            b, h = int(r.choice([3, 8, 33, 64, 70, 130])), int(r.integers(1, 13))
            cin, cout = int(r.choice([32, 64, 96, 128, 160, 192, 256, 384])), int(r.choice([8, 16, 24, 33, 40, 48, 64, 100]))
            R, stride = int(r.choice([1, 3, 3, 3, 5])), int(r.choice([1, 1, 2]))
            x, f = rm.pm1(r, (b, h, h, cin)), rm.pm1(r, (R, R, cin, cout))
            pad, buf, _ = orc.conv_geometry(h, R, stride)
            want = orc.bconv(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), cin, cout, R, R, stride, pad, buf, buf)
            got = gpuops.bconv(gpuops.pack_conv_input(x), gpuops.pack_conv_filter(f), b, h, h, cin, cout, R, R, stride,
                               pad, buf, buf, V)
            np.testing.assert_array_equal(got, want, err_msg=str(("bconv", b, h, cin, cout, R, stride, variant)))


# --------------------------------------------------------------------------- Conv128 layer
class _PackedSource:
    """Stands in for the previous layer: a device buffer holding packed activations."""

    def __init__(self, packed):
        self.buf = gpuops.dev(packed)


def _residual_source(res_in, fmt):
    """Device copy of a residual [Hr][Wr][B][C] in the engine layout of format `fmt`, tagged the way the
    layer classes tag the tensors they produce (channel count, format, bound of |value|)."""
    hr, wr, b, c = res_in.shape
    if fmt == 2:  # 12 bits: groups of 16 channels, per pixel and group w0..w3 of every image, then w4, w5
        host = _pack_i12(res_in)
    else:
        grp, dt = (8, np.int16) if fmt == 1 else (4, np.int32)  # [Hr][Wr][ceil(C/grp)][B][grp]
        ng = (c + grp - 1) // grp
        pad = np.zeros((hr, wr, b, ng * grp), dt)
        pad[..., :c] = res_in
        host = np.ascontiguousarray(pad.reshape(hr, wr, b, ng, grp).transpose(0, 1, 3, 2, 4))
    rbuf = gpuops.dev(host)
    rbuf.channels, rbuf.format, rbuf.bound = c, fmt, int(np.abs(res_in).max())
    return rbuf


def _pack_i12(res):
    """int32 [Hr][Wr][B][C] -> the engine's 12-bit layout, written from its definition: value e of a group of 16
    channels at bits 12e..12e+11 (two's complement) of the 192-bit string w0..w5; per pixel and group the words
    w0..w3 of every image, then w4, w5 of every image."""
    hr, wr, b, c = res.shape
    assert np.abs(res).max() <= 2047 and b % 2 == 0
    g = (c + 15) // 16
    v = np.zeros((hr, wr, b, g * 16), np.int64)
    v[..., :c] = res
    v = (v & 0xfff).reshape(hr, wr, b, g, 16)
    big = np.zeros((hr, wr, b, g), object)
    for e in range(16):
        big = big + (v[..., e].astype(object) << (12 * e))
    words = np.stack([((big >> (32 * k)) & 0xffffffff).astype(np.uint64) for k in range(6)], axis=-1).astype(np.uint32)
    words = words.transpose(0, 1, 3, 2, 4)  # [Hr][Wr][G][B][6]
    return np.ascontiguousarray(np.concatenate([words[..., :4].reshape(hr, wr, g, 4 * b),
                                                words[..., 4:].reshape(hr, wr, g, 2 * b)], axis=-1))


def _run_conv_layer(gpu, variant, x, f, bn, stride=1, pool=1, ahead_fc=False, save_residual=False,
                    inject_residual=False, residual_channels=0, residual_pool=False, res_in=None, in_fmt=0,
                    out_fmt=None):
    b, h, w, cin = x.shape
    R, S, _, cout = f.shape
    layer = gpu.Conv128LayerParam("C", h, w, R, S, cin, cout, b, stride, stride, True, pool, pool, ahead_fc,
                                  save_residual, inject_residual, residual_channels, residual_pool,
                                  variant=_variant(gpu, variant), residual_format=out_fmt)
    src = gpuops.pack_conv_input(x)
    rbuf = _residual_source(res_in, in_fmt) if inject_residual else None
    layer.initialize(gpu.ArrayWeights([f, bn]), src, rbuf)
    layer.output_gpu.fill(0xCD)  # every output word must be written by the call
    if layer.output_residual_gpu is not None:
        layer.output_residual_gpu.fill(0xCD)
    layer.forward()
    layer.forward()  # idempotent: a second run on the same objects gives the same result
    gpuops.sync()
    return layer


CONV_CASES = [
    # b, h, cin, cout, stride, pool, ahead_fc
    (8, 8, 128, 128, 1, 1, False), (70, 8, 128, 128, 1, 2, False), (8, 7, 64, 96, 1, 2, False),
    (130, 12, 64, 128, 2, 1, False), (8, 9, 256, 32, 1, 3, False), (24, 4, 512, 512, 1, 2, True),
    (8, 4, 64, 160, 1, 2, True), (256, 7, 128, 64, 1, 1, False),
    # Cin = 192 / 384 (alexnet.cu:154-162) and 2x2 pooling with them
    (40, 13, 192, 384, 1, 1, False), (72, 13, 384, 256, 1, 1, False), (8, 6, 192, 96, 1, 2, True),
    (130, 9, 384, 64, 2, 1, False),
    # frames of one to three pixels (every tile is a border tile), odd sizes with stride 2
    (8, 1, 64, 64, 1, 1, False), (40, 2, 128, 32, 1, 2, False), (40, 3, 64, 64, 2, 1, False),
    (72, 5, 512, 40, 2, 1, True),
    # a single image, an odd handful, one more than a tile
    (1, 6, 64, 64, 1, 1, False), (3, 5, 128, 96, 2, 1, False), (33, 4, 256, 64, 1, 2, True),
    # pooled sizes that are rounded up: the last windows hold pixels past the convolution's own output, which
    # the reference computes from the taps still in the frame and ORs in (kernel.cuh:685-690); with a 4x4 pool
    # on 5 rows the windows' last two rows have no tap left (sum 0, decided by the sign of the threshold)
    (8, 5, 64, 64, 1, 4, False), (40, 7, 128, 96, 1, 2, True), (8, 11, 64, 40, 2, 2, False),
    (8, 3, 256, 64, 1, 2, False),
]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,h,cin,cout,stride,pool,ahead_fc", CONV_CASES)
def test_conv128_layer(gpu, variant, b, h, cin, cout, stride, pool, ahead_fc):
    r = rng(b + h + cin + cout + pool)
    x = rm.pm1(r, (b, h, h, cin))
    f = rm.pm1(r, (3, 3, cin, cout))
    bn = r.normal(0, np.sqrt(9 * cin), cout).astype(np.float32)
    inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)
    _, res = orc.conv128(inp, filt, bn, cin, cout, 3, 3, stride, True, 1, save_residual=True)
    bn[:4] = res[0, 0, 0, :4]  # ties on a border pixel
    bn[4:8] = [0.0, -0.0, 0.5, -0.5]  # decide pixels whose window has no tap in the frame (sum 0)
    want, _ = orc.conv128(inp, filt, bn, cin, cout, 3, 3, stride, True, pool, ahead_fc)
    layer = _run_conv_layer(gpu, variant, x, f, bn, stride, pool, ahead_fc)
    np.testing.assert_array_equal(layer.download_packed(), want)
    # what the reference's download_output() would return (tile-contiguous layout)
    oh = layer.output_height
    if ahead_fc:
        want_fmt = orc.fc_to_fmt(want, b, oh * oh * orc.pad128(cout))
    else:
        want_fmt = orc.conv_to_fmt(want, cout)
    np.testing.assert_array_equal(layer.download_output(), want_fmt)
    full = layer.download_full_output()
    assert full.shape == (b, oh, oh, cout)
    if not ahead_fc:
        np.testing.assert_array_equal(full, np.transpose(orc.unpack_bits(want, cout), (2, 0, 1, 3)))
    layer.release()


# (cin, cout): the persistent 3x3 kernel's instantiations (Cin 64 .. 512), a channel count that is not a
# multiple of 32 and an odd one (half-filled last 16-bit pair); formats of the injected and saved tensors
RES_SHAPES = [(64, 96), (128, 64), (256, 35), (512, 64), (192, 64), (384, 40), (96, 35)]
RES_FORMATS = [(0, 0), (1, 1), (0, 1), (1, 0)]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("in_fmt,out_fmt", RES_FORMATS)
@pytest.mark.parametrize("cin,cout", RES_SHAPES)
def test_conv128_residual_modes(gpu, variant, cin, cout, in_fmt, out_fmt):
    _residual_modes(gpu, variant, cin, cout, in_fmt, out_fmt, 72)


# the 12-bit format (|value| <= 2047: short filters, small injected values), against itself and the other two
@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("in_fmt,out_fmt", [(2, 2), (2, 1), (1, 2), (0, 2), (2, 0)])
@pytest.mark.parametrize("cin,cout", [(64, 96), (128, 64), (64, 35), (128, 160)])
def test_conv128_residual_modes_12_bit(gpu, variant, cin, cout, in_fmt, out_fmt):
    _residual_modes(gpu, variant, cin, cout, in_fmt, out_fmt, 72, amp=800)


@pytest.mark.parametrize("b", [2, 34, 66])
def test_conv128_residual_modes_12_bit_small_batch(gpu, b):
    _residual_modes(gpu, "mfma_f4", 64, 64, 2, 2, b, amp=800)


@pytest.mark.parametrize("b", [1, 5, 33])
@pytest.mark.parametrize("cin,cout", [(64, 64), (256, 96), (512, 64)])
def test_conv128_residual_modes_small_batch(gpu, b, cin, cout):
    """Batches below and just above one 32-image tile: lanes without an image must neither load nor store."""
    _residual_modes(gpu, "mfma_f4", cin, cout, 1, 1, b)


def _residual_modes(gpu, variant, cin, cout, in_fmt, out_fmt, b, amp=3000):
    r = rng(41 + cin + cout + b)
    h = 6
    x = rm.pm1(r, (b, h, h, cin))
    f = rm.pm1(r, (3, 3, cin, cout))
    bn = r.normal(0, 20, cout).astype(np.float32)
    inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)

    layer = _run_conv_layer(gpu, variant, x, f, bn, save_residual=True, out_fmt=out_fmt)
    assert layer.output_residual_gpu.format == out_fmt
    want, wres = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True)
    np.testing.assert_array_equal(layer.download_packed(), want)
    np.testing.assert_array_equal(layer.download_residual(), wres)
    np.testing.assert_array_equal(layer.download_residual_reference(), orc.residual_to_reference(wres))
    layer.release()

    # source narrower than the consumer and a limit that cuts through a channel tile
    src_ch, lim = (cout * 2) // 3, (cout * 5) // 6
    src = r.integers(-amp, amp, size=(h, h, b, src_ch)).astype(np.int32)
    layer = _run_conv_layer(gpu, variant, x, f, bn, save_residual=True, inject_residual=True,
                            residual_channels=lim, res_in=src, in_fmt=in_fmt, out_fmt=out_fmt)
    want, wres = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                             residual_channels=lim, res_in=src)
    np.testing.assert_array_equal(layer.download_packed(), want)
    np.testing.assert_array_equal(layer.download_residual(), wres)
    layer.release()

    # 2x2 max of a source twice the size; source wider than the limit
    src2 = r.integers(-amp, amp, size=(2 * h, 2 * h, b, cout)).astype(np.int32)
    layer = _run_conv_layer(gpu, variant, x, f, bn, save_residual=True, inject_residual=True,
                            residual_channels=cout // 2, residual_pool=True, res_in=src2, in_fmt=in_fmt,
                            out_fmt=out_fmt)
    want, wres = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                             residual_channels=cout // 2, residual_pool=True, res_in=src2)
    np.testing.assert_array_equal(layer.download_packed(), want)
    np.testing.assert_array_equal(layer.download_residual(), wres)
    layer.release()

    # inject only (the last block of the ResNet saves nothing)
    layer = _run_conv_layer(gpu, variant, x, f, bn, inject_residual=True, residual_channels=cout,
                            res_in=src2[:h, :h], in_fmt=in_fmt)
    want, _ = orc.conv128(inp, filt, bn, cin, cout, 3, 3, inject_residual=True, residual_channels=cout,
                          res_in=src2[:h, :h])
    np.testing.assert_array_equal(layer.download_packed(), want)
    layer.release()


def _window_maximum(res):
    """[P][Q][B][O] -> [P/2][Q/2][B][O]: the maximum over non-overlapping 2x2 windows of pixels (kernel.cuh:775-782)."""
    p, q, b, o = res.shape
    return res.reshape(p // 2, 2, q // 2, 2, b, o).max(axis=(1, 3))


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,h,cin,cout,in_fmt,amp,lim", [
    (64, 8, 64, 64, 2, 100, 64), (70, 6, 128, 128, 1, 3000, 128), (8, 4, 256, 256, 1, 500, 128),
    (40, 10, 64, 128, 2, 2000, 64), (8, 4, 512, 512, 1, 20000, 512), (24, 6, 192, 64, 2, 50, 32),
    (40, 4, 384, 128, 1, 900, 96),
    # more windows than workgroups (a workgroup walks several windows, the last round ragged)
    (256, 28, 64, 64, 2, 100, 64), (128, 20, 128, 128, 1, 3000, 128),
    # not served: odd frame, int32 output (bound above 32767), output channels not a multiple of 64, int32 source
    (8, 7, 64, 64, 2, 100, 64), (8, 4, 64, 64, 1, 32700, 64), (8, 4, 64, 96, 2, 100, 96), (8, 4, 128, 64, 0, 100, 64)])
def test_conv128_saved_residual_as_window_maximum(gpu, variant, b, h, cin, cout, in_fmt, amp, lim):
    """A saved residual whose only reader injects it with residual_pool is stored as its 2x2 maximum (a quarter of
    the tensor), which that reader then injects as it is.  Same bits and residuals as the reference's order of
    operations (save the full tensor, kernel.cuh:818-824; take the maximum when reading, kernel.cuh:775-782); the
    full tensor is still there when somebody asks for it."""
    r = rng(b * 7 + h + cin + cout)
    x = rm.pm1(r, (b, h, h, cin))
    f = rm.pm1(r, (3, 3, cin, cout))
    bn = r.normal(0, 20, cout).astype(np.float32)
    src = r.integers(-amp, amp + 1, size=(h, h, b, cout)).astype(np.int32)
    h2 = (h + 1) // 2
    x2 = rm.pm1(r, (b, h2, h2, cout))
    f2 = rm.pm1(r, (3, 3, cout, cout))
    bn2 = r.normal(0, 40, cout).astype(np.float32)
    inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)
    want_p, res_p = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                                residual_channels=lim, res_in=src)

    prod = gpu.Conv128LayerParam("P", h, h, 3, 3, cin, cout, b, 1, 1, True, 1, 1, False, True, True, lim, False,
                                 variant=_variant(gpu, variant))
    prod.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x), _residual_source(src, in_fmt))
    served = variant == "mfma_f4" and h % 2 == 0 and cout % 64 == 0 and in_fmt != 0 and prod.output_residual_gpu.format != 0
    if h % 2:  # an odd frame has no 2x2 reader at all: the producer alone
        prod.forward()
        got, pooled = prod.download_saved_residual()
        assert not pooled
        np.testing.assert_array_equal(got, res_p)
        prod.release()
        return
    want_c, res_c = orc.conv128(orc.pack_conv_input_nhwc(x2), orc.pack_conv_filter(f2), bn2, cout, cout, 3, 3,
                                save_residual=True, inject_residual=True, residual_channels=cout // 2,
                                residual_pool=True, res_in=res_p)
    cons = gpu.Conv128LayerParam("C", h2, h2, 3, 3, cout, cout, b, 1, 1, True, 1, 1, False, True, True, cout // 2, True,
                                 variant=_variant(gpu, variant))
    cons.initialize(gpu.ArrayWeights([f2, bn2]), gpuops.pack_conv_input(x2), prod.get_output_residual_gpu())
    assert ("conv3x3_mfma_f4_kernel" in prod.kernel_name() and ", 2, true>" in prod.kernel_name()) == served
    prod.output_residual_gpu.fill(0xCD)
    for _ in range(2):
        prod.forward()
        cons.forward()
    got, pooled = prod.download_saved_residual()
    assert pooled == served
    np.testing.assert_array_equal(got, _window_maximum(res_p) if pooled else res_p)
    np.testing.assert_array_equal(prod.download_packed(), want_p)
    np.testing.assert_array_equal(cons.download_packed(), want_c)
    np.testing.assert_array_equal(cons.download_saved_residual()[0], res_c)
    # somebody asks for the full tensor: it is produced, and it is what the layers work with from then on
    np.testing.assert_array_equal(prod.download_residual(), res_p)
    np.testing.assert_array_equal(prod.download_residual_reference(), orc.residual_to_reference(res_p))
    prod.forward()
    cons.output_gpu.fill(0xCD)
    cons.forward()
    assert not prod.download_saved_residual()[1]
    np.testing.assert_array_equal(cons.download_packed(), want_c)
    np.testing.assert_array_equal(cons.download_residual(), res_c)
    cons.release()
    prod.release()


@pytest.mark.parametrize("b,h,w,cin,cout,in_fmt", [(40, 6, 10, 64, 64, 2), (16, 8, 4, 128, 128, 1),
                                                   (64, 2, 14, 256, 256, 1), (8, 12, 2, 64, 128, 2)])
def test_conv128_window_maximum_on_frames_that_are_not_square(gpu, b, h, w, cin, cout, in_fmt):
    """The window walk of the producer and the pooled injection of the reader on frames with different heights and
    widths (a transposed row / column count anywhere would mix up pixels)."""
    r = rng(b + 13 * h + 29 * w + cin)
    x, f = rm.pm1(r, (b, h, w, cin)), rm.pm1(r, (3, 3, cin, cout))
    bn = r.normal(0, 20, cout).astype(np.float32)
    src = r.integers(-300, 301, size=(h, w, b, cout)).astype(np.int32)
    x2, f2 = rm.pm1(r, (b, h // 2, w // 2, cout)), rm.pm1(r, (3, 3, cout, cout))
    bn2 = r.normal(0, 40, cout).astype(np.float32)
    want_p, res_p = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, cin, cout, 3, 3,
                                save_residual=True, inject_residual=True, residual_channels=cout, res_in=src)
    want_c, res_c = orc.conv128(orc.pack_conv_input_nhwc(x2), orc.pack_conv_filter(f2), bn2, cout, cout, 3, 3,
                                save_residual=True, inject_residual=True, residual_channels=cout // 2,
                                residual_pool=True, res_in=res_p)
    prod = gpu.Conv128LayerParam("P", h, w, 3, 3, cin, cout, b, 1, 1, True, 1, 1, False, True, True, cout, False)
    prod.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x), _residual_source(src, in_fmt))
    cons = gpu.Conv128LayerParam("C", h // 2, w // 2, 3, 3, cout, cout, b, 1, 1, True, 1, 1, False, True, True, cout // 2,
                                 True)
    cons.initialize(gpu.ArrayWeights([f2, bn2]), gpuops.pack_conv_input(x2), prod.get_output_residual_gpu())
    assert ", 2, true>" in prod.kernel_name()
    prod.forward()
    cons.forward()
    got, pooled = prod.download_saved_residual()
    assert pooled
    np.testing.assert_array_equal(got, _window_maximum(res_p))
    np.testing.assert_array_equal(prod.download_packed(), want_p)
    np.testing.assert_array_equal(cons.download_packed(), want_c)
    np.testing.assert_array_equal(cons.download_saved_residual()[0], res_c)
    cons.release()
    prod.release()


def test_saved_residual_stays_full_for_other_readers(gpu):
    """The 2x2 maximum alone is stored only while every hand-out of the tensor went to a pooling Conv128 reader."""
    r = rng(31)
    b, h, c = 8, 8, 64
    x, f = rm.pm1(r, (b, h, h, c)), rm.pm1(r, (3, 3, c, c))
    bn = r.normal(0, 20, c).astype(np.float32)
    src = r.integers(-50, 51, size=(h, h, b, c)).astype(np.int32)
    _, res_p = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, c, c, 3, 3, save_residual=True,
                           inject_residual=True, residual_channels=c, res_in=src)

    def producer():
        p = gpu.Conv128LayerParam("P", h, h, 3, 3, c, c, b, 1, 1, True, 1, 1, False, True, True, c, False)
        return p.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x), _residual_source(src, 2))

    def reader(p, pool, size):
        x2, f2 = rm.pm1(r, (b, size, size, c)), rm.pm1(r, (3, 3, c, c))
        q = gpu.Conv128LayerParam("C", size, size, 3, 3, c, c, b, 1, 1, True, 1, 1, False, False, True, c, pool)
        return q.initialize(gpu.ArrayWeights([f2, bn]), gpuops.pack_conv_input(x2), p.get_output_residual_gpu())

    # no reader at all; a pooling reader; a pooling and a plain reader; a pooling reader and a pointer nobody registered
    for readers, extra_handout, want_pooled in (((), 0, False), ((True,), 0, True), ((True, False), 0, False),
                                                 ((True,), 1, False), ((True, True), 0, True)):
        p = producer()
        qs = [reader(p, pool, h // 2 if pool else h) for pool in readers]
        for _ in range(extra_handout):
            p.get_output_residual_gpu()
        p.forward()
        for q in qs:
            q.forward()
        got, pooled = p.download_saved_residual()
        assert pooled == want_pooled, (readers, extra_handout)
        np.testing.assert_array_equal(got, _window_maximum(res_p) if pooled else res_p)
        if want_pooled:  # a reader that goes away takes its registration with it
            qs[0].release()
            p.forward()
            assert not p.download_saved_residual()[1]
        for q in qs:
            q.release()
        p.release()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("b,cin,cout,R,ahead_fc", [(8, 512, 128, 1, True), (40, 128, 64, 1, False), (33, 256, 96, 1, True),
                                                   (8, 1024, 256, 1, False), (8, 128, 64, 3, True)])
def test_conv128_on_a_one_pixel_frame(gpu, variant, b, cin, cout, R, ahead_fc):
    """A convolution whose frame is one pixel has the shape of a fully connected layer (one output pixel, and one
    tap with a 1x1 filter), but its filter buffer is a convolution's: it holds the sign-bit rows only, not the copy in
    lane order that the fully connected kernel of the FP4 engine reads."""
    r = rng(b + cin + cout + R)
    x, f = rm.pm1(r, (b, 1, 1, cin)), rm.pm1(r, (R, R, cin, cout))
    bn = r.normal(0, np.sqrt(cin) * 0.5, cout).astype(np.float32)
    want, _ = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, cin, cout, R, R, 1, True, 1, ahead_fc)
    layer = gpu.Conv128LayerParam("C", 1, 1, R, R, cin, cout, b, 1, 1, True, 1, 1, ahead_fc, variant=_variant(gpu, variant))
    layer.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x))
    assert "fc_mfma" not in layer.kernel_name()
    layer.output_gpu.fill(0xCD)
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(layer.download_packed(), want)
    layer.release()


def test_conv128_random_shapes(gpu):
    """Seeded random bit-convolution layers: non-square frames of 1-14 pixels, 3x3 mostly (also 1x1 / 3x5 / 5x5 ...),
    strides, pools, FC-ready outputs, every residual mode with random storage formats, channel limits that cut through
    tiles and sources narrower or wider than the consumer, all three engines."""
    r = rng(777)
    kernels = set()
    for it in range(90):
        R, S = (3, 3) if r.integers(0, 5) else (int(r.choice([1, 3, 5])), int(r.choice([1, 3, 5])))
        stride, pool = int(r.choice([1, 1, 2])), int(r.choice([1, 1, 1, 2, 2, 3]))
        h, w = int(r.integers(1, 15)), int(r.integers(1, 15))
        b = int(r.choice([1, 3, 8, 32, 33, 40, 64, 70, 128, 130]))
        cin = int(r.choice([32, 64, 64, 96, 128, 128, 160, 192, 256, 384, 512]))
        cout = int(r.choice([32, 35, 40, 64, 64, 96, 128, 160, 256]))
        if b * h * w * cin > 3e6:
            b = max(1, int(3e6 // (h * w * cin)))
        ahead_fc = bool(r.integers(0, 4) == 0)
        variant = str(r.choice(["mfma_f4"] * 4 + ["popc", "mfma_i8"]))
        # 0 none, 1 save, 2 inject + save, 3 inject the 2x2 maximum + save, 4 inject only
        mode = int(r.integers(0, 5)) if pool == 1 and not ahead_fc else 0
        save, inject, rpool = mode in (1, 2, 3), mode in (2, 3, 4), mode == 3
        in_fmt, out_fmt = int(r.integers(0, 3)), int(r.integers(0, 3))
        amp = 800 if 2 in (in_fmt, out_fmt) else 3000
        if 2 in (in_fmt, out_fmt) and b % 2:
            b += 1  # the 12-bit format pairs images
        if out_fmt == 2 and cin * R * S + amp > 2047:
            out_fmt = 1
        x, f = rm.pm1(r, (b, h, w, cin)), rm.pm1(r, (R, S, cin, cout))
        bn = r.normal(0, np.sqrt(cin * R * S) * 0.5, cout).astype(np.float32)
        bn[:4] = [0.0, -0.0, 0.5, np.nan]
        inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)
        ph, pw = gpu.lib.tcbnn_conv_out(h, R, stride, 1, 1), gpu.lib.tcbnn_conv_out(w, S, stride, 1, 1)
        lim = int(r.choice([cout, cout // 2, (cout * 5) // 6, max(1, cout - 1)])) if inject else 0
        src = None
        if inject:
            src_ch = int(r.choice([cout, max(1, (cout * 2) // 3), cout + 16]))
            src = r.integers(-amp, amp, size=((2 * ph, 2 * pw) if rpool else (ph, pw)) + (b, src_ch)).astype(np.int32)
        case = dict(it=it, b=b, h=h, w=w, cin=cin, cout=cout, R=R, S=S, stride=stride, pool=pool, ahead_fc=ahead_fc,
                    variant=variant, mode=mode, in_fmt=in_fmt, out_fmt=out_fmt, lim=lim)
        want, wres = orc.conv128(inp, filt, bn, cin, cout, R, S, stride, True, pool, ahead_fc, save, inject, lim,
                                 rpool, src)
        layer = gpu.Conv128LayerParam("C", h, w, R, S, cin, cout, b, stride, stride, True, pool, pool, ahead_fc,
                                      save, inject, lim, rpool, variant=_variant(gpu, variant),
                                      residual_format=out_fmt if save else None)
        layer.initialize(gpu.ArrayWeights([f, bn]), gpuops.pack_conv_input(x),
                         _residual_source(src, in_fmt) if inject else None)
        layer.output_gpu.fill(0xCD)
        kernels.add(layer.kernel_name())
        layer.forward()
        gpuops.sync()
        np.testing.assert_array_equal(layer.download_packed(), want, err_msg=str(case))
        if save:
            np.testing.assert_array_equal(layer.download_residual(), wres, err_msg=str(case))
        layer.release()
    assert sum(k.startswith("conv3x3_mfma_f4_kernel") for k in kernels) >= 15, kernels


def test_residual_format_follows_the_bound(gpu):
    """The layer classes store a residual in 16 bits only when |value| <= 32767 is certain: the first
    layer's bound comes from the actual input, every bit convolution adds Cin*R*S."""
    lib = gpu.lib
    assert lib.tcbnn_residual_format_for_bound(32767) == 1 and lib.tcbnn_residual_format_for_bound(32768) == 0
    assert lib.tcbnn_residual_format_narrowest(2047, 8) == 2 and lib.tcbnn_residual_format_narrowest(2048, 8) == 1
    assert lib.tcbnn_residual_format_narrowest(2047, 7) == 1 and lib.tcbnn_residual_format_narrowest(40000, 8) == 0
    assert lib.tcbnn_residual_bytes(3, 5, 17, 12, 2) == 3 * 5 * 2 * 12 * 24  # 17 channels: 2 groups of 16, 24 bytes
    assert lib.tcbnn_inconv_residual_bound(7, 7, float("inf")) == 2 ** 31 - 1
    assert lib.tcbnn_inconv_residual_bound(7, 7, float("nan")) == 2 ** 31 - 1
    assert 147 * 5 <= lib.tcbnn_inconv_residual_bound(7, 7, 5.0) <= 147 * 5 + 3
    assert lib.tcbnn_conv_residual_bound(512, 3, 3, 1000) == 5608
    assert lib.tcbnn_residual_bytes(3, 5, 7, 11, 0) == 3 * 5 * 2 * 11 * 16  # 7 channels: 2 groups of 4
    assert lib.tcbnn_residual_bytes(3, 5, 9, 11, 1) == 3 * 5 * 2 * 11 * 16  # 9 channels: 2 groups of 8
    r = rng(77)
    b, h, cout = 4, 16, 64
    f = rm.pm1(r, (7, 7, 3, cout))
    bn = r.normal(0, 12, cout).astype(np.float32)
    # the bound is the largest window sum of |x| (147 terms of mean 0.8 here): 12 bits; x 20: 16 bits; x 400: int32
    for scale, fmt in ((1.0, 2), (20.0, 1), (400.0, 0)):
        x = (r.standard_normal((b, 3, h, h)) * scale).astype(np.float32)
        want, wres = orc.inconv128(x, f, bn, 4, True, 1, True)
        layer = gpu.InConv128LayerParam("Conv1", h, h, 7, 7, 3, cout, b, 4, 4, True, 1, 1, True)
        layer.initialize(x, gpu.ArrayWeights([f, bn]))
        assert layer.output_residual_gpu.format == fmt
        assert np.abs(wres).max() <= layer.output_residual_gpu.bound
        # the bound is the window sum of |x|, within its slack, and never below what any filter can reach
        xa = np.abs(x).sum(axis=1)
        win = max(xa[i, max(0, 4 * y - 3):4 * y + 4, max(0, 4 * q - 3):4 * q + 4].sum()
                  for i in range(b) for y in range(4) for q in range(4))
        assert win <= layer.output_residual_gpu.bound <= win * 1.002 + 2
        layer.forward()
        gpuops.sync()
        np.testing.assert_array_equal(layer.download_packed(), want)
        np.testing.assert_array_equal(layer.download_residual(), wres)
        if fmt != 0:
            with pytest.raises(gpu.TcbnnError):
                layer.set_input(x * 1000)
        layer.release()


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("with_residual", [False, True])
def test_conv128_special_thresholds(gpu, variant, with_residual):
    """NaN, +-inf and exactly met thresholds (kernel.cuh:795-796: bit = (res < bn) ? 0 : 1, so NaN gives 1),
    on full 32-channel tiles, where the matrix-core kernel derives the bit from the sign of res - bn."""
    r = rng(99)
    b, h, cin, cout = 40, 5, 128, 64
    x = rm.pm1(r, (b, h, h, cin))
    f = rm.pm1(r, (3, 3, cin, cout))
    inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)
    src = r.integers(-500, 500, size=(h, h, b, cout)).astype(np.int32) if with_residual else None
    kw = dict(save_residual=True, inject_residual=True, residual_channels=cout, res_in=src) if with_residual else {}
    _, res = orc.conv128(inp, filt, np.zeros(cout, np.float32), cin, cout, 3, 3, save_residual=True,
                         **{k: v for k, v in kw.items() if k != "save_residual"})
    bn = r.normal(0, 30, cout).astype(np.float32)
    bn[0:8] = np.nan
    bn[8:12] = np.inf
    bn[12:16] = -np.inf
    bn[16:48] = res[2, 2, 3, 16:48]          # met exactly by one (pixel, image) each
    bn[48:52] = res[0, 0, 0, 48:52] + 0.5    # half-way values
    want, _ = orc.conv128(inp, filt, bn, cin, cout, 3, 3, **kw)
    layer = _run_conv_layer(gpu, variant, x, f, bn, **({"in_fmt": 1, **kw} if with_residual else {}))
    np.testing.assert_array_equal(layer.download_packed(), want)
    bits = orc.unpack_bits(want, cout)       # [H][W][B][C] of +-1
    assert (bits[..., 0:8] == 1).all() and (bits[..., 8:12] == -1).all() and (bits[..., 12:16] == 1).all()
    layer.release()


def test_conv128_rejects_residual_with_pooling(gpu):
    x = rm.pm1(rng(1), (8, 4, 4, 64))
    f = rm.pm1(rng(2), (3, 3, 64, 32))
    layer = gpu.Conv128LayerParam("C", 4, 4, 3, 3, 64, 32, 8, 1, 1, True, 2, 2, False, True)
    layer.initialize(gpu.ArrayWeights([f, np.zeros(32, np.float32)]), gpuops.pack_conv_input(x))
    with pytest.raises(gpu.TcbnnError):
        layer.forward()


# --------------------------------------------------------------------------- first layer
@pytest.mark.parametrize("b,h,R,stride,cout,pool,save", [(8, 32, 3, 1, 128, 1, False), (5, 20, 7, 4, 64, 1, True),
                                                         (70, 12, 3, 1, 32, 2, False), (3, 13, 5, 2, 96, 1, True),
                                                         (2, 224, 7, 4, 64, 1, True),
                                                         # staging schemes of the tiled kernel: wide filter (linear
                                                         # scheme), partial image tiles, whole tiles, odd channel counts
                                                         (70, 24, 11, 4, 64, 1, True), (66, 20, 7, 4, 40, 1, True),
                                                         (9, 17, 3, 2, 33, 1, True), (64, 16, 7, 4, 64, 1, True),
                                                         (128, 10, 3, 1, 64, 1, True),
                                                         # three image tiles: not a divisor of the 8 XCD slots, so
                                                         # the plain workgroup order of both un-pooled kernels
                                                         (130, 12, 3, 1, 32, 1, True), (192, 9, 5, 2, 64, 1, False),
                                                         # pooled first layers (alexnet.cu:143-144): tiled kernel
                                                         # with 2x2 windows, odd row / column counts, a 3x3 pool
                                                         # (generic kernel)
                                                         (70, 24, 11, 4, 64, 2, False), (8, 26, 3, 2, 64, 2, False),
                                                         (9, 18, 7, 2, 40, 2, False), (5, 18, 3, 1, 64, 3, False),
                                                         # pooled sizes that are rounded up (kernel.cuh:587-596
                                                         # walks pool * output pixels): generic and tiled kernels,
                                                         # windows whose last rows have no tap in the frame
                                                         (5, 17, 3, 1, 64, 3, False), (6, 5, 3, 1, 40, 4, False),
                                                         (70, 7, 3, 1, 64, 2, False), (9, 21, 7, 4, 64, 2, False)])
def test_inconv128_layer(gpu, b, h, R, stride, cout, pool, save):
    r = rng(b + h + R + cout)
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    f = rm.pm1(r, (R, R, 3, cout))
    bn = r.normal(0, np.sqrt(3 * R * R), cout).astype(np.float32)
    bn[:4] = [0.0, -0.0, 1e-30, -1e-30]  # decide pixels whose window has no tap in the frame (sum 0)
    want, wres = orc.inconv128(x, f, bn, stride, True, pool, save)
    # the kernel that stages [batch][3][H][W] through LDS and, for un-pooled layers, the one that reads a packed
    # copy of the input: two paths of the same entry point (a pooled layer ignores the request for a packed copy)
    for layout in ([None, gpu._lib.INCONV_INPUT_PACKED] if pool == 1 else [gpu._lib.INCONV_INPUT_PACKED]):
        layer = gpu.InConv128LayerParam("Conv1", h, h, R, R, 3, cout, b, stride, stride, True, pool, pool, save,
                                        input_layout=layout)
        layer.initialize(x, gpu.ArrayWeights([f, bn]))
        assert ("direct" in layer.kernel_name()) == (pool == 1 and layout is not None), layer.kernel_name()
        layer.forward()
        gpuops.sync()
        np.testing.assert_array_equal(layer.download_packed(), want)
        np.testing.assert_array_equal(layer.download_output(), orc.conv_to_fmt(want, cout))
        if save:
            np.testing.assert_array_equal(layer.download_residual(), wres)
        layer.release()


@pytest.mark.parametrize("b,h,w,R,S,sh,sw,padding", [(5, 20, 20, 7, 7, 4, 4, 1), (70, 9, 13, 3, 5, 1, 2, 1),
                                                     (64, 70, 66, 3, 3, 1, 1, 1), (3, 16, 16, 3, 3, 1, 1, 0),
                                                     (130, 11, 8, 11, 3, 4, 1, 1)])
def test_inconv_pack_input(gpu, b, h, w, R, S, sh, sw, padding):
    """The packed copy of a first-layer input: [Hp][Wp][batch][3], the frame at the padding offsets, zeros around."""
    lib = gpu._lib.lib
    x = rng(b + h + w).standard_normal((b, 3, h, w)).astype(np.float32)
    P, Q = lib.tcbnn_conv_out(h, R, sh, padding, 1), lib.tcbnn_conv_out(w, S, sw, padding, 1)
    Hp, Wp = (P - 1) * sh + R, (Q - 1) * sw + S
    ph, pw = lib.tcbnn_conv_pad(h, R, sh, padding), lib.tcbnn_conv_pad(w, S, sw, padding)
    n = lib.tcbnn_inconv_packed_input_floats(b, h, w, R, S, sh, sw, padding)
    assert n == Hp * Wp * b * 3
    want = np.zeros((max(Hp, ph + h), max(Wp, pw + w), b, 3), np.float32)
    want[ph:ph + h, pw:pw + w] = np.transpose(x, (2, 3, 0, 1))
    want = want[:Hp, :Wp]  # (without padding the last rows / columns that no window reaches are cut)
    src = gpuops.DeviceBuffer.from_numpy(x)
    dst = gpuops.DeviceBuffer(4 * n)
    dst.fill(0xff)
    gpu._lib.check(lib.tcbnn_inconv_pack_input(src.ptr, dst.ptr, b, h, w, R, S, sh, sw, padding, None))
    gpuops.sync()
    got = dst.to_numpy(np.float32, (Hp, Wp, b, 3))
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    src.free()
    dst.free()


def test_inconv128_random_shapes(gpu):
    """Seeded random first layers (non-square frames and filters, strides 1-4, pools 1-3, with and without padding,
    ragged batches and channel counts, thresholds 0 / -0 / NaN / inf) on every kernel the entry point chooses from,
    both input layouts where the layer is un-pooled."""
    r = rng(2024)
    kernels = set()
    for it in range(70):
        R, S = int(r.choice([1, 2, 3, 5, 7, 11])), int(r.choice([1, 2, 3, 5, 7, 11]))
        stride, pool = int(r.choice([1, 1, 2, 3, 4])), int(r.choice([1, 1, 1, 2, 3]))
        padding = bool(r.integers(0, 4) > 0)
        h, w = int(r.integers(max(R, 2), 41)), int(r.integers(max(S, 2), 41))
        b = int(r.choice([1, 2, 7, 33, 64, 65, 128, 130, 192]))
        cout = int(r.choice([8, 32, 33, 40, 64, 96, 100, 128]))
        save = bool(r.integers(0, 2)) and pool == 1
        x = (r.standard_normal((b, 3, h, w)) * r.choice([0.1, 1.0, 3.0])).astype(np.float32)
        f = rm.pm1(r, (R, S, 3, cout))
        bn = r.normal(0, np.sqrt(3 * R * S), cout).astype(np.float32)
        bn[:4] = [0.0, -0.0, np.nan, np.inf]
        want, wres = orc.inconv128(x, f, bn, stride, padding, pool, save)
        if want.size == 0:
            continue
        for layout in ([None, gpu._lib.INCONV_INPUT_PACKED] if pool == 1 else [None]):
            case = dict(b=b, h=h, w=w, R=R, S=S, stride=stride, pool=pool, padding=padding, cout=cout, save=save,
                        layout=layout)
            layer = gpu.InConv128LayerParam("Conv1", h, w, R, S, 3, cout, b, stride, stride, padding, pool, pool,
                                            save, input_layout=layout)
            layer.initialize(x, gpu.ArrayWeights([f, bn]))
            kernels.add(layer.kernel_name())
            layer.forward()
            gpuops.sync()
            np.testing.assert_array_equal(layer.download_packed(), want, err_msg=str(case))
            if save:
                np.testing.assert_array_equal(layer.download_residual(), wres, err_msg=str(case))
            layer.release()
    assert {"inconv_direct_kernel", "inconv_generic_kernel"} <= kernels and len(kernels) >= 8, kernels


def test_inconv128_packed_input_rules(gpu):
    """A packed input is refused for a pooled layer and for an unknown layout value; set_input repacks."""
    r = rng(77)
    b, h, cout = 6, 18, 64
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    f = rm.pm1(r, (3, 3, 3, cout))
    bn = r.normal(0, 5, cout).astype(np.float32)
    plain = gpu.InConv128LayerParam("Conv1", h, h, 3, 3, 3, cout, b, 1, 1, True, 1, 1, True)
    assert plain.input_layout is None and plain._packed_floats() == 0  # the packed copy is a request, never a default
    layer = gpu.InConv128LayerParam("Conv1", h, h, 3, 3, 3, cout, b, 1, 1, True, 1, 1, True,
                                    input_layout=gpu._lib.INCONV_INPUT_PACKED)
    layer.initialize(x, gpu.ArrayWeights([f, bn]))
    d = layer._desc()
    assert d.input_layout == gpu._lib.INCONV_INPUT_PACKED
    d.pool_height = d.pool_width = 2
    assert gpu._lib.lib.tcbnn_inconv128_forward(d, None) != 0
    d = layer._desc()
    d.input_layout = 7
    assert gpu._lib.lib.tcbnn_inconv128_forward(d, None) != 0
    x2 = (0.5 * r.standard_normal((b, 3, h, h))).astype(np.float32)
    want, wres = orc.inconv128(x2, f, bn, 1, True, 1, True)
    layer.set_input(x2)
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(layer.download_packed(), want)
    np.testing.assert_array_equal(layer.download_residual(), wres)
    layer.release()


_LINEAR_STAGING_CHECK = """
import numpy as np
import tcbnn_amd
from tcbnn_amd import _lib
from oracle import orc
_lib.set_device(0)
r = np.random.default_rng(3)
for (b, h, R, stride, cout, pool, save) in [(70, 24, 11, 4, 64, 2, False), (9, 20, 7, 4, 40, 1, True), (64, 12, 3, 1, 64, 1, True)]:
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    f = (r.integers(0, 2, size=(R, R, 3, cout)) * 2 - 1).astype(np.float32)
    bn = r.normal(0, np.sqrt(3 * R * R), cout).astype(np.float32)
    want, wres = orc.inconv128(x, f, bn, stride, True, pool, save)
    layer = tcbnn_amd.InConv128LayerParam("Conv1", h, h, R, R, 3, cout, b, stride, stride, True, pool, pool, save)
    layer.initialize(x, tcbnn_amd.ArrayWeights([f, bn]))
    assert layer.kernel_name().split(", ")[1] == "false", layer.kernel_name()  # <passes, row-wise staging, ...>
    layer.forward()
    _lib.device_synchronize()
    assert np.array_equal(layer.download_packed(), want)
    if save:
        assert np.array_equal(layer.download_residual(), wres)
print("linear staging ok")
"""


def test_inconv128_linear_staging(gpu):
    """The staging scheme for images too large for 32-bit buffer offsets, selected here by its switch (the
    library reads it once per process, hence the child process)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, TCBNN_INCONV_STAGING="linear", PYTHONPATH=root)
    proc = subprocess.run([sys.executable, "-c", _LINEAR_STAGING_CHECK], env=env, cwd=root, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and "linear staging ok" in proc.stdout, proc.stdout


def test_inconv128_special_thresholds(gpu):
    """NaN, +-inf and exactly met thresholds in the first layer (kernel.cuh:655: bit = !(acc < bn))."""
    r = rng(321)
    b, h, cout = 6, 16, 64
    x = rm.pm1(r, (b, 3, h, h))  # +-1 input: sums are exact integers, ties can be constructed
    f = rm.pm1(r, (7, 7, 3, cout))
    _, res = orc.inconv128(x, f, np.zeros(cout, np.float32), 4, True, 1, True)
    bn = r.normal(0, 8, cout).astype(np.float32)
    bn[0:4] = np.array([0x7fc00000, 0xffc00000, 0x7fa00000, 0xff800001], np.uint32).view(np.float32)  # quiet,
    bn[4:6] = np.inf                                                     # negative, signalling, smallest payload
    bn[6:8] = -np.inf
    bn[8:40] = res[1, 2, 3, 8:40]
    want, wres = orc.inconv128(x, f, bn, 4, True, 1, True)
    bits = orc.unpack_bits(want, cout)
    assert (bits[..., 0:4] == 1).all() and (bits[..., 4:6] == -1).all() and (bits[..., 6:8] == 1).all()
    for layout in (None, gpu._lib.INCONV_INPUT_PACKED):  # the two kernels test a threshold for NaN in different ways
        layer = gpu.InConv128LayerParam("Conv1", h, h, 7, 7, 3, cout, b, 4, 4, True, 1, 1, True, input_layout=layout)
        layer.initialize(x, gpu.ArrayWeights([f, bn]))
        layer.forward()
        gpuops.sync()
        np.testing.assert_array_equal(layer.download_packed(), want)
        np.testing.assert_array_equal(layer.download_residual(), wres)
        layer.release()


def test_inconv128_small_batch_is_repeatable(gpu):
    """Few waves per SIMD is the worst case for the register-indexed accumulation of the
    first layer (index write -> use needs wait states): every repeat must match the oracle."""
    r = rng(226)
    b, h, cout = 2, 224, 64
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    f = rm.pm1(r, (7, 7, 3, cout))
    bn = r.normal(0, 12, cout).astype(np.float32)
    want, wres = orc.inconv128(x, f, bn, 4, True, 1, True)
    layer = gpu.InConv128LayerParam("Conv1", h, h, 7, 7, 3, cout, b, 4, 4, True, 1, 1, True)
    layer.initialize(x, gpu.ArrayWeights([f, bn]))
    for _ in range(12):
        layer.output_gpu.fill(0)
        layer.forward()
        gpuops.sync()
        np.testing.assert_array_equal(layer.download_packed(), want)
        np.testing.assert_array_equal(layer.download_residual(), wres)
    layer.release()


def test_inconv128_presigned_input_is_exact_integer_conv(gpu):
    """The config's 'input binarized by sign' variant: +-1.0f input, sums are exact integers."""
    r = rng(5)
    b, h, cout = 8, 32, 128
    xs = rm.pm1(r, (b, 3, h, h))
    f = rm.pm1(r, (3, 3, 3, cout))
    want = rm.xcorr_pm1(np.transpose(xs, (0, 2, 3, 1)), f, 1, 1, 1, h, h)
    layer = gpu.InConv128LayerParam("Conv1", h, h, 3, 3, 3, cout, b, 1, 1, True, 1, 1, True)
    layer.initialize(xs, gpu.ArrayWeights([f, np.zeros(cout, np.float32)]))
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(np.transpose(layer.download_residual(), (2, 0, 1, 3)), want)
    layer.release()


# --------------------------------------------------------------------------- whole networks
@pytest.mark.parametrize("fmt", [0, 1, 2])
@pytest.mark.parametrize("h,b,c", [(5, 9, 64), (3, 70, 35), (2, 8, 130)])
def test_residual_from_reference(gpu, h, b, c, fmt):
    """Reference layout int32 [P][Q][PAD8(B)][PAD128(C)] -> engine layouts: against a host transpose, and back
    through the existing converter (whose oracle twin is pinned on the CPU)."""
    from tcbnn_amd import _lib
    from tcbnn_amd.device import DeviceBuffer
    if fmt == 2 and b % 2:
        b += 1  # the 12-bit layout wants an even batch
    r = rng(h * 100 + b + c + fmt)
    amp = 2047 if fmt == 2 else 30000
    res = r.integers(-amp, amp + 1, size=(h, h, b, c)).astype(np.int32)
    ref_host = orc.residual_to_reference(res)
    ref_host[:, :, b:, :] = 0x5A5A5A5A  # padding images / channels of a foreign buffer hold anything
    ref_host[:, :, :, c:] = 0x5A5A5A5A
    ref = gpuops.dev(ref_host)
    own = DeviceBuffer(_lib.lib.tcbnn_residual_bytes(h, h, c, b, fmt))
    own.fill(0xCD)
    gpuops.check(_lib.lib.tcbnn_residual_from_reference(ref.ptr, own.ptr, h, h, b, c, fmt, None))
    gpuops.sync()
    want = _residual_source(res, fmt)  # the engine layout by host transpose, channels past c zero
    if fmt == 2:  # (channels past c in the last group are zero on both sides)
        G = (c + 15) // 16
        words = lambda buf: buf.to_numpy(np.uint32, (h, h, G, 6 * b))
        np.testing.assert_array_equal(words(own), words(want))
    else:
        grp, dt = (8, np.int16) if fmt == 1 else (4, np.int32)
        shape = (h, h, (c + grp - 1) // grp, b, grp)
        np.testing.assert_array_equal(own.to_numpy(dt, shape), want.to_numpy(dt, shape))
    back = DeviceBuffer(ref_host.nbytes)
    gpuops.check(_lib.lib.tcbnn_residual_to_reference(own.ptr, back.ptr, h, h, b, c, fmt, None))
    gpuops.sync()
    np.testing.assert_array_equal(back.to_numpy(np.int32, ref_host.shape), orc.residual_to_reference(res))


@pytest.mark.parametrize("variant", ["popc", "mfma_f4"])
def test_reference_layout_between_layers(gpu, variant):
    """Every hand-over through device buffers in the reference's tile layouts (as if each neighbour were a layer
    of the reference): stem (saves a residual) -> conv (injects it, saves its own) -> stride-2 conv -> FC-ready
    conv (injects through the 2x2 max) -> FC -> output, against the oracle run on the plain tensors."""
    r = rng(77)
    b, h, ch, hid, classes = 12, 8, 64, 256, 10
    v = _variant(gpu, variant)
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    f0, f1, f2 = rm.pm1(r, (3, 3, 3, ch)), rm.pm1(r, (3, 3, ch, ch)), rm.pm1(r, (3, 3, ch, 2 * ch))
    f3 = rm.pm1(r, (3, 3, 2 * ch, 2 * ch))
    bn0 = r.normal(0, 5, ch).astype(np.float32)
    bn1, bn2 = r.normal(0, 24, ch).astype(np.float32), r.normal(0, 24, 2 * ch).astype(np.float32)
    bn3 = r.normal(0, 34, 2 * ch).astype(np.float32)
    feats = (h // 2) * (h // 2) * 2 * ch
    wfc, bnfc = rm.pm1(r, (feats, hid)), r.normal(0, 30, hid).astype(np.float32)
    wout, sc, bi = rm.pm1(r, (hid, classes)), r.normal(1, 0.1, classes).astype(np.float32), \
        r.normal(0, 1, classes).astype(np.float32)

    # oracle on plain tensors
    o0, r0 = orc.inconv128(x, f0, bn0, 1, True, 1, True)
    o1, r1 = orc.conv128(o0, orc.pack_conv_filter(f1), bn1, ch, ch, 3, 3, save_residual=True, inject_residual=True,
                         residual_channels=ch, res_in=r0)
    o2, _ = orc.conv128(o1, orc.pack_conv_filter(f2), bn2, ch, 2 * ch, 3, 3, stride=2)
    o3, _ = orc.conv128(o2, orc.pack_conv_filter(f3), bn3, 2 * ch, 2 * ch, 3, 3, ahead_fc=True, inject_residual=True,
                        residual_channels=ch, residual_pool=True, res_in=r1)
    o4 = orc.fc128(o3, orc.pack_fc_weight(wfc), bnfc, feats, hid)
    want = orc.out128(o4, orc.pack_fc_weight(wout), sc, bi, hid, classes)

    stem = gpu.InConv128LayerParam("Conv1", h, h, 3, 3, 3, ch, b, 1, 1, True, 1, 1, True)
    stem.initialize(x, gpu.ArrayWeights([f0, bn0]))
    stem.forward()
    t0, q0 = stem.get_output_gpu_reference_fmt(), stem.get_output_residual_gpu_reference()
    c1 = gpu.Conv128LayerParam("C1", h, h, 3, 3, ch, ch, b, 1, 1, True, 1, 1, False, True, True, ch, variant=v)
    c1.initialize(gpu.ArrayWeights([f1, bn1]), t0, q0)
    c1.set_input_gpu_reference_fmt(t0)
    c1.set_input_residual_gpu_reference(q0)
    c1.forward()
    t1, q1 = c1.get_output_gpu_reference_fmt(), c1.get_output_residual_gpu_reference()
    c2 = gpu.Conv128LayerParam("C2", h, h, 3, 3, ch, 2 * ch, b, 2, 2, variant=v)
    c2.initialize(gpu.ArrayWeights([f2, bn2]), t1)
    c2.set_input_gpu_reference_fmt(t1)
    c2.forward()
    t2 = c2.get_output_gpu_reference_fmt()
    c3 = gpu.Conv128LayerParam("C3", h // 2, h // 2, 3, 3, 2 * ch, 2 * ch, b, 1, 1, True, 1, 1, True, False, True, ch,
                               True, variant=v)
    c3.initialize(gpu.ArrayWeights([f3, bn3]), t2, q1)
    c3.set_input_gpu_reference_fmt(t2)
    c3.set_input_residual_gpu_reference(q1)
    c3.forward()
    t3 = c3.get_output_gpu_reference_fmt()
    fc = gpu.Fc128LayerParam("Fc1", b, feats, hid, variant=v)
    fc.initialize(gpu.ArrayWeights([wfc, bnfc]), t3)
    fc.set_input_gpu_reference_fmt(t3)
    fc.forward()
    t4 = fc.get_output_gpu_reference_fmt()
    out = gpu.Out128LayerParam("Fout", b, hid, classes, variant=v)
    out.initialize(gpu.ArrayWeights([wout, sc, bi]), t4)
    out.set_input_gpu_reference_fmt(t4)
    out.forward()
    gpuops.sync()

    words = lambda buf: buf.to_numpy(np.uint32, (buf.nbytes // 4,))
    np.testing.assert_array_equal(words(t0), orc.conv_to_fmt(o0, ch))
    np.testing.assert_array_equal(q0.to_numpy(np.int32, (h, h, orc.pad8(b), orc.pad128(ch))),
                                  orc.residual_to_reference(r0))
    np.testing.assert_array_equal(words(t1), orc.conv_to_fmt(o1, ch))
    np.testing.assert_array_equal(q1.to_numpy(np.int32, (h, h, orc.pad8(b), orc.pad128(ch))),
                                  orc.residual_to_reference(r1))
    np.testing.assert_array_equal(words(t2), orc.conv_to_fmt(o2, 2 * ch))
    np.testing.assert_array_equal(words(t3), orc.fc_to_fmt(o3, b, feats))
    np.testing.assert_array_equal(words(t4), orc.fc_to_fmt(o4, b, hid))
    got = out.download_output()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)  # fp32 logits: 1e-5 relative
    for layer in (stem, c1, c2, c3, fc, out):
        layer.release()


def _check_layers(net, spec, want):
    """Every layer's packed activations and saved residual (as stored: the full tensor, or its 2x2 maximum where
    only pooling readers exist) against the oracle; the names of the layers that store the maximum."""
    pooled_layers = []
    for L in spec:
        if L["kind"] in ("out", "avgfc"):
            continue
        layer, w = net.layers[L["name"]], want[L["name"]]
        got = layer.download_packed()
        np.testing.assert_array_equal(got, w["out"].reshape(got.shape), err_msg=L["name"])
        if w.get("res") is not None:
            got, pooled = layer.download_saved_residual()
            np.testing.assert_array_equal(got, _window_maximum(w["res"]) if pooled else w["res"], err_msg=L["name"])
            if pooled:
                pooled_layers.append(L["name"])
    return pooled_layers


def _compare_network(gpu, spec, seed, variant, residual_format=None):
    weights = gpu.synthetic_weights(spec, seed)
    x = gpu.synthetic_input(spec, seed)
    want = orc_nets.run(spec, weights, x)
    net = gpu.Network(spec, weights, x, variant=_variant(gpu, variant), residual_format=residual_format)
    net.forward()
    logits = net.logits()
    pooled_layers = []
    for L in spec:
        layer = net.layers[L["name"]]
        w = want[L["name"]]
        if L["kind"] == "out":
            np.testing.assert_allclose(logits, w["out"], rtol=1e-5, atol=0)
            np.testing.assert_array_equal(logits, w["out"])
        elif L["kind"] == "avgfc":  # fp32 head: 1e-5 of the logits' scale
            np.testing.assert_allclose(logits, w["out"], rtol=1e-5, atol=1e-5 * float(np.abs(w["out"]).max()))
        else:
            got = layer.download_packed()
            np.testing.assert_array_equal(got, w["out"].reshape(got.shape), err_msg=L["name"])
            if w.get("res") is not None:
                # (what the buffer holds: the full tensor, or its 2x2 maximum where only pooling readers exist)
                got, pooled = layer.download_saved_residual()
                np.testing.assert_array_equal(got, _window_maximum(w["res"]) if pooled else w["res"], err_msg=L["name"])
                if pooled:
                    pooled_layers.append(L["name"])
    # second forward on the same objects: identical logits (no stale-bit accumulation)
    net.forward()
    np.testing.assert_array_equal(net.logits(), logits)
    # the full tensors on request, and the same logits from the layers working with them
    for name in pooled_layers:
        np.testing.assert_array_equal(net.layers[name].download_residual(), want[name]["res"], err_msg=name)
    if pooled_layers:
        net.forward()
        np.testing.assert_array_equal(net.logits(), logits)
        assert not any(net.layers[name].download_saved_residual()[1] for name in pooled_layers)
    net.release()
    return logits


@pytest.mark.parametrize("variant", VARIANTS)
def test_mnist_mlp_full_batch(gpu, variant):
    from tcbnn_amd import nets
    _compare_network(gpu, nets.mnist_mlp_spec(batch=8192), 1, variant)


@pytest.mark.parametrize("variant", VARIANTS)
def test_cifar10_vgg(gpu, variant):
    from tcbnn_amd import nets
    _compare_network(gpu, nets.cifar10_vgg_spec(batch=16), 2, variant)


def test_cifar10_vgg_batch256(gpu):
    """cifar10_vgg.cu:162-199 at its configured batch of 256, every layer and image against the oracle."""
    from tcbnn_amd import nets
    _compare_network(gpu, nets.cifar10_vgg_spec(batch=256), 2, "mfma_f4")


def test_cifar10_vgg_batch256_presigned_input(gpu):
    """The same network on an input binarized by sign beforehand (+-1.0f): the first layer's sums are then exact
    small integers whatever the order of the additions, every layer is compared, and the first layer's bits
    are checked against the integer cross-correlation as well."""
    from tcbnn_amd import nets
    spec = nets.cifar10_vgg_spec(batch=256)
    weights = gpu.synthetic_weights(spec, 4)
    x = np.where(gpu.synthetic_input(spec, 4) >= 0, np.float32(1.0), np.float32(-1.0))
    want = orc_nets.run(spec, weights, x)
    net = gpu.Network(spec, weights, x)
    net.forward()
    np.testing.assert_allclose(net.logits(), want["Fout"]["out"], rtol=1e-5, atol=0)
    for L in spec[:-1]:
        got = net.layers[L["name"]].download_packed()
        np.testing.assert_array_equal(got, want[L["name"]]["out"].reshape(got.shape), err_msg=L["name"])
    first = spec[0]
    f, bn = weights[0], weights[1]  # weight-file order: the first layer's filter (HWIO) and thresholds
    sums = rm.xcorr_pm1(np.transpose(x[:4], (0, 2, 3, 1)), f, 1, 1, 1, 32, 32)  # [4][32][32][128]
    bits = orc.unpack_bits(net.layers[first["name"]].download_packed(), 128)[:, :, :4] > 0  # [32][32][4][128]
    np.testing.assert_array_equal(np.transpose(bits, (2, 0, 1, 3)), ~(sums.astype(np.float32) < bn))
    net.release()


@pytest.mark.parametrize("residual_format", [None, 0, 1], ids=["narrowest", "int32", "int16"])
@pytest.mark.parametrize("variant", VARIANTS)
def test_imagenet_resnet18(gpu, variant, residual_format):
    """Residuals in the narrowest exact format (for N(0,1) input: 12 bits for the first layer's and the first
    stage's tensors, whose bounds stay below 2048, and 16 bits from the second stage on: the test checks that this
    is what was chosen), all in 16 bits, and, as the reference stores them, in int32: same bits every way."""
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=8)
    if residual_format is None:
        net = gpu.Network(spec, gpu.synthetic_weights(spec, 3), gpu.synthetic_input(spec, 3))
        fmts = {L["name"]: net.layers[L["name"]].output_residual_gpu.format for L in spec if L.get("save_residual")}
        net.release()
        assert fmts and all(f == (2 if name in ("Conv1", "L1B1C2", "L1B2C2") else 1) for name, f in fmts.items()), fmts
    _compare_network(gpu, spec, 3, variant, residual_format)


@pytest.mark.parametrize("variant", VARIANTS)
def test_alexnet(gpu, variant):
    """alexnet.cu:143-177 at full image size: 11x11 stride-4 pooled first layer, 5x5 layer, 192 / 384
    channels (words that are only partly used), three FC layers."""
    from tcbnn_amd import nets
    _compare_network(gpu, nets.alexnet_spec(batch=8), 11, variant)


@pytest.mark.parametrize("variant", VARIANTS)
def test_cifar10_resnet(gpu, variant):
    """cifar10_resnet.cu:189-259 at full image size: 3x3 first layer with saved residual, pooled
    residuals at both stage entries."""
    from tcbnn_amd import nets
    _compare_network(gpu, nets.cifar10_resnet_spec(batch=16), 12, variant)


@pytest.mark.parametrize("variant", ["mfma_f4"])
def test_imagenet_vgg(gpu, variant):
    """imagenet_vgg.cu:217-286 (VGG-16) at full image size."""
    from tcbnn_amd import nets
    _compare_network(gpu, nets.imagenet_vgg_spec(batch=8), 13, variant)


@pytest.mark.parametrize("variant", VARIANTS)
def test_imagenet_resnet18_textbook_wiring(gpu, variant):
    """7x7/2 first layer + 3x3/2 max-pool, 1x1/2 shortcut convolutions, average-pool + fp32 FC head: no
    reference driver exists for this wiring, the CPU oracle (pinned against torch) is the only check."""
    from tcbnn_amd import nets
    _compare_network(gpu, nets.imagenet_resnet_textbook_spec(batch=8), 14, variant)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name,batch,seed", [("alexnet", 256, 21), ("cifar10_resnet", 256, 22),
                                             ("imagenet_resnet_textbook", 256, 23), ("imagenet_vgg", 64, 24)])
def test_other_networks_at_their_configured_batch(gpu, name, batch, seed):
    """alexnet.cu:143-177, cifar10_resnet.cu:189-259 and the textbook-wired ResNet-18 at batch 256, VGG-16
    (imagenet_vgg.cu:217-286) at batch 64, full image size, default engine: every layer and every image against the
    oracle.  Launch shapes that only occur at this size (grids sized to the whole machine, the pooling layer at
    112 x 112 x 64 x 256, the 1x1 stride-2 convolutions of the generic kernel) are only covered here."""
    from tcbnn_amd import nets
    spec = nets.SPECS[name](batch=batch)
    weights = gpu.synthetic_weights(spec, seed)
    x = gpu.synthetic_input(spec, seed)
    want = orc_nets.run(spec, weights, x)
    net = gpu.Network(spec, weights, x)
    net.forward()
    last = spec[-1]
    if last["kind"] == "avgfc":  # fp32 head: 1e-5 of the logits' scale
        w = want[last["name"]]["out"]
        np.testing.assert_allclose(net.logits(), w, rtol=1e-5, atol=1e-5 * float(np.abs(w).max()))
    else:
        np.testing.assert_allclose(net.logits(), want[last["name"]]["out"], rtol=1e-5, atol=0)
    _check_layers(net, spec, want)
    net.release()


def test_set_input_accepts_batches_of_the_same_distribution(gpu):
    """The residual formats are chosen from the first batch's window sums of |x|.  Later batches of the same
    distribution have slightly larger or smaller sums: they must be accepted (nothing would wrap) and give what
    the oracle gives; so must a batch scaled up as far as every tensor's format still holds; one step beyond
    that is refused."""
    from tcbnn_amd import nets
    from tcbnn_amd.layers import _residual_bound_limit
    spec = nets.imagenet_resnet_spec(batch=8, image=64, output_size=100)
    weights = gpu.synthetic_weights(spec, 40)
    net = gpu.Network(spec, weights, gpu.synthetic_input(spec, 40))
    first = net.order[0]
    bound0 = first.output_residual_gpu.bound
    fmts = {L["name"]: net.layers[L["name"]].output_residual_gpu.format for L in spec if L.get("save_residual")}
    larger = 0
    for seed in range(41, 49):
        x = gpu.synthetic_input(spec, seed)
        larger += first._residual_bound(x) > bound0
        net.set_input(x)
        net.forward()
        want = orc_nets.run(spec, weights, x)
        np.testing.assert_allclose(net.logits(), want["Fout"]["out"], rtol=1e-5, atol=0)
        _check_layers(net, spec, want)
    assert larger >= 1  # (some of these batches do exceed the first batch's exact bound)
    # as large as the formats allow: the limit is set by the 12-bit tensors of the first stage
    limit = _residual_bound_limit(first.output_residual_gpu)
    assert limit == 2047 - 2 * 64 * 9
    x = gpu.synthetic_input(spec, 50)
    x = (x * (0.98 * limit / first._residual_bound(x))).astype(np.float32)
    assert bound0 < first._residual_bound(x) <= limit
    net.set_input(x)
    net.forward()
    want = orc_nets.run(spec, weights, x)
    np.testing.assert_allclose(net.logits(), want["Fout"]["out"], rtol=1e-5, atol=0)
    _check_layers(net, spec, want)
    for L in spec:  # nothing was re-allocated, every recorded bound covers what the oracle saw
        if L.get("save_residual"):
            buf = net.layers[L["name"]].output_residual_gpu
            assert buf.format == fmts[L["name"]] and np.abs(want[L["name"]]["res"]).max() <= buf.bound
    with pytest.raises(gpu.TcbnnError):
        net.set_input((x * 1.1).astype(np.float32))
    net.release()


@pytest.mark.parametrize("fmt", [0, 1, 2])
@pytest.mark.parametrize("b,h,c,window,stride,pad", [(8, 12, 64, 3, 2, 1), (70, 7, 40, 3, 2, 1), (5, 9, 100, 2, 2, 0),
                                                     (3, 5, 33, 3, 1, 1)])
def test_pool128(gpu, b, h, c, window, stride, pad, fmt):
    """Overlapping OR / max pooling: bits and residual against the oracle, every residual format, odd shapes."""
    from tcbnn_amd import layers
    if fmt == 2 and b % 2:
        b += 1  # the 12-bit layout wants an even batch
    r = rng(b + h + c)
    x = rm.pm1(r, (b, h, h, c))
    amp = 2047 if fmt == 2 else 30000
    res = r.integers(-amp, amp + 1, size=(h, h, b, c)).astype(np.int32)
    inp = orc.pack_conv_input_nhwc(x)
    want_bits, want_res = orc.pool128(inp, c, window, stride, pad, res)
    layer = layers.Pool128LayerParam("p", h, h, c, b, window, stride, pad, pool_residual=True)
    layer.initialize(gpuops.pack_conv_input(x), _residual_source(res, fmt))
    layer.forward()
    gpuops.sync()
    np.testing.assert_array_equal(layer.download_packed(), want_bits)
    np.testing.assert_array_equal(layer.download_residual(), want_res)
    layer.release()


@pytest.mark.parametrize("fmt", [0, 1, 2])
@pytest.mark.parametrize("b,h,c,n", [(8, 7, 512, 1000), (70, 3, 100, 37), (33, 1, 64, 10)])
def test_avgpool_fc(gpu, b, h, c, n, fmt):
    from tcbnn_amd import layers
    if fmt == 2 and b % 2:
        b += 1  # the 12-bit layout wants an even batch
    r = rng(b + h + c + n)
    amp = 2047 if fmt == 2 else 20000
    res = r.integers(-amp, amp + 1, size=(h, h, b, c)).astype(np.int32)
    w = r.standard_normal((c, n)).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    want = orc.avgpool_fc(res, w, bias)
    layer = layers.AvgPoolFcLayerParam("head", h, h, c, b, n)
    layer.initialize(layers.ArrayWeights([w, bias]), _residual_source(res, fmt))
    layer.forward()
    gpuops.sync()
    got = layer.download_output()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * float(np.abs(want).max()))
    layer.release()


def test_forward_captured_in_a_hip_graph(gpu):
    """The whole forward (no allocation, no memset) is captured into a HIP graph and replayed several
    times, with eager work and synchronisations between the replays and a new input before the last
    one; every replay must reproduce the eager logits."""
    from tcbnn_amd import nets
    from tcbnn_amd.device import Graph, Stream
    spec = nets.imagenet_resnet_spec(batch=16, image=64, output_size=100)
    weights = gpu.synthetic_weights(spec, 21)
    # the second input stays inside the magnitude bound the residual formats were chosen for
    x0, x1 = gpu.synthetic_input(spec, 21), gpu.synthetic_input(spec, 22) * np.float32(0.9)
    net = gpu.Network(spec, weights, x0)
    stream = Stream()
    net.forward(stream)
    stream.synchronize()
    eager0 = net.logits().copy()
    graph = Graph(stream, net.forward)
    for _ in range(3):
        net.layers["Fout"].output_gpu.fill(0)  # eager work between the replays
        gpuops.sync()
        graph.launch()
        stream.synchronize()
        np.testing.assert_array_equal(net.logits(), eager0)
    net.set_input(x1)
    graph.launch()
    stream.synchronize()
    replay1 = net.logits().copy()
    net.forward(stream)
    stream.synchronize()
    np.testing.assert_array_equal(replay1, net.logits())
    assert not np.array_equal(replay1, eager0)
    want = orc_nets.run(spec, weights, x1)["Fout"]["out"]
    np.testing.assert_array_equal(replay1, want)
    net.release()


def test_two_networks_in_flight_on_two_streams(gpu):
    """Two copies of the network (own activations, residuals and inputs, same weights) run at the same time on two
    streams, batches dealt alternately: the persistent kernels of one copy share the GPU with those of the
    other.  Each copy's logits after several interleaved passes must equal its own solo result bit for bit."""
    from tcbnn_amd import nets
    from tcbnn_amd.device import Stream
    spec = nets.imagenet_resnet_spec(batch=64, image=96, output_size=200)
    weights = gpu.synthetic_weights(spec, 31)
    xs = [gpu.synthetic_input(spec, 31), gpu.synthetic_input(spec, 32)]
    copies = [gpu.Network(spec, weights, x) for x in xs]
    streams = [Stream(), Stream()]
    solo = []
    for net, st in zip(copies, streams):
        net.forward(st)
        st.synchronize()
        solo.append(net.logits().copy())
    assert not np.array_equal(solo[0], solo[1])
    for net in copies:
        net.layers["Fout"].output_gpu.fill(0)
    gpuops.sync()
    for k in range(10):  # no synchronisation inside: the two forwards overlap on the device
        copies[k % 2].forward(streams[k % 2])
    for st in streams:
        st.synchronize()
    for net, want in zip(copies, solo):
        np.testing.assert_array_equal(net.logits(), want)
    want0 = orc_nets.run(spec, weights, xs[0])["Fout"]["out"]
    np.testing.assert_allclose(solo[0], want0, rtol=1e-5, atol=0)
    for net in copies:
        net.release()


def test_imagenet_resnet18_batch256_every_image(gpu):
    """Full configured size on the default engine, every one of the 256 images and every layer against the
    oracle (packed activations and residuals bit for bit, logits to 1e-5 relative), three forward passes:
    kernels whose lanes, tiles or workgroups are only all in use at full batch are only covered here."""
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=256)
    weights = gpu.synthetic_weights(spec, 0)
    x = gpu.synthetic_input(spec, 0)
    want = orc_nets.run(spec, weights, x)
    net = gpu.Network(spec, weights, x)
    for _ in range(3):
        net.forward()
        logits = net.logits()
        np.testing.assert_allclose(logits, want["Fout"]["out"], rtol=1e-5, atol=0)
        pooled = _check_layers(net, spec, want)
        assert pooled == ["L1B2C2", "L2B2C2", "L3B2C2"]  # (the tensors that only the next stage's entry reads)
    # the full tensors on request, and the same logits from the layers working with them
    for name in pooled:
        np.testing.assert_array_equal(net.layers[name].download_residual(), want[name]["res"], err_msg=name)
    net.forward()
    np.testing.assert_array_equal(net.logits(), logits)
    assert _check_layers(net, spec, want) == []
    net.release()


def test_imagenet_resnet18_ragged_batch_above_256(gpu):
    """Batch 328 (five full groups of 64 images and a group of 8) at full image size, every image and every
    layer against the oracle: the last image group of each kernel is only partly filled, and element offsets
    go beyond the ones a batch of 256 reaches."""
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=328)
    weights = gpu.synthetic_weights(spec, 5)
    x = gpu.synthetic_input(spec, 5)
    want = orc_nets.run(spec, weights, x)
    net = gpu.Network(spec, weights, x)
    net.forward()
    np.testing.assert_allclose(net.logits(), want["Fout"]["out"], rtol=1e-5, atol=0)
    assert len(_check_layers(net, spec, want)) == 3
    net.release()


@pytest.mark.parametrize("variant", VARIANTS)
def test_imagenet_resnet18_batch256_properties(gpu, variant):
    """Full configured size: images are independent, so the first 8 images of a batch-256 run
    must reproduce the batch-8 run (which the oracle checks above) bit for bit."""
    from tcbnn_amd import nets
    spec256, spec8 = nets.imagenet_resnet_spec(batch=256), nets.imagenet_resnet_spec(batch=8)
    weights = gpu.synthetic_weights(spec256, 3)
    x = gpu.synthetic_input(spec256, 3)
    net = gpu.Network(spec256, weights, x, variant=_variant(gpu, variant))
    net.forward()
    big = net.logits()
    net.release()
    net8 = gpu.Network(spec8, weights, x[:8], variant=_variant(gpu, variant))
    net8.forward()
    small = net8.logits()
    net8.release()
    assert np.isfinite(big).all()
    np.testing.assert_array_equal(big[:8], small)
    want = orc_nets.run(spec8, weights, x[:8])["Fout"]["out"]
    np.testing.assert_allclose(small, want, rtol=1e-5, atol=0)
