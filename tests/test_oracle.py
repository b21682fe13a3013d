"""Pins the CPU oracle (oracle/tcbnn_oracle.cpp) against what the mathematics fixes.

The reference holds no golden vectors or stored fixtures for this path (its only checks are
run-time comparisons with cuBLAS / cuDNN and a CPU popcount loop), so each oracle function is
checked against an independent statement: integer matmul / library cross-correlation on
unpacked +-1 tensors, brute force, round trips and invariants.  The checks are chosen so that a
dropped term, a wrong sign, a transposed operand or a shifted window fails at least one of them.
"""
import numpy as np
import pytest

from oracle import orc
from tests import refmath as rm


def rng(seed):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ geometry (param.h:719-728)
def test_conv_geometry_closed_forms():
    worked = {(224, 4, 7): 3, (56, 1, 3): 1, (56, 2, 3): 1, (28, 2, 3): 1, (14, 2, 3): 1, (32, 1, 3): 1,
              (224, 4, 11): 5}
    for (h, s, r), pad in worked.items():
        assert orc.conv_geometry(h, r, s)[0] == pad
    for h in range(1, 65):
        for s in (1, 2, 4):
            for r in (1, 3, 5, 7, 11):
                for pool in (1, 2, 3):
                    pad, buf, out = orc.conv_geometry(h, r, s, True, pool)
                    assert (pad, buf, out) == rm.conv_pad_out(h, r, s, True, pool)
                    assert buf == -(-h // s) and out == -(-buf // pool)
                    if h % s == 0 and s == 1:
                        assert pad == (r - 1) // 2
                    if h >= r:
                        pad0, buf0, _ = orc.conv_geometry(h, r, s, False, 1)
                        assert pad0 == 0 and buf0 == (h - r) // s + 1


# ------------------------------------------------------------------ packing
@pytest.mark.parametrize("k", [1, 31, 32, 33, 100, 128, 784, 1000])
def test_pack_rows_is_msb_first_sign(k):
    x = rng(k).standard_normal((9, k)).astype(np.float32)
    x[0, 0] = 0.0  # zero counts as +1 (>= 0)
    x[1, -1] = -0.0
    got = orc.in128(x)
    assert got.shape == (9, orc.kw128(k))
    np.testing.assert_array_equal(got, rm.packbits_msb(x >= 0, orc.kw128(k)))
    assert (orc.unpack_bits(got, k) == np.where(x >= 0, 1, -1)).all()
    # explicit spot check of the bit position: element e -> bit 31-e of word e//32
    e = min(k - 1, 37)
    assert ((int(got[2, e // 32]) >> (31 - e % 32)) & 1) == int(x[2, e] >= 0)


def test_pack_fc_weight_is_column_major_bits():
    r = rng(1)
    w = r.standard_normal((200, 37)).astype(np.float32)  # [K][N]
    got = orc.pack_fc_weight(w)
    np.testing.assert_array_equal(got, rm.packbits_msb((w >= 0).T, orc.kw128(200)))


def test_pack_conv_filter_layout():
    r = rng(2)
    f = r.standard_normal((3, 2, 70, 5)).astype(np.float32)  # HWIO
    got = orc.pack_conv_filter(f)  # [O][RS][CW]
    want = rm.packbits_msb((f >= 0).transpose(3, 0, 1, 2).reshape(5, 6, 70), 3)
    np.testing.assert_array_equal(got, want)


# ------------------------------------------------------------------ bmm / fc / out
@pytest.mark.parametrize("m,n,k", [(8, 8, 128), (17, 40, 256), (64, 32, 1024), (3, 5, 32)])
def test_bmm_equals_integer_matmul(m, n, k):
    r = rng(m * n + k)
    a, b = rm.pm1(r, (m, k)), rm.pm1(r, (k, n))
    got = orc.bmm(orc.pack_rows(a), orc.pack_rows(b.T.copy()), k)
    np.testing.assert_array_equal(got, (a.astype(np.int64) @ b.astype(np.int64)).astype(np.int32))
    # a transposed operand would break this asymmetric check
    assert not np.array_equal(got, got.T) or m != n


@pytest.mark.parametrize("b,k,n", [(8, 128, 128), (13, 784, 100), (5, 100, 10), (32, 1024, 1024)])
def test_fc128_threshold_and_true_k(b, k, n):
    r = rng(b + k + n)
    x = r.standard_normal((b, k)).astype(np.float32)
    w = rm.pm1(r, (k, n))
    dots = (np.where(x >= 0, 1, -1).astype(np.int64) @ w.astype(np.int64))
    bn = r.normal(0, np.sqrt(k), n).astype(np.float32)
    bn[: min(n, 4)] = dots[0, : min(n, 4)]  # exact ties: >= must give bit 1
    out, acc = orc.fc128(orc.in128(x), orc.pack_fc_weight(w), bn, k, n, want_acc=True)
    # popcount accumulators: K - 2c is the +-1 dot product with the TRUE K (pad bits add 0)
    np.testing.assert_array_equal(k - 2 * acc, dots)
    want_bits = dots.astype(np.float32) >= bn[None, :]
    np.testing.assert_array_equal(out, rm.packbits_msb(want_bits, orc.kw128(n)))
    assert want_bits[0, : min(n, 4)].all()


def test_fc128_nan_threshold_gives_zero_bit():
    r = rng(5)
    x = r.standard_normal((8, 128)).astype(np.float32)
    w = rm.pm1(r, (128, 32))
    bn = np.full(32, np.nan, np.float32)
    assert not orc.fc128(orc.in128(x), orc.pack_fc_weight(w), bn, 128, 32).any()


@pytest.mark.parametrize("b,k,n", [(8, 1024, 10), (7, 512, 1000), (3, 100, 33)])
def test_out128_affine(b, k, n):
    r = rng(b * k + n)
    x = r.standard_normal((b, k)).astype(np.float32)
    w = rm.pm1(r, (k, n))
    scale = r.normal(1, 0.1, n).astype(np.float32)
    bias = r.normal(0, 1, n).astype(np.float32)
    got = orc.out128(orc.in128(x), orc.pack_fc_weight(w), scale, bias, k, n)
    dots = (np.where(x >= 0, 1, -1).astype(np.int64) @ w.astype(np.int64))
    want64 = dots.astype(np.float64) * scale.astype(np.float64) + bias.astype(np.float64)
    np.testing.assert_allclose(got, want64, rtol=1e-5, atol=1e-5)
    # separate fp32 multiply and add (no contraction): reproducible bit pattern
    want32 = (dots.astype(np.float32) * scale[None, :]).astype(np.float32) + bias[None, :]
    np.testing.assert_array_equal(got, want32.astype(np.float32))


# ------------------------------------------------------------------ bconv / conv128
def _rand_conv(r, b, h, w, cin, cout, R, S):
    x = rm.pm1(r, (b, h, w, cin))
    f = rm.pm1(r, (R, S, cin, cout))
    return x, f


@pytest.mark.parametrize("b,h,cin,cout,R,stride", [
    (2, 8, 128, 32, 3, 1), (3, 7, 64, 40, 3, 1), (2, 9, 32, 16, 3, 2), (1, 12, 160, 8, 5, 2),
    (2, 6, 96, 24, 1, 2), (1, 16, 64, 8, 7, 4), (2, 5, 256, 64, 3, 1)])
def test_bconv_equals_zero_padded_cross_correlation(b, h, cin, cout, R, stride):
    r = rng(h * cin + cout)
    x, f = _rand_conv(r, b, h, h, cin, cout, R, R)
    pad, buf, _ = orc.conv_geometry(h, R, stride)
    got = orc.bconv(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), cin, cout, R, R, stride, pad, buf, buf)
    want = rm.xcorr_pm1(x, f, stride, pad, pad, buf, buf)
    np.testing.assert_array_equal(got, want.astype(np.int32))


def test_bconv_brute_force_tiny():
    r = rng(11)
    b, h, w, cin, cout, R, S, stride, pad = 2, 4, 5, 40, 3, 3, 2, 1, 1
    x, f = _rand_conv(r, b, h, w, cin, cout, R, S)
    oh, ow = h, w
    want = np.zeros((b, oh, ow, cout), np.int32)
    for n in range(b):
        for y in range(oh):
            for xx in range(ow):
                for o in range(cout):
                    s_ = 0
                    for i in range(R):
                        for j in range(S):
                            ay, ax = y * stride - pad + i, xx * stride - pad + j
                            if 0 <= ay < h and 0 <= ax < w:
                                s_ += int(np.dot(x[n, ay, ax], f[i, j, :, o]))
                    want[n, y, xx, o] = s_
    inp = orc.pack_conv_input_nhwc(x)
    import ctypes  # rectangular filter: call through the generic entry
    out = np.empty((b, oh, ow, cout), np.int32)
    filt = orc.pack_conv_filter(f)
    orc._lib.orc_bconv(inp.ctypes.data, filt.ctypes.data, out.ctypes.data, b, h, w, cin, cout, R, S, stride,
                       stride, pad, pad, oh, ow)
    np.testing.assert_array_equal(out, want)


def _conv128_numpy(x, f, bn, stride, pool, res_in=None, residual_channels=0, residual_pool=False):
    """Independent statement of Conv128LayerFMT on unpacked tensors:
    res = xcorr (+ residual rule); bit = !(res < bn); pooled bit = max over window.
    The reference walks pool*output_height x pool*output_width pixels (kernel.cuh:685-690), not the
    pre-pool size: the zero-padded cross-correlation is therefore evaluated on that larger grid (a pixel
    past the convolution's own output sums the taps still inside the frame), and the windows are whole."""
    b, h, w, cin = x.shape
    R, S, _, cout = f.shape
    pad_h, ph, oh = rm.conv_pad_out(h, R, stride, True, pool)
    pad_w, pw, ow = rm.conv_pad_out(w, S, stride, True, pool)
    full = rm.xcorr_pm1(x, f, stride, pad_h, pad_w, pool * oh, pool * ow)  # [B][pool*oh][pool*ow][O]
    res = full[:, :ph, :pw, :].copy()
    if res_in is not None:
        assert pool == 1
        src = np.transpose(res_in, (2, 0, 1, 3)).astype(np.int64)  # [B][Hr][Wr][Cr]
        if residual_pool:
            src = rm.maxpool_nhwc(src.astype(np.float64), 2, 2).astype(np.int64)
        add = np.zeros_like(res)
        lim = min(residual_channels, src.shape[-1], cout)
        add[..., :lim] = src[:, :ph, :pw, :lim]
        res = res + add
        full = res
    bits = ~(full.astype(np.float32) < bn[None, None, None, :])
    pooled = rm.maxpool_nhwc(bits.astype(np.float64), pool, pool) > 0.5
    return res, pooled  # residual [B][ph][pw][O], bits [B][oh][ow][O]


@pytest.mark.parametrize("h,pool,stride,R", [(7, 2, 1, 3), (9, 3, 1, 3), (3, 2, 1, 3), (7, 4, 1, 3), (11, 2, 2, 3),
                                              (5, 2, 1, 5)])
def test_conv128_rounded_up_pool_walks_pool_times_output_pixels(h, pool, stride, R):
    """Brute force, straight from the reference's loop bounds: by in [0, pool*output_height), bx likewise
    (kernel.cuh:685-690, 703-711); per pixel the in-frame taps only, `exclude` for the others (l.720-757);
    res = Cin*R*S - exclude*Cin - 2*popc (l.766-768); bit ORed into (by/pool, bx/pool) (l.811-815).
    H=7 / pool 2 and H=9 / pool 3 have pooled sizes that are rounded up: their last windows hold pixels
    past the convolution's own 7 or 9 rows."""
    r = rng(1000 * h + 10 * pool + stride)
    b, cin, cout = 2, 64, 40
    x, f = _rand_conv(r, b, h, h, cin, cout, R, R)
    bn = r.normal(0, 6, cout).astype(np.float32)
    bn[:5] = [0.0, -0.0, 0.5, -1e-30, 1e-30]  # a pixel with no tap in the frame has res = 0: decided here
    pad, buf, oh = rm.conv_pad_out(h, R, stride, True, pool)
    assert oh * pool >= buf
    want = np.zeros((oh, oh, b, cout), bool)
    seen_past = False
    for by in range(pool * oh):
        for bx in range(pool * oh):
            ay0, ax0 = by * stride - pad, bx * stride - pad
            seen_past |= by >= buf or bx >= buf
            for n in range(b):
                for o in range(cout):
                    exclude, popc = 0, 0
                    for i in range(R):
                        for j in range(R):
                            ay, ax = ay0 + i, ax0 + j
                            if 0 <= ay < h and 0 <= ax < h:
                                popc += int(np.sum((x[n, ay, ax] >= 0) != (f[i, j, :, o] >= 0)))
                            else:
                                exclude += 1
                    res = cin * R * R - exclude * cin - 2 * popc
                    if not (np.float32(res) < bn[o]):
                        want[by // pool, bx // pool, n, o] = True
    assert seen_past == (buf % pool != 0)
    out, _ = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, cin, cout, R, R, stride,
                         True, pool)
    np.testing.assert_array_equal(out, rm.packbits_msb(want, orc.step32(cout)))


@pytest.mark.parametrize("h,pool,stride,R", [(7, 2, 1, 3), (9, 3, 1, 3), (13, 2, 4, 7), (6, 4, 1, 3)])
def test_inconv128_rounded_up_pool_walks_pool_times_output_pixels(h, pool, stride, R):
    """The same for the first layer (kernel.cuh:587-596, 604-643): pixels past the convolution's own output
    accumulate the in-frame taps in the reference's order, 0 when there is none.  Pre-signed +-1 inputs keep
    every sum an exact small integer, so the expected bits need no care about the order."""
    r = rng(77 * h + pool)
    b, cout = 2, 40
    f = rm.pm1(r, (R, R, 3, cout))
    x = rm.pm1(r, (b, 3, h, h))
    bn = np.round(r.normal(0, 4, cout)).astype(np.float32)
    bn[:5] = [0.0, -0.0, 0.5, -1e-30, 1e-30]
    pad, buf, oh = rm.conv_pad_out(h, R, stride, True, pool)
    want = np.zeros((oh, oh, b, cout), bool)
    for by in range(pool * oh):
        for bx in range(pool * oh):
            ay0, ax0 = by * stride - pad, bx * stride - pad
            for n in range(b):
                acc = np.zeros(cout, np.float32)
                for i in range(R):
                    for j in range(R):
                        ay, ax = ay0 + i, ax0 + j
                        if 0 <= ay < h and 0 <= ax < h:
                            t = [np.where(f[i, j, c] >= 0, x[n, c, ay, ax], -x[n, c, ay, ax]).astype(np.float32)
                                 for c in range(3)]
                            acc = (acc + ((t[0] + t[1]) + t[2])).astype(np.float32)
                want[by // pool, bx // pool, n] |= ~(acc < bn)
    out, _ = orc.inconv128(x, f, bn, stride, True, pool)
    np.testing.assert_array_equal(out, rm.packbits_msb(want, orc.step32(cout)))


@pytest.mark.parametrize("b,h,cin,cout,stride,pool", [
    (3, 8, 128, 64, 1, 1), (2, 8, 128, 128, 1, 2), (2, 7, 64, 96, 1, 2), (2, 12, 64, 128, 2, 1),
    (1, 9, 256, 32, 1, 3)])
def test_conv128_threshold_pool(b, h, cin, cout, stride, pool):
    r = rng(h + cin + cout + pool)
    x, f = _rand_conv(r, b, h, h, cin, cout, 3, 3)
    bn = r.normal(0, np.sqrt(9 * cin), cout).astype(np.float32)
    res, pooled = _conv128_numpy(x, f, bn, stride, pool)
    bn[:3] = res[0, 0, 0, :3]  # ties at a border pixel: !(res < bn) -> 1
    res, pooled = _conv128_numpy(x, f, bn, stride, pool)
    out, _ = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, cin, cout, 3, 3, stride,
                         True, pool)
    want = rm.packbits_msb(np.transpose(pooled, (1, 2, 0, 3)), orc.step32(cout))
    np.testing.assert_array_equal(out, want)


def test_conv128_ahead_fc_feature_order():
    r = rng(21)
    b, h, cin, cout = 3, 4, 64, 160  # cout not a multiple of 128: padded to 256 per pixel
    x, f = _rand_conv(r, b, h, h, cin, cout, 3, 3)
    bn = r.normal(0, 10, cout).astype(np.float32)
    _, pooled = _conv128_numpy(x, f, bn, 1, 2)
    out, _ = orc.conv128(orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f), bn, cin, cout, 3, 3, 1, True, 2,
                         ahead_fc=True)
    feat = np.zeros((b, 2, 2, 256), bool)
    feat[..., :cout] = pooled
    np.testing.assert_array_equal(out, rm.packbits_msb(feat.reshape(b, -1), 2 * 2 * 8))


def test_conv128_residual_rules():
    r = rng(31)
    b, h, cin, cout = 2, 6, 64, 96
    x, f = _rand_conv(r, b, h, h, cin, cout, 3, 3)
    bn = r.normal(0, 20, cout).astype(np.float32)
    inp, filt = orc.pack_conv_input_nhwc(x), orc.pack_conv_filter(f)
    base_out, base_res = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True)
    want_res, _ = _conv128_numpy(x, f, bn, 1, 1)
    np.testing.assert_array_equal(np.transpose(base_res, (2, 0, 1, 3)), want_res)

    # same-size source with fewer channels than the limit: channels past the source read 0
    src = r.integers(-300, 300, size=(h, h, b, 64)).astype(np.int32)
    out, res = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                           residual_channels=80, res_in=src)
    want_res, want_bits = _conv128_numpy(x, f, bn, 1, 1, src, 80)
    np.testing.assert_array_equal(np.transpose(res, (2, 0, 1, 3)), want_res)
    np.testing.assert_array_equal(out, rm.packbits_msb(np.transpose(want_bits, (1, 2, 0, 3)), 3))
    assert (res[..., 64:] == base_res[..., 64:]).all() and (res[..., :64] == base_res[..., :64] + src).all()

    # residual_channels = 0 is the same as no injection
    out0, res0 = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                             residual_channels=0, res_in=src)
    np.testing.assert_array_equal(out0, base_out)
    np.testing.assert_array_equal(res0, base_res)

    # 2x2 max pooling of a source twice the size; a constant field pools to itself
    src2 = r.integers(-300, 300, size=(2 * h, 2 * h, b, 96)).astype(np.int32)
    out, res = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                           residual_channels=48, residual_pool=True, res_in=src2)
    want_res, want_bits = _conv128_numpy(x, f, bn, 1, 1, src2, 48, True)
    np.testing.assert_array_equal(np.transpose(res, (2, 0, 1, 3)), want_res)
    np.testing.assert_array_equal(out, rm.packbits_msb(np.transpose(want_bits, (1, 2, 0, 3)), 3))
    const = np.full((2 * h, 2 * h, b, 96), 7, np.int32)
    _, resc = orc.conv128(inp, filt, bn, cin, cout, 3, 3, save_residual=True, inject_residual=True,
                          residual_channels=96, residual_pool=True, res_in=const)
    np.testing.assert_array_equal(resc, base_res + 7)


# ------------------------------------------------------------------ fp32 first layer
@pytest.mark.parametrize("h,R,stride,cout,pool", [(16, 3, 1, 64, 1), (20, 7, 4, 40, 1), (12, 3, 1, 32, 2),
                                                   (13, 5, 2, 96, 1)])
def test_inconv128_against_fp64_and_exact_integers(h, R, stride, cout, pool):
    import torch
    r = rng(h * R + cout)
    b = 3
    f = rm.pm1(r, (R, R, 3, cout))
    bn = r.normal(0, np.sqrt(3 * R * R), cout).astype(np.float32)
    pad, ph, oh = rm.conv_pad_out(h, R, stride, True, pool)

    # (1) pre-signed +-1.0 input: every partial sum is a small integer, so the result is
    # order-free and must be exact.
    xs = rm.pm1(r, (b, 3, h, h))
    # evaluated on the pool*output grid the reference walks (kernel.cuh:587-596)
    full = rm.xcorr_pm1(np.transpose(xs, (0, 2, 3, 1)), f, stride, pad, pad, pool * oh, pool * oh)
    want = full[:, :ph, :ph, :]  # [B][ph][pw][O]
    bn_i = np.round(bn).astype(np.float32)
    bn_i[:4] = want[0, 0, 0, :4]  # ties
    out, res = orc.inconv128(xs, f, bn_i, stride, True, pool, save_residual=(pool == 1))
    bits = ~(full.astype(np.float32) < bn_i[None, None, None, :])
    pooled = rm.maxpool_nhwc(bits.astype(np.float64), pool, pool) > 0.5
    np.testing.assert_array_equal(out, rm.packbits_msb(np.transpose(pooled, (1, 2, 0, 3)), orc.step32(cout)))
    if pool == 1:
        np.testing.assert_array_equal(np.transpose(res, (2, 0, 1, 3)), want)

    # (2) N(0,1) input: compare with an fp64 convolution away from threshold ties
    x = r.standard_normal((b, 3, h, h)).astype(np.float32)
    xt = torch.from_numpy(x).double()
    ft = torch.from_numpy(f).double().permute(3, 2, 0, 1)
    need = (ph - 1) * stride + R
    xp = torch.nn.functional.pad(xt, (pad, max(0, need - h - pad), pad, max(0, need - h - pad)))
    y = torch.nn.functional.conv2d(xp, ft, stride=stride)[:, :, :ph, :ph].permute(0, 2, 3, 1).numpy()
    absum = torch.nn.functional.conv2d(xp.abs(), torch.ones_like(ft), stride=stride)[:, :, :ph, :ph] \
        .permute(0, 2, 3, 1).numpy()
    out, res = orc.inconv128(x, f, bn, stride, True, 1, save_residual=True)
    got_bits = orc.unpack_bits(out, cout) > 0  # [ph][pw][B][O]
    got_bits = np.transpose(got_bits, (2, 0, 1, 3))
    safe = np.abs(y - bn[None, None, None, :]) > 1e-4 * absum
    assert safe.mean() > 0.99
    np.testing.assert_array_equal(got_bits[safe], (y >= bn[None, None, None, :])[safe])
    # residual = truncation toward zero of the fp32 sum
    res_b = np.transpose(res, (2, 0, 1, 3))
    safe_i = np.abs(y - np.round(y)) > 1e-3
    np.testing.assert_array_equal(res_b[safe_i], np.trunc(y)[safe_i].astype(np.int32))


def test_inconv128_add_order_is_the_reference_order():
    """acc += ((+-f0)+(+-f1))+(+-f2) per tap, taps in raster order: replay in numpy float32."""
    r = rng(77)
    h, R, cout = 6, 3, 32
    x = (r.standard_normal((1, 3, h, h)) * 1000).astype(np.float32)
    f = rm.pm1(r, (R, R, 3, cout))
    out, res = orc.inconv128(x, f, np.zeros(cout, np.float32), 1, True, 1, save_residual=True)
    y0, x0 = 2, 3
    acc = np.zeros(cout, np.float32)
    for i in range(R):
        for j in range(R):
            ay, ax = y0 - 1 + i, x0 - 1 + j
            t = [np.where(f[i, j, c] >= 0, x[0, c, ay, ax], -x[0, c, ay, ax]).astype(np.float32) for c in range(3)]
            acc = (acc + ((t[0] + t[1]).astype(np.float32) + t[2]).astype(np.float32)).astype(np.float32)
    np.testing.assert_array_equal(res[y0, x0, 0], np.trunc(acc).astype(np.int32))
    np.testing.assert_array_equal(orc.unpack_bits(out, cout)[y0, x0, 0] > 0, acc >= 0)


# ------------------------------------------------------------------ reference FMT layouts
@pytest.mark.parametrize("b,k", [(8, 128), (13, 300), (16, 1024)])
def test_fc_fmt_round_trip_through_reference_unpack(b, k):
    x = rng(b + k).standard_normal((b, k)).astype(np.float32)
    fmt = orc.fc_to_fmt(orc.in128(x), b, k)
    np.testing.assert_array_equal(rm.unpack_fc_fmt(fmt, b, k), np.where(x >= 0, 1.0, -1.0))
    # kernel.cuh:170: block (bx, by) word warpid=r*4+w  ->  (bx*gdy+by)*32 + warpid
    assert fmt[(0 * orc.step128(k) + 0) * 32 + 1 * 4 + 2] == orc.in128(x)[1, 2]


@pytest.mark.parametrize("b,h,w,c", [(8, 3, 2, 128), (5, 2, 3, 64), (9, 2, 2, 320)])
def test_conv_fmt_round_trip_through_reference_unpack(b, h, w, c):
    x = rng(b + c).standard_normal((b, h, w, c)).astype(np.float32)
    fmt = orc.conv_to_fmt(orc.pack_conv_input_nhwc(x), c)
    np.testing.assert_array_equal(rm.unpack_conv_fmt(fmt, h, w, c, b), np.where(x >= 0, 1.0, -1.0))


def test_weight_and_filter_fmt_match_reference_tile_addressing():
    r = rng(9)
    k, n = 300, 20
    w = r.standard_normal((k, n)).astype(np.float32)
    fmt = orc.fc_weight_to_fmt(orc.pack_fc_weight(w), k, n)
    gdk = orc.step128(k)
    # Fc128LayerFMT loads the 8x128 tile of neurons by*8.. and chunk i at by*8*gdk*4 + i*32,
    # row j of the tile = words j*4..j*4+3 (kernel.cuh:200)
    for nn in (0, 7, 8, 19):
        for kk in (0, 127, 128, 299):
            word = fmt[(nn // 8) * 8 * gdk * 4 + (kk // 128) * 32 + (nn % 8) * 4 + (kk % 128) // 32]
            assert ((int(word) >> (31 - kk % 32)) & 1) == int(w[kk, nn] >= 0)
    R, S, c, o = 3, 3, 192, 40
    f = r.standard_normal((R, S, c, o)).astype(np.float32)
    ffmt = orc.conv_filter_to_fmt(orc.pack_conv_filter(f), R, S, c, o)
    ins, ots = orc.step128(c), orc.step32(o)
    # Conv128LayerFMT: tile of out-channels bo*32+8t.. at (r*S+s)*ots*32*ins*4 + (bo*32+8t)*ins*4 + c*32
    for (t, oc, ch) in ((0, 0, 0), (4, 39, 191), (8, 9, 130), (2, 33, 64)):
        base = t * ots * 32 * ins * 4 + (oc // 8) * 8 * ins * 4 + (ch // 128) * 32
        word = ffmt[base + (oc % 8) * 4 + (ch % 128) // 32]
        assert ((int(word) >> (31 - ch % 32)) & 1) == int(f[t // S, t % S, ch, oc] >= 0)


def test_residual_reference_layout():
    res = rng(4).integers(-9, 9, size=(2, 3, 5, 64)).astype(np.int32)
    ref = orc.residual_to_reference(res)
    assert ref.shape == (2, 3, 8, 128)
    np.testing.assert_array_equal(ref[:, :, :5, :64], res)
    assert not ref[:, :, 5:, :].any() and not ref[..., 64:].any()


# --------------------------------------------------------------------------- layers of the textbook wiring
@pytest.mark.parametrize("b,h,c,window,stride,pad", [(3, 11, 40, 3, 2, 1), (2, 8, 64, 3, 2, 1), (4, 9, 33, 2, 2, 0),
                                                     (1, 5, 96, 3, 1, 1)])
def test_pool128_is_max_pool_of_values_and_of_the_residual(b, h, c, window, stride, pad):
    """OR of sign bits == sign of the maximum of the +-1 values; residual == integer max-pool
    (torch.nn.functional.max_pool2d pads with -inf, i.e. ignores taps outside the frame)."""
    import torch
    r = np.random.default_rng(b + h + c)
    x = rm.pm1(r, (b, h, h, c))
    res = r.integers(-30000, 30000, size=(h, h, b, c)).astype(np.int32)
    out, pooled = orc.pool128(orc.pack_conv_input_nhwc(x), c, window, stride, pad, res)
    want = torch.nn.functional.max_pool2d(torch.tensor(x).permute(0, 3, 1, 2), window, stride, pad)
    np.testing.assert_array_equal(orc.unpack_bits(out, c), want.permute(2, 3, 0, 1).numpy())
    want_res = torch.nn.functional.max_pool2d(torch.tensor(res.astype(np.float64)).permute(2, 3, 0, 1), window, stride, pad)
    np.testing.assert_array_equal(pooled, want_res.permute(2, 3, 0, 1).numpy().astype(np.int32))
    # thresholding commutes with the maximum: pooling the bits of (res >= t) equals the bit of the pooled residual
    t = 123
    bits = (res >= t).astype(np.float32) * 2 - 1  # [H][W][B][C] -> NHWC
    out2, _ = orc.pool128(orc.pack_conv_input_nhwc(np.ascontiguousarray(bits.transpose(2, 0, 1, 3))), c, window, stride, pad)
    np.testing.assert_array_equal(orc.unpack_bits(out2, c) > 0, pooled >= t)


@pytest.mark.parametrize("b,h,c,n", [(3, 7, 512, 10), (5, 2, 40, 7), (2, 1, 64, 3)])
def test_avgpool_fc_against_fp64(b, h, c, n):
    r = np.random.default_rng(b + h + c + n)
    res = r.integers(-20000, 20000, size=(h, h, b, c)).astype(np.int32)
    w = r.standard_normal((c, n)).astype(np.float32)
    bias = r.standard_normal(n).astype(np.float32)
    got = orc.avgpool_fc(res, w, bias)
    want = res.astype(np.float64).mean(axis=(0, 1)) @ w.astype(np.float64) + bias
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    # a constant residual averages to itself exactly
    const = np.full((h, h, b, c), 7, np.int32)
    one = orc.avgpool_fc(const, np.ones((c, 1), np.float32), np.zeros(1, np.float32))
    np.testing.assert_array_equal(one, np.full((b, 1), 7.0 * c, np.float32))
