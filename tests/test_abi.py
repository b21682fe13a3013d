"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares; host-only entry points (geometry, sizes, error reporting) behave."""
import os
import re

import pytest

from tests import refmath as rm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    txt = open(os.path.join(ROOT, "include", "tcbnn_hip.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(tcbnn_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    from tcbnn_amd import _lib
    syms = _declared_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(_lib.lib, s), "libtcbnn_hip.so does not export %s" % s
    assert sorted(_lib.ABI) == syms, "Python binding table and header disagree"
    assert _lib.lib.tcbnn_abi_version() == 7
    # the build entry point refuses a library of another ABI version: it must expect this one
    import inspect
    import __graft_entry__
    assert "tcbnn_abi_version() == 7" in inspect.getsource(__graft_entry__.build)


def test_geometry_entry_points_match_reference_formulas():
    from tcbnn_amd import _lib
    for h in range(1, 40):
        for s in (1, 2, 4):
            for r in (1, 3, 7, 11):
                for pool in (1, 2):
                    pad, buf, out = rm.conv_pad_out(h, r, s, True, pool)
                    assert _lib.lib.tcbnn_conv_pad(h, r, s, 1) == pad
                    assert _lib.lib.tcbnn_conv_out(h, r, s, 1, pool) == out
                    assert _lib.lib.tcbnn_conv_pad(h, r, s, 0) == 0


def test_size_helpers():
    from tcbnn_amd import _lib
    L = _lib.lib
    assert L.tcbnn_fc_act_words(8192, 784) == 8192 * 28
    assert L.tcbnn_conv_act_words(56, 56, 256, 64) == 56 * 56 * 256 * 2
    assert L.tcbnn_fc_weight_words(784, 10) == 32 * 28 + 32 * 8 * 4  # sign-bit rows + the copy in lane order
    assert L.tcbnn_conv_filter_words(3, 3, 64, 64) == 64 * 9 * 2 * 2   # sign bits + a copy in MFMA lane order
    assert L.tcbnn_conv_filter_words(3, 3, 96, 64) == 64 * 9 * 3       # sign bits only
    assert L.tcbnn_conv_filter_words(5, 5, 64, 40) == 64 * 25 * 2
    assert L.tcbnn_inconv_filter_words(7, 7, 3, 64) == 49 * 64 * 5
    # packed first-layer input: (P - 1) stride + R rows and columns of [batch][3]
    assert L.tcbnn_inconv_packed_input_floats(256, 224, 224, 7, 7, 4, 4, 1) == 227 * 227 * 256 * 3
    assert L.tcbnn_inconv_packed_input_floats(5, 32, 30, 3, 5, 1, 2, 1) == 34 * 33 * 5 * 3
    assert L.tcbnn_inconv_packed_input_floats(5, 16, 16, 3, 3, 2, 2, 0) == 15 * 15 * 5 * 3  # the last row is unused
    assert L.tcbnn_inconv_packed_input_floats(0, 16, 16, 3, 3, 1, 1, 1) == 0
    assert L.tcbnn_inconv_packed_input_floats(4, 2, 16, 3, 3, 1, 1, 0) == 0   # no output row


def test_errors_are_codes_not_exits():
    from tcbnn_amd import _lib
    L = _lib.lib
    assert L.tcbnn_fc128_forward(None, None) == -2
    assert b"NULL" in L.tcbnn_last_error()
    d = _lib.Fc128Desc(1, 1, 1, 1, 0, 128, 128, 0, None, 0)  # batch 0; never launches
    assert L.tcbnn_fc128_forward(d, None) == -1
    assert L.tcbnn_bmm(1, 1, 1, 8, 8, 100, 1, None) == -1  # K not a multiple of 32
    assert L.tcbnn_set_default_variant(99) == -1
    assert L.tcbnn_inconv_pack_input(None, None, 4, 8, 8, 3, 3, 1, 1, 1, None) == -2
    assert L.tcbnn_inconv_pack_input(1, 1, 0, 8, 8, 3, 3, 1, 1, 1, None) == -1  # batch 0; never launches
    with pytest.raises(_lib.TcbnnError):
        _lib.check(-1)


def test_network_specs_match_reference_wiring():
    from tcbnn_amd import nets
    spec = nets.imagenet_resnet_spec(batch=256)
    assert len(spec) == 19
    by = {L["name"]: L for L in spec}
    assert by["Conv1"]["stride"] == 4 and by["Conv1"]["save_residual"]
    assert by["L2B1C2"]["residual_pool"] and by["L2B1C2"]["res_src"] == "L1B2C2"
    assert by["L3B1C2"]["residual_channels"] == 128 and by["L4B1C2"]["residual_channels"] == 256
    assert by["L1B2C2"]["residual_channels"] == 128 and by["L4B2C2"]["ahead_fc"]
    assert by["Fc1"]["inp"] == 7 * 7 * 512
    bops, flops = nets.binary_ops(spec)
    assert abs(bops / 256 / 1e9 - 3.379) < 0.01  # binary ops per image
    assert abs(flops / 1e9 - 15.1) < 0.1
    bops, _ = nets.binary_ops(nets.mnist_mlp_spec(8192))
    assert abs(bops / 1e9 - 47.68) < 0.05
    bops, _ = nets.binary_ops(nets.cifar10_vgg_spec(256))
    assert abs(bops / 1e9 - 314.1) < 0.5


def test_residual_formats_sizes_and_choice():
    """Host-only helpers of the residual storage formats: bytes per tensor, and the narrowest format a bound allows
    (12 bits need an even batch: the format's 128-bit accesses are aligned only then)."""
    from tcbnn_amd import _lib
    L = _lib.lib
    h, w, c, b = 5, 7, 64, 6
    assert L.tcbnn_residual_bytes(h, w, c, b, _lib.RES_I32) == h * w * c * b * 4
    assert L.tcbnn_residual_bytes(h, w, c, b, _lib.RES_I16) == h * w * c * b * 2
    assert L.tcbnn_residual_bytes(h, w, c, b, _lib.RES_I12) == h * w * c * b * 3 // 2
    # channels are stored in whole groups: 4 (int32), 8 (int16) or 16 (12 bits)
    assert L.tcbnn_residual_bytes(1, 1, 17, 2, _lib.RES_I32) == 20 * 2 * 4
    assert L.tcbnn_residual_bytes(1, 1, 17, 2, _lib.RES_I16) == 24 * 2 * 2
    assert L.tcbnn_residual_bytes(1, 1, 17, 2, _lib.RES_I12) == 32 * 2 * 3 // 2
    for bound, batch, want in ((0, 2, _lib.RES_I12), (2047, 256, _lib.RES_I12), (2048, 256, _lib.RES_I16),
                               (2047, 255, _lib.RES_I16), (32767, 8, _lib.RES_I16), (32768, 8, _lib.RES_I32),
                               (-1, 8, _lib.RES_I32), (2 ** 31 - 1, 8, _lib.RES_I32)):
        assert L.tcbnn_residual_format_narrowest(bound, batch) == want, (bound, batch)
    assert L.tcbnn_residual_format_for_bound(2047) == _lib.RES_I16  # (never 12 bits: it does not know the batch)
    assert L.tcbnn_conv_residual_bound(64, 3, 3, 155) == 155 + 576
    assert L.tcbnn_conv_residual_bound(64, 3, 3, 0) == 576


def test_first_layer_bound_of_input_is_the_largest_window_sum():
    """tcbnn_inconv_residual_bound_of_input against a brute-force window walk in numpy: no first-layer sum can
    exceed the largest sum of |x| over one filter window (all three channels), and the returned bound lies between
    that sum and that sum * 1.001 + 2."""
    import ctypes as C

    import numpy as np
    from tcbnn_amd import _lib
    L = _lib.lib
    rng = np.random.default_rng(11)
    for (b, h, w, r, s, sh, sw, padding) in ((2, 9, 11, 3, 3, 1, 1, 1), (3, 16, 13, 7, 7, 4, 4, 1), (1, 12, 12, 5, 3, 2, 1, 0),
                                             (2, 23, 19, 11, 11, 4, 4, 1), (1, 7, 7, 7, 7, 1, 1, 1)):
        x = (rng.standard_normal((b, 3, h, w)) * rng.uniform(0.1, 30)).astype(np.float32)
        pad_h, pad_w = L.tcbnn_conv_pad(h, r, sh, padding), L.tcbnn_conv_pad(w, s, sw, padding)
        oh, ow = L.tcbnn_conv_out(h, r, sh, padding, 1), L.tcbnn_conv_out(w, s, sw, padding, 1)
        a = np.abs(x.astype(np.float64)).sum(axis=1)
        worst = 0.0
        for y in range(oh):
            for xx in range(ow):
                y0, x0 = y * sh - pad_h, xx * sw - pad_w
                win = a[:, max(0, y0):min(h, y0 + r), max(0, x0):min(w, x0 + s)]
                worst = max(worst, float(win.sum(axis=(1, 2)).max()))
        got = L.tcbnn_inconv_residual_bound_of_input(x.ctypes.data_as(C.c_void_p), b, h, w, r, s, sh, sw, padding)
        assert worst <= got <= worst * 1.001 + 2, (got, worst)
        # and it is a bound: the largest |sum| any +-1 filter can reach is that window's sum of |x|
        assert got >= np.floor(worst)
    bad = np.ones((1, 3, 8, 8), np.float32)
    bad[0, 1, 3, 3] = np.nan
    assert L.tcbnn_inconv_residual_bound_of_input(bad.ctypes.data_as(C.c_void_p), 1, 8, 8, 3, 3, 1, 1, 1) == 2 ** 31 - 1
    assert L.tcbnn_inconv_residual_bound_of_input(None, 1, 8, 8, 3, 3, 1, 1, 1) == 2 ** 31 - 1


def test_host_abs_max_and_threaded_window_scan_on_a_large_batch():
    """tcbnn_host_abs_max against numpy (sizes below and above its threading threshold, NaN / infinity), and the
    window scan on a batch large enough for every host thread to take several images."""
    import numpy as np
    from tcbnn_amd import _lib
    L = _lib.lib
    rng = np.random.default_rng(12)
    for n in (1, 1000, (3 << 20) + 17):
        x = (rng.standard_normal(n) * 7).astype(np.float32)
        assert L.tcbnn_host_abs_max(x.ctypes.data, n) == float(np.abs(x).max())
        x[n // 2] = np.inf if n % 2 else np.nan
        assert L.tcbnn_host_abs_max(x.ctypes.data, n) == float("inf")
    assert L.tcbnn_host_abs_max(None, 5) == 0.0
    b, h, w = 70, 20, 24
    x = rng.standard_normal((b, 3, h, w)).astype(np.float32)
    x[41] *= 9.0  # the image that sets the bound sits in the middle of the batch
    a = np.abs(x.astype(np.float64)).sum(axis=1)
    worst = max(float(a[:, max(0, 4 * y - 3):4 * y + 4, max(0, 4 * q - 3):4 * q + 4].sum(axis=(1, 2)).max())
                for y in range(5) for q in range(6))
    got = L.tcbnn_inconv_residual_bound_of_input(x.ctypes.data, b, h, w, 7, 7, 4, 4, 1)
    assert worst <= got <= worst * 1.001 + 2, (got, worst)
