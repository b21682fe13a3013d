"""TEST INFRASTRUCTURE — ctypes/numpy front end of the CPU oracle (oracle/tcbnn_oracle.cpp).

Never imported by the product package.  Arrays are numpy, layouts are the oracle's logical
layouts (see the header of tcbnn_oracle.cpp)."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libtcbnn_oracle.so")


def build(force=False):
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = C.CDLL(build())
_vp, _i = C.c_void_p, C.c_int


def _sig(name, args, res=None):
    fn = getattr(_lib, name)
    fn.argtypes, fn.restype = args, res
    return fn


_sig("orc_num_threads", [], _i)
_sig("orc_conv_geometry", [_i] * 5 + [C.POINTER(_i)] * 3)
_sig("orc_pack_rows", [_vp, _vp, C.c_long, _i, C.c_long, _i])
_sig("orc_in128", [_vp, _vp, _i, _i])
_sig("orc_pack_fc_weight", [_vp, _vp, _i, _i])
_sig("orc_pack_conv_filter", [_vp, _vp] + [_i] * 4)
_sig("orc_pack_conv_input_nhwc", [_vp, _vp] + [_i] * 4)
_sig("orc_bmm", [_vp] * 3 + [_i] * 3)
_sig("orc_fc128", [_vp] * 5 + [_i] * 3)
_sig("orc_out128", [_vp] * 5 + [_i] * 3)
_sig("orc_bconv", [_vp] * 3 + [_i] * 13)
_sig("orc_conv128", [_vp] * 6 + [_i] * 17)
_sig("orc_inconv128", [_vp] * 5 + [_i] * 11)
_sig("orc_fc_to_fmt", [_vp, _vp, _i, _i])
_sig("orc_conv_to_fmt", [_vp, _vp] + [_i] * 4)
_sig("orc_fc_weight_to_fmt", [_vp, _vp, _i, _i])
_sig("orc_conv_filter_to_fmt", [_vp, _vp] + [_i] * 4)
_sig("orc_residual_to_reference", [_vp, _vp] + [_i] * 4)
_sig("orc_pool128", [_vp] * 4 + [_i] * 7)
_sig("orc_avgpool_fc", [_vp] * 4 + [_i] * 5)


def step32(x):
    return (x + 31) >> 5


def step128(x):
    return (x + 127) >> 7


def pad8(x):
    return ((x + 7) >> 3) << 3


def pad128(x):
    return step128(x) << 7


def kw128(k):
    return 4 * step128(k)


def _p(a):
    return a.ctypes.data if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def num_threads():
    return _lib.orc_num_threads()


def conv_geometry(in_size, filt, stride, padding=True, pool=1):
    pad, buf, out = _i(), _i(), _i()
    _lib.orc_conv_geometry(in_size, filt, stride, int(padding), pool, C.byref(pad), C.byref(buf), C.byref(out))
    return pad.value, buf.value, out.value


def pack_rows(x, kwords=None):
    x = _f32(x)
    rows, k = x.shape
    kwords = kwords or step32(k)
    out = np.empty((rows, kwords), np.uint32)
    _lib.orc_pack_rows(_p(x), _p(out), rows, k, k, kwords)
    return out


def in128(x):
    x = _f32(x)
    b, k = x.shape
    out = np.empty((b, kw128(k)), np.uint32)
    _lib.orc_in128(_p(x), _p(out), b, k)
    return out


def pack_fc_weight(w_kn):
    w = _f32(w_kn)
    k, n = w.shape
    out = np.empty((n, kw128(k)), np.uint32)
    _lib.orc_pack_fc_weight(_p(w), _p(out), k, n)
    return out


def pack_conv_filter(hwio):
    f = _f32(hwio)
    r, s, c, o = f.shape
    out = np.empty((o, r * s, step32(c)), np.uint32)
    _lib.orc_pack_conv_filter(_p(f), _p(out), r, s, c, o)
    return out


def pack_conv_input_nhwc(x):
    x = _f32(x)
    b, h, w, c = x.shape
    out = np.empty((h, w, b, step32(c)), np.uint32)
    _lib.orc_pack_conv_input_nhwc(_p(x), _p(out), b, h, w, c)
    return out


def bmm(a, b, k):
    a, b = _u32(a), _u32(b)
    m, n = a.shape[0], b.shape[0]
    c = np.empty((m, n), np.int32)
    _lib.orc_bmm(_p(a), _p(b), _p(c), m, n, k)
    return c


def fc128(inp, w, bn, k, n, want_acc=False):
    inp, w, bn = _u32(inp), _u32(w), _f32(bn)
    b = inp.shape[0]
    out = np.empty((b, kw128(n)), np.uint32)
    acc = np.empty((b, n), np.int32) if want_acc else None
    _lib.orc_fc128(_p(inp), _p(w), _p(bn), _p(out), _p(acc), b, k, n)
    return (out, acc) if want_acc else out


def out128(inp, w, scale, bias, k, n):
    inp, w, scale, bias = _u32(inp), _u32(w), _f32(scale), _f32(bias)
    b = inp.shape[0]
    out = np.empty((b, n), np.float32)
    _lib.orc_out128(_p(inp), _p(w), _p(scale), _p(bias), _p(out), b, k, n)
    return out


def bconv(inp, filt, cin, cout, r, s, stride, pad, oh, ow):
    inp, filt = _u32(inp), _u32(filt)
    h, w, b, _ = inp.shape
    out = np.empty((b, oh, ow, cout), np.int32)
    _lib.orc_bconv(_p(inp), _p(filt), _p(out), b, h, w, cin, cout, r, s, stride, stride, pad, pad, oh, ow)
    return out


def conv128(inp, filt, bn, cin, cout, r, s, stride=1, padding=True, pool=1, ahead_fc=False,
            save_residual=False, inject_residual=False, residual_channels=0, residual_pool=False,
            res_in=None):
    """Returns (packed output, saved residual or None)."""
    inp, filt, bn = _u32(inp), _u32(filt), _f32(bn)
    h, w, b, _ = inp.shape
    _, ph, oh = conv_geometry(h, r, stride, padding, pool)
    _, pw, ow = conv_geometry(w, s, stride, padding, pool)
    if ahead_fc:
        out = np.empty((b, oh * ow * kw128(cout)), np.uint32)
    else:
        out = np.empty((oh, ow, b, step32(cout)), np.uint32)
    res_out = np.zeros((ph, pw, b, cout), np.int32) if save_residual else None
    res_in_ch = 0
    if inject_residual:
        res_in = np.ascontiguousarray(res_in, dtype=np.int32)
        res_in_ch = res_in.shape[-1]
    _lib.orc_conv128(_p(inp), _p(filt), _p(bn), _p(out), _p(res_in) if inject_residual else None,
                     _p(res_out), h, w, cin, cout, b, r, s, stride, stride, int(padding), pool, pool,
                     int(ahead_fc), int(inject_residual), residual_channels, int(residual_pool), res_in_ch)
    return out, res_out


def inconv128(x, hwio, bn, stride=1, padding=True, pool=1, save_residual=False):
    x, f, bn = _f32(x), _f32(hwio), _f32(bn)
    b, c, h, w = x.shape
    assert c == 3
    r, s, _, cout = f.shape
    _, ph, oh = conv_geometry(h, r, stride, padding, pool)
    _, pw, ow = conv_geometry(w, s, stride, padding, pool)
    out = np.empty((oh, ow, b, step32(cout)), np.uint32)
    res = np.zeros((ph, pw, b, cout), np.int32) if save_residual else None
    _lib.orc_inconv128(_p(x), _p(f), _p(bn), _p(out), _p(res), h, w, cout, b, r, s, stride, stride,
                       int(padding), pool, pool)
    return out, res


def pool128(inp, c, window, stride, padding, res_in=None):
    """Overlapping OR / max pooling (no counterpart in the reference).  inp: [H][W][B][CW] words; res_in:
    int32 [H][W][B][C] or None.  Returns (packed output, pooled residual or None)."""
    inp = _u32(inp)
    h, w, b, cw = inp.shape
    oh, ow = (h + 2 * padding - window) // stride + 1, (w + 2 * padding - window) // stride + 1
    out = np.empty((oh, ow, b, cw), np.uint32)
    res_out = None
    if res_in is not None:
        res_in = np.ascontiguousarray(res_in, dtype=np.int32)
        res_out = np.empty((oh, ow, b, c), np.int32)
    _lib.orc_pool128(_p(inp), _p(out), _p(res_in) if res_in is not None else None,
                     _p(res_out) if res_out is not None else None, h, w, c, b, window, stride, padding)
    return out, res_out


def avgpool_fc(res, weight, bias):
    """Global average pool + fp32 FC head (no counterpart in the reference).  res: int32 [H][W][B][C];
    weight fp32 [C][N]; bias [N].  Returns fp32 [B][N]."""
    res = np.ascontiguousarray(res, dtype=np.int32)
    weight, bias = _f32(weight), _f32(bias)
    h, w, b, c = res.shape
    n = weight.shape[1]
    out = np.empty((b, n), np.float32)
    _lib.orc_avgpool_fc(_p(res), _p(weight), _p(bias), _p(out), h, w, c, b, n)
    return out


def fc_to_fmt(logical, batch, k):
    logical = _u32(logical)
    out = np.empty(pad8(batch) * step128(k) * 4, np.uint32)
    _lib.orc_fc_to_fmt(_p(logical), _p(out), batch, k)
    return out


def conv_to_fmt(logical, c):
    logical = _u32(logical)
    h, w, b, _ = logical.shape
    out = np.empty(h * w * pad8(b) * step128(c) * 4, np.uint32)
    _lib.orc_conv_to_fmt(_p(logical), _p(out), h, w, b, c)
    return out


def fc_weight_to_fmt(logical, k, n):
    logical = _u32(logical)
    out = np.empty(pad128(n) * step128(k) * 4, np.uint32)
    _lib.orc_fc_weight_to_fmt(_p(logical), _p(out), k, n)
    return out


def conv_filter_to_fmt(logical, r, s, c, o):
    logical = _u32(logical)
    out = np.empty(r * s * (step32(o) * 32) * 4 * step128(c), np.uint32)
    _lib.orc_conv_filter_to_fmt(_p(logical), _p(out), r, s, c, o)
    return out


def residual_to_reference(res):
    res = np.ascontiguousarray(res, dtype=np.int32)
    h, w, b, c = res.shape
    out = np.empty((h, w, pad8(b), pad128(c)), np.int32)
    _lib.orc_residual_to_reference(_p(res), _p(out), h, w, b, c)
    return out


def unpack_bits(words, n):
    """uint32 [..., W] MSB first -> int8 +-1 [..., n]."""
    words = _u32(words)
    shifts = np.arange(31, -1, -1, dtype=np.uint32)
    bits = (words[..., :, None] >> shifts) & 1
    bits = bits.reshape(*words.shape[:-1], -1)[..., :n]
    return (bits.astype(np.int8) * 2 - 1)
