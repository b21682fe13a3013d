"""numpy-in / numpy-out wrappers that drive single operations through the C ABI (test helper)."""
import ctypes as C

import numpy as np

from tcbnn_amd import _lib
from tcbnn_amd._lib import lib, check
from tcbnn_amd.device import DeviceBuffer


def dev(a):
    return DeviceBuffer.from_numpy(np.ascontiguousarray(a))


def sync():
    _lib.device_synchronize()


def pack_fc_weight(w_kn):
    k, n = w_kn.shape
    out = DeviceBuffer(4 * lib.tcbnn_fc_weight_words(k, n))
    src = dev(w_kn.astype(np.float32))
    check(lib.tcbnn_pack_fc_weight(src.ptr, out.ptr, k, n, None))
    sync()
    return out


def pack_conv_filter(f):
    r, s, c, o = f.shape
    out = DeviceBuffer(4 * lib.tcbnn_conv_filter_words(r, s, c, o))
    src = dev(f.astype(np.float32))
    check(lib.tcbnn_pack_conv_filter(src.ptr, out.ptr, r, s, c, o, None))
    sync()
    return out


def pack_conv_input(x_nhwc):
    b, h, w, c = x_nhwc.shape
    out = DeviceBuffer(4 * lib.tcbnn_conv_act_words(h, w, b, c))
    src = dev(x_nhwc.astype(np.float32))
    check(lib.tcbnn_pack_conv_input_nhwc(src.ptr, out.ptr, b, h, w, c, None))
    sync()
    return out


def in128(x):
    b, k = x.shape
    out = DeviceBuffer(4 * lib.tcbnn_fc_act_words(b, k))
    src = dev(x.astype(np.float32))
    d = _lib.In128Desc(src.ptr, out.ptr, b, k)
    check(lib.tcbnn_in128_forward(C.byref(d), None))
    sync()
    return out


def fc128(inp_buf, w_buf, bn, b, k, n, variant=0, workspace=True):
    """Returns the packed output as [B][KW128(n)] rows."""
    out = DeviceBuffer(4 * lib.tcbnn_fc_act_words(b, n))
    out.fill(0xAB)  # the call must overwrite every word, padding included
    bnb = dev(bn.astype(np.float32))
    ws_words = ((n + 31) // 32) * 32 * b
    ws = DeviceBuffer(4 * ws_words) if workspace else None
    if ws is not None:
        ws.fill(0x5A)  # the call must clear what it accumulates into
    d = _lib.Fc128Desc(inp_buf.ptr, w_buf.ptr, bnb.ptr, out.ptr, b, k, n, variant,
                       ws.ptr if ws else None, ws_words if ws else 0)
    check(lib.tcbnn_fc128_forward(C.byref(d), None))
    sync()
    kw = lib.tcbnn_fc_act_words(1, n)
    return np.ascontiguousarray(out.to_numpy(np.uint32, (kw, b)).T)


def out128(inp_buf, w_buf, scale, bias, b, k, n, variant=0):
    out = DeviceBuffer(4 * b * n)
    sb, bb = dev(scale.astype(np.float32)), dev(bias.astype(np.float32))
    d = _lib.Out128Desc(inp_buf.ptr, w_buf.ptr, sb.ptr, bb.ptr, out.ptr, b, k, n, variant)
    check(lib.tcbnn_out128_forward(C.byref(d), None))
    sync()
    return out.to_numpy(np.float32, (b, n))


def bmm(a_packed, b_packed, m, n, k, variant=0):
    """a_packed: [M][K/32] rows (uploaded in the engine's [K/32][M] layout); b_packed: [N][K/32]."""
    a, b = dev(np.ascontiguousarray(a_packed.T)), dev(b_packed)
    c = DeviceBuffer(4 * m * n)
    check(lib.tcbnn_bmm(a.ptr, b.ptr, c.ptr, m, n, k, variant, None))
    sync()
    return c.to_numpy(np.int32, (m, n))


def bconv(inp_buf, filt_buf, b, h, w, cin, cout, r, s, stride, pad, oh, ow, variant=0):
    out = DeviceBuffer(4 * b * oh * ow * cout)
    check(lib.tcbnn_bconv(inp_buf.ptr, filt_buf.ptr, out.ptr, b, h, w, cin, cout, r, s, stride, stride, pad, pad,
                          oh, ow, variant, None))
    sync()
    return out.to_numpy(np.int32, (b, oh, ow, cout))
