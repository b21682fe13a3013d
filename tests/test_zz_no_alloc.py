"""The fully connected layer's entry point that allocates nothing (split-K partial sums in a buffer built into
the library) against the ordinary entry point with a caller's workspace: same bits, on two calls in a row, the
second with a smaller input (the shared buffer keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

from oracle import orc
from tests import gpuops, refmath as rm

pytestmark = pytest.mark.gpu


def _fc(gpu, entry, inp, wbuf, bn, b, k, n, variant, workspace):
    from tcbnn_amd import _lib
    from tcbnn_amd.device import DeviceBuffer
    lib = _lib.lib
    out = DeviceBuffer(4 * lib.tcbnn_fc_act_words(b, n))
    out.fill(0xAB)
    bnb = gpuops.dev(bn)
    ws_words = ((n + 31) // 32) * 32 * b
    ws = DeviceBuffer(4 * ws_words) if workspace else None
    if ws is not None:
        ws.fill(0x5A)
    d = _lib.Fc128Desc(inp.ptr, wbuf.ptr, bnb.ptr, out.ptr, b, k, n, variant, ws.ptr if ws else None,
                       ws_words if ws else 0)
    _lib.check(getattr(lib, entry)(C.byref(d), None))
    gpuops.sync()
    kw = lib.tcbnn_fc_act_words(1, n)
    return np.ascontiguousarray(out.to_numpy(np.uint32, (kw, b)).T)


@pytest.mark.parametrize("variant", ["popc", "mfma_i8", "mfma_f4"])
def test_fc128_static_scratch_matches_workspace_entry(gpu, variant):
    from tcbnn_amd import _lib
    v = gpu.VARIANTS[variant]
    r = np.random.default_rng(17)
    # (batch, K, N): split over K by the popcount and int8 engines (few rows, long K); the second call is smaller
    # in every dimension, the third larger again
    for b, k, n in [(130, 25088, 64), (40, 4096, 40), (256, 2048, 160), (8, 128, 128)]:
        x = r.standard_normal((b, k)).astype(np.float32)
        w = rm.pm1(r, (k, n))
        bn = r.normal(0, np.sqrt(k), n).astype(np.float32)
        inp, wbuf = gpuops.in128(x), gpuops.pack_fc_weight(w)
        want = _fc(gpu, "tcbnn_fc128_forward", inp, wbuf, bn, b, k, n, v, True)
        got = _fc(gpu, "tcbnn_fc128_forward_static_scratch", inp, wbuf, bn, b, k, n, v, False)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got, orc.fc128(orc.in128(x), orc.pack_fc_weight(w), bn, k, n))
        # again on the same input: the buffer now holds this call's own partial sums
        got = _fc(gpu, "tcbnn_fc128_forward_static_scratch", inp, wbuf, bn, b, k, n, v, False)
        np.testing.assert_array_equal(got, want)
    if variant == "popc":  # the split over K really happened for the first shape (kernel mode 4 = partial sums)
        d = _lib.Fc128Desc(1, 1, 1, 1, 130, 25088, 64, v, 1, 64 * 130)
        name = C.create_string_buffer(128)
        _lib.check(_lib.lib.tcbnn_fc128_kernel_name(C.byref(d), name, 128))
        assert name.value.decode().endswith(", 4>"), name.value


def test_fc128_static_scratch_allocates_nothing(gpu):
    """The property the entry point exists for: with every operand allocated beforehand, repeated calls leave the
    device's free memory exactly where it was (hipMemGetInfo), for the split-K shape as well as a small one."""
    from tcbnn_amd import _lib
    from tcbnn_amd.device import DeviceBuffer
    lib, hip = _lib.lib, _lib.hip
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    v = gpu.VARIANTS["popc"]
    r = np.random.default_rng(18)
    for b, k, n in [(130, 25088, 64), (8, 128, 128)]:
        x = r.standard_normal((b, k)).astype(np.float32)
        inp, wbuf = gpuops.in128(x), gpuops.pack_fc_weight(rm.pm1(r, (k, n)))
        bnb = gpuops.dev(r.normal(0, np.sqrt(k), n).astype(np.float32))
        out = DeviceBuffer(4 * lib.tcbnn_fc_act_words(b, n))
        d = _lib.Fc128Desc(inp.ptr, wbuf.ptr, bnb.ptr, out.ptr, b, k, n, v, None, 0)
        _lib.check(lib.tcbnn_fc128_forward_static_scratch(C.byref(d), None))  # (first call: resolves the buffer's address)
        gpuops.sync()
        free0, free1, total = C.c_size_t(0), C.c_size_t(0), C.c_size_t(0)
        _lib.hip_check(hip.hipMemGetInfo(C.byref(free0), C.byref(total)), "hipMemGetInfo")
        for _ in range(5):
            _lib.check(lib.tcbnn_fc128_forward_static_scratch(C.byref(d), None))
        gpuops.sync()
        _lib.hip_check(hip.hipMemGetInfo(C.byref(free1), C.byref(total)), "hipMemGetInfo")
        assert free1.value == free0.value, (free0.value, free1.value)
        out.free()


def test_fc128_static_scratch_rejects_oversize(gpu):
    from tcbnn_amd import _lib
    d = _lib.Fc128Desc(1, 1, 1, 1, 8192, 1024, 1024, 0, None, 0)  # 8 Mi words: beyond the built-in 1 Mi
    assert _lib.lib.tcbnn_fc128_forward_static_scratch(C.byref(d), None) == -1
    assert b"exceeds" in _lib.lib.tcbnn_last_error()
    assert _lib.lib.tcbnn_fc128_forward_static_scratch(None, None) == -2
