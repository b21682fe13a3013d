"""Device memory, streams and events for the Python host mirror (thin HIP runtime plumbing)."""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import hip, hip_check


class DeviceBuffer:
    """Owning handle on a hipMalloc allocation."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p(0)
        hip_check(hip.hipMalloc(C.byref(p), max(self.nbytes, 4)), "hipMalloc(%d)" % self.nbytes)
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            hip_check(hip.hipMemcpy(buf.ptr, arr.ctypes.data, arr.nbytes, _lib.H2D), "hipMemcpy H2D")
        return buf

    @classmethod
    def zeros(cls, nbytes):
        buf = cls(nbytes)
        buf.fill(0)
        return buf

    def fill(self, byte):
        if self.nbytes:
            hip_check(hip.hipMemset(self.ptr, byte, self.nbytes), "hipMemset")

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        hip_check(hip.hipMemcpy(self.ptr, arr.ctypes.data, arr.nbytes, _lib.H2D), "hipMemcpy H2D")

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes, (out.nbytes, self.nbytes)
        if out.nbytes:
            hip_check(hip.hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, _lib.D2H), "hipMemcpy D2H")
        return out

    def free(self):
        if getattr(self, "ptr", None):
            hip.hipFree(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    """A HIP stream at the default priority."""

    def __init__(self):
        p = C.c_void_p(0)
        hip_check(hip.hipStreamCreate(C.byref(p)), "hipStreamCreate")
        self.handle = p.value

    def synchronize(self):
        hip_check(hip.hipStreamSynchronize(self.handle), "hipStreamSynchronize")

    def __del__(self):
        try:
            if self.handle:
                hip.hipStreamDestroy(self.handle)
        except Exception:
            pass


class Event:
    def __init__(self):
        p = C.c_void_p(0)
        hip_check(hip.hipEventCreate(C.byref(p)), "hipEventCreate")
        self.handle = p.value

    def record(self, stream=None):
        hip_check(hip.hipEventRecord(self.handle, stream.handle if stream else None), "hipEventRecord")

    def synchronize(self):
        hip_check(hip.hipEventSynchronize(self.handle), "hipEventSynchronize")

    def elapsed_ms(self, end):
        ms = C.c_float(0)
        hip_check(hip.hipEventElapsedTime(C.byref(ms), self.handle, end.handle), "hipEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self.handle:
                hip.hipEventDestroy(self.handle)
        except Exception:
            pass


class Graph:
    """A HIP graph captured from the launches `record(stream)` makes on `stream` (the layers' forward
    calls allocate nothing and clear nothing with memset, so a whole network can be captured); replay
    with launch().  The caller warms the launches up once before capturing."""

    def __init__(self, stream, record):
        self.stream = stream
        g = C.c_void_p(0)
        hip_check(hip.hipStreamBeginCapture(stream.handle, 0), "hipStreamBeginCapture")  # global mode
        try:
            record(stream)
        finally:
            hip_check(hip.hipStreamEndCapture(stream.handle, C.byref(g)), "hipStreamEndCapture")
        self.graph = g.value
        e = C.c_void_p(0)
        hip_check(hip.hipGraphInstantiate(C.byref(e), self.graph, None, None, 0), "hipGraphInstantiate")
        self.exec = e.value

    def launch(self):
        hip_check(hip.hipGraphLaunch(self.exec, self.stream.handle), "hipGraphLaunch")

    def __del__(self):
        try:
            if getattr(self, "exec", None):
                hip.hipGraphExecDestroy(self.exec)
            if getattr(self, "graph", None):
                hip.hipGraphDestroy(self.graph)
        except Exception:
            pass

