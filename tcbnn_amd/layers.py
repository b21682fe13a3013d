"""Python host mirror of the reference's layer objects (param.h:115-1065).

Same class names, constructor arguments, public field names and method names as
In128LayerParam / Fc128LayerParam / Out128LayerParam / InConv128LayerParam /
Conv128LayerParam.  Differences forced by the redesign:
  * `initialize` takes a weight source with a `launch_array(n)` method (the
    reference reads a FILE* with launch_array, utility.h:188-196) and returns self;
  * each layer has `forward(stream=None)` — one stream-ordered launch — in place of
    the device function called inside the reference's cooperative network kernel;
  * `download_output()` returns the packed activations in the reference's
    tile-contiguous layout (what the reference's download_output() yields);
    `download_packed()` returns them as plain row-major words ([B][KW] for FC layers,
    [H][W][B][CW] for conv layers), transposed on the host from the engine's
    batch-innermost device layout.
All compute goes through the C ABI of libtcbnn_hip.so.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import lib, check
from .device import DeviceBuffer


def STEP8(x):
    return (x + 7) >> 3


def STEP32(x):
    return (x + 31) >> 5


def STEP128(x):
    return (x + 127) >> 7


def PAD8(x):
    return STEP8(x) << 3


def PAD32(x):
    return STEP32(x) << 5


def PAD128(x):
    return STEP128(x) << 7


class ArrayWeights:
    """Weight source over in-memory arrays, consumed strictly in order like the
    reference's weight file (utility.h:188-196)."""

    def __init__(self, arrays):
        self._flat = np.concatenate([np.asarray(a, dtype=np.float32).ravel() for a in arrays]) \
            if arrays else np.zeros(0, np.float32)
        self._pos = 0

    def launch_array(self, size):
        if self._pos + size > self._flat.size:
            raise _lib.TcbnnError("weight source exhausted: need %d more values" % size)
        out = self._flat[self._pos:self._pos + size]
        self._pos += size
        return out


class TextWeightFile:
    """Text file of floats separated by white space and/or commas (the reference's .csv)."""

    def __init__(self, path):
        with open(path) as f:
            txt = f.read().replace(",", " ")
        self._src = ArrayWeights([np.array(txt.split(), dtype=np.float32)])

    def launch_array(self, size):
        return self._src.launch_array(size)


def _stream_handle(stream):
    return stream.handle if stream is not None else None


def _residual_buffer(channels, height, width, batch, bound, force_format=None):
    """Device buffer of a saved residual.  `bound` is an upper bound of |value| (INT32_MAX when
    unknown); the narrowest format the bound allows is chosen: 12 bits up to 2047 (even batches), 16 bits up to
    32767, else int32 (or as `force_format` says)."""
    fmt = lib.tcbnn_residual_format_narrowest(bound, batch) if force_format is None else force_format
    buf = DeviceBuffer(lib.tcbnn_residual_bytes(height, width, channels, batch, fmt))
    buf.channels, buf.height, buf.width, buf.batch = channels, height, width, batch
    buf.bound, buf.format = bound, fmt
    # Who reads the tensor decides whether its producer may store only the maximum over 2x2 windows of pixels
    # (_SavedResidualUse): how often the pointer was handed out, how many Conv128 consumers registered with
    # residual_pool, how many other consumers, whether the full tensor was ever asked for, and what the buffer
    # holds since the producer's last forward().
    buf.handed_out = buf.pool_consumers = buf.other_consumers = 0
    buf.observed = buf.pooled = buf.written = False
    buf.producer = None
    buf.readers = []  # the layers of this library that read the tensor (their own saved residuals depend on its bound)
    return buf


def _register_residual_consumer(buf, pools, sign=1, layer=None):
    """A layer of this library starts (sign = +1) or stops (-1) reading the saved residual `buf`."""
    if buf is not None and hasattr(buf, "pool_consumers"):
        if pools:
            buf.pool_consumers += sign
        else:
            buf.other_consumers += sign
        if layer is not None:
            if sign > 0:
                buf.readers.append(layer)
            elif layer in buf.readers:
                buf.readers.remove(layer)


_FORMAT_LIMIT = {_lib.RES_I12: 2047, _lib.RES_I16: 32767, _lib.RES_I32: _lib.INT32_MAX // 4}


def _residual_bound_limit(buf):
    """The largest bound of |value| the saved residual `buf` can take with every tensor that depends on it
    staying in the format it was allocated in: its own format's range, and for every reader that saves a
    residual of its own, that tensor's limit less what the reader adds (Cin*R*S for a bit convolution)."""
    lim = _FORMAT_LIMIT[buf.format]
    for reader in buf.readers:
        out, add = reader._residual_dependency()
        if out is not None:
            lim = min(lim, _residual_bound_limit(out) - add)
    return lim


def _raise_residual_bound(buf, bound):
    """Record a larger bound for `buf` (within _residual_bound_limit) and for everything that depends on it."""
    if bound <= buf.bound:
        return
    buf.bound = bound
    for reader in buf.readers:
        out, add = reader._residual_dependency()
        if out is not None:
            _raise_residual_bound(out, bound + add)


def _residual_holds_window_maximum(buf):
    """Does `buf` hold (after its producer's forward) the maximum over 2x2 windows instead of the full tensor?"""
    if buf is None or getattr(buf, "producer", None) is None:
        return False
    return buf.pooled if buf.written else buf.producer._pooled_save_now()


def _unpack_residual(buf, P, Q, O, B):
    """A residual tensor of P x Q pixels in the engine layout `buf.format` -> int32 [P][Q][B][O]."""
    if buf.format == _lib.RES_I12:
        # groups of 16 channels; per pixel and group the words w0..w3 of every image, then w4, w5 of every image;
        # value e sits at bits 12e..12e+11 of the 192-bit string w0..w5 (two's complement)
        G = (O + 15) // 16
        raw = buf.to_numpy(np.uint32, (P, Q, G, 6 * B)).astype(np.uint64)
        words = np.concatenate([raw[..., :4 * B].reshape(P, Q, G, B, 4), raw[..., 4 * B:].reshape(P, Q, G, B, 2)],
                               axis=-1)
        vals = np.empty((P, Q, G, B, 16), np.int64)
        for e in range(16):
            k, sh = (12 * e) >> 5, (12 * e) & 31
            v = words[..., k] >> np.uint64(sh)
            if sh > 20:
                v = v | (words[..., k + 1] << np.uint64(32 - sh))
            v = (v & np.uint64(0xfff)).astype(np.int64)
            vals[..., e] = (v ^ 0x800) - 0x800
        return np.ascontiguousarray(vals.transpose(0, 1, 3, 2, 4).reshape(P, Q, B, G * 16)[..., :O].astype(np.int32))
    # engine layouts: int32 [P][Q][ceil(O/4)][B][4] or int16 [P][Q][ceil(O/8)][B][8]
    grp, dt = (8, np.int16) if buf.format == _lib.RES_I16 else (4, np.int32)
    ng = (O + grp - 1) // grp
    eng = buf.to_numpy(dt, (P, Q, ng, B, grp))
    return np.ascontiguousarray(eng.transpose(0, 1, 3, 2, 4).reshape(P, Q, B, ng * grp)[..., :O].astype(np.int32))


class _ReferenceLayoutIO:
    """Device buffers in the reference's own tile layouts at a layer's edges, for a neighbour that is a
    layer of the reference (FC tiles [B/8][K/128][8][4], kernel.cuh:170,187-191,222-223; conv tiles
    [H][W][B/8][C/128][8][4], kernel.cuh:650-660,741-749,811-815; residuals int32
    [P][Q][PAD8(B)][PAD128(O)], kernel.cuh:666-668,770-791,820-823).  Every accessor enqueues a conversion
    on `stream` between such a buffer and one in the engine's layout that the layer owns: copies, not
    views, so imports are repeated when the source changes and exports after every forward()."""

    def _ref_buf(self, key, nbytes):
        bufs = self.__dict__.setdefault("_ref_bufs", {})
        if key not in bufs:
            bufs[key] = DeviceBuffer(nbytes)
        return bufs[key]

    def _release_ref_bufs(self):
        for b in self.__dict__.pop("_ref_bufs", {}).values():
            b.free()

    # how this layer's input / output bits are tiled: ("fc", batch, features) or ("conv", h, w, batch, channels)
    def _input_tiling(self):
        if hasattr(self, "input_channels"):
            return ("conv", self.input_height, self.input_width, self.batch, self.input_channels)
        return ("fc", self.input_height, self.input_width)

    def _output_tiling(self):
        if hasattr(self, "output_channels"):
            if getattr(self, "ahead_fc", False):
                return ("fc", self.batch, self.output_height * self.output_width * PAD128(self.output_channels))
            return ("conv", self.output_height, self.output_width, self.batch, self.output_channels)
        return ("fc", self.output_height, self.output_width)

    def set_input_gpu_reference_fmt(self, fmt_gpu, stream=None):
        t = self._input_tiling()
        if t[0] == "fc":
            own = self._ref_buf("in", 4 * lib.tcbnn_fc_act_words(t[1], t[2]))
            check(lib.tcbnn_fc_from_reference_fmt(fmt_gpu.ptr, own.ptr, t[1], t[2], _stream_handle(stream)))
        else:
            own = self._ref_buf("in", 4 * lib.tcbnn_conv_act_words(t[1], t[2], t[3], t[4]))
            check(lib.tcbnn_conv_from_reference_fmt(fmt_gpu.ptr, own.ptr, t[1], t[2], t[3], t[4],
                                                    _stream_handle(stream)))
        self.input_gpu = own

    def get_output_gpu_reference_fmt(self, stream=None):
        t = self._output_tiling()
        fmt = self._ref_buf("out", 16 * self.output_bit_size())
        if t[0] == "fc":
            check(lib.tcbnn_fc_to_reference_fmt(self.output_gpu.ptr, fmt.ptr, t[1], t[2], _stream_handle(stream)))
        else:
            check(lib.tcbnn_conv_to_reference_fmt(self.output_gpu.ptr, fmt.ptr, t[1], t[2], t[3], t[4],
                                                  _stream_handle(stream)))
        return fmt

    def get_output_residual_gpu_reference(self, stream=None):
        src = self.output_residual_gpu
        if src is None:
            raise _lib.TcbnnError("Error: NULL pointer (output_residual_gpu)")
        self._want_full_residual(stream)
        ref = self._ref_buf("res_out", 4 * self.buf_height * self.buf_width * PAD8(self.batch)
                            * PAD128(self.output_channels))
        check(lib.tcbnn_residual_to_reference(src.ptr, ref.ptr, self.buf_height, self.buf_width, self.batch,
                                              self.output_channels, src.format, _stream_handle(stream)))
        return ref

    def set_input_residual_gpu_reference(self, ref_gpu, stream=None):
        """Nothing is known about a foreign residual's values: it is kept as int32 with an unknown bound, so a
        layer that also saves a residual must have been initialized with an equally unbounded source."""
        scale = 2 if self.residual_pool else 1
        rh, rw = self.buf_height * scale, self.buf_width * scale
        bufs = self.__dict__.setdefault("_ref_bufs", {})
        if "res_in" not in bufs:
            bufs["res_in"] = _residual_buffer(self.residual_channels, rh, rw, self.batch, _lib.INT32_MAX,
                                              _lib.RES_I32)
        own = bufs["res_in"]
        check(lib.tcbnn_residual_from_reference(ref_gpu.ptr, own.ptr, rh, rw, self.batch, self.residual_channels,
                                                _lib.RES_I32, _stream_handle(stream)))
        self.set_input_residual_gpu(own)


class In128LayerParam(_ReferenceLayoutIO):
    """param.h:115-222; forward = In128LayerFMT (kernel.cuh:153-172)."""

    def __init__(self, name, input_height, input_width):
        self.name = name
        self.input_height = self.output_height = input_height
        self.input_width = self.output_width = input_width
        self.input_gpu = self.output_gpu = None

    def output_bit_size(self):
        return PAD8(self.output_height) * STEP128(self.output_width)

    def output_bit_bytes(self):
        return self.output_bit_size() * 16

    def initialize(self, input):
        if input is None:
            raise _lib.TcbnnError("Error: NULL pointer (input)")
        x = np.ascontiguousarray(input, dtype=np.float32).reshape(self.input_height, self.input_width)
        self.input_gpu = DeviceBuffer.from_numpy(x)
        self.output_gpu = DeviceBuffer(4 * lib.tcbnn_fc_act_words(self.output_height, self.output_width))
        return self

    def set_input(self, input):
        self.input_gpu.upload(np.ascontiguousarray(input, dtype=np.float32))

    def get_output_gpu(self):
        return self.output_gpu

    def forward(self, stream=None):
        d = _lib.In128Desc(self.input_gpu.ptr, self.output_gpu.ptr, self.input_height, self.input_width)
        check(lib.tcbnn_in128_forward(C.byref(d), _stream_handle(stream)))

    def download_packed(self):
        eng = self.output_gpu.to_numpy(np.uint32, (4 * STEP128(self.output_width), self.output_height))
        return np.ascontiguousarray(eng.T)

    def download_output(self):
        return _fc_download_fmt(self.output_gpu, self.output_height, self.output_width)

    def download_full_output(self):
        return _fc_download_full(self.output_gpu, self.output_height, self.output_width)

    def release(self):
        self._release_ref_bufs()
        for b in (self.input_gpu, self.output_gpu):
            if b is not None:
                b.free()
        self.input_gpu = self.output_gpu = None


def _fc_download_fmt(buf, batch, features):
    words = PAD8(batch) * STEP128(features) * 4
    tmp = DeviceBuffer(4 * words)
    check(lib.tcbnn_fc_to_reference_fmt(buf.ptr, tmp.ptr, batch, features, None))
    _lib.device_synchronize()
    return tmp.to_numpy(np.uint32, (words,))


def _fc_download_full(buf, batch, features):
    tmp = DeviceBuffer(4 * batch * features)
    check(lib.tcbnn_unpack_fc_output(buf.ptr, tmp.ptr, batch, features, None))
    _lib.device_synchronize()
    return tmp.to_numpy(np.float32, (batch, features))


class Fc128LayerParam(_ReferenceLayoutIO):
    """param.h:224-385; forward = Fc128LayerFMT (kernel.cuh:174-226)."""

    def __init__(self, name, input_height, input_width, weight_width, variant=_lib.VARIANT_AUTO):
        self.name = name
        self.weight_height, self.weight_width = input_width, weight_width
        self.input_height, self.input_width = input_height, input_width
        self.output_height, self.output_width = input_height, weight_width
        self.bn_width = weight_width
        self.variant = variant
        self.weight = self.bn = None
        self.weight_gpu = self.bn_gpu = self.output_gpu = self.input_gpu = None

    def weight_size(self):
        return self.weight_height * self.weight_width

    def bn_size(self):
        return self.bn_width

    def output_bit_size(self):
        return PAD8(self.output_height) * STEP128(self.output_width)

    def set_input_gpu(self, input_gpu):
        self.input_gpu = input_gpu

    def initialize(self, config_file, prev_layer_gpu):
        self.weight = np.array(config_file.launch_array(self.weight_size()), dtype=np.float32)
        self.weight_gpu = DeviceBuffer(4 * lib.tcbnn_fc_weight_words(self.weight_height, self.weight_width))
        wf = DeviceBuffer.from_numpy(self.weight)
        check(lib.tcbnn_pack_fc_weight(wf.ptr, self.weight_gpu.ptr, self.weight_height, self.weight_width, None))
        _lib.device_synchronize()
        wf.free()
        self.bn = np.array(config_file.launch_array(self.bn_size()), dtype=np.float32)
        self.bn_gpu = DeviceBuffer.from_numpy(self.bn)
        self.output_gpu = DeviceBuffer(4 * lib.tcbnn_fc_act_words(self.output_height, self.output_width))
        # scratch for split-K: int32 [PAD32(N)][B]
        self.workspace_words = PAD32(self.weight_width) * self.input_height
        self.workspace_gpu = DeviceBuffer(4 * self.workspace_words)
        self.set_input_gpu(prev_layer_gpu)
        if self.input_gpu is None:
            raise _lib.TcbnnError("Error: NULL pointer (input_gpu)")
        return self

    def get_output_gpu(self):
        return self.output_gpu

    def _desc(self):
        return _lib.Fc128Desc(self.input_gpu.ptr, self.weight_gpu.ptr, self.bn_gpu.ptr, self.output_gpu.ptr,
                              self.input_height, self.input_width, self.weight_width, self.variant,
                              self.workspace_gpu.ptr, self.workspace_words)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_fc128_forward(C.byref(d), _stream_handle(stream)))

    def kernel_name(self):
        buf = C.create_string_buffer(128)
        d = self._desc()
        check(lib.tcbnn_fc128_kernel_name(C.byref(d), buf, 128))
        return buf.value.decode()

    def download_packed(self):
        eng = self.output_gpu.to_numpy(np.uint32, (4 * STEP128(self.output_width), self.output_height))
        return np.ascontiguousarray(eng.T)

    def download_output(self):
        return _fc_download_fmt(self.output_gpu, self.output_height, self.output_width)

    def download_full_output(self):
        return _fc_download_full(self.output_gpu, self.output_height, self.output_width)

    def release(self):
        self._release_ref_bufs()
        for b in (self.weight_gpu, self.bn_gpu, self.output_gpu, getattr(self, "workspace_gpu", None)):
            if b is not None:
                b.free()
        self.weight_gpu = self.bn_gpu = self.output_gpu = self.workspace_gpu = None


class Out128LayerParam(_ReferenceLayoutIO):
    """param.h:388-531; forward = Out128LayerFMT (kernel.cuh:230-280)."""

    def __init__(self, name, input_height, input_width, weight_width, variant=_lib.VARIANT_AUTO):
        self.name = name
        self.input_height, self.input_width = input_height, input_width
        self.weight_height, self.weight_width = input_width, weight_width
        self.output_height, self.output_width = input_height, weight_width
        self.variant = variant
        self.weight = self.bn_scale = self.bn_bias = None
        self.weight_gpu = self.bn_scale_gpu = self.bn_bias_gpu = self.output_gpu = self.input_gpu = None

    def weight_size(self):
        return self.weight_height * self.weight_width

    def bn_size(self):
        return self.output_width

    def set_input_gpu(self, input_gpu):
        self.input_gpu = input_gpu

    def initialize(self, config_file, prev_layer_gpu):
        self.weight = np.array(config_file.launch_array(self.weight_size()), dtype=np.float32)
        self.weight_gpu = DeviceBuffer(4 * lib.tcbnn_fc_weight_words(self.weight_height, self.weight_width))
        wf = DeviceBuffer.from_numpy(self.weight)
        check(lib.tcbnn_pack_fc_weight(wf.ptr, self.weight_gpu.ptr, self.weight_height, self.weight_width, None))
        _lib.device_synchronize()
        wf.free()
        self.bn_scale = np.array(config_file.launch_array(self.bn_size()), dtype=np.float32)
        self.bn_scale_gpu = DeviceBuffer.from_numpy(self.bn_scale)
        self.bn_bias = np.array(config_file.launch_array(self.bn_size()), dtype=np.float32)
        self.bn_bias_gpu = DeviceBuffer.from_numpy(self.bn_bias)
        self.output_gpu = DeviceBuffer.zeros(4 * self.output_height * self.output_width)
        self.set_input_gpu(prev_layer_gpu)
        if self.input_gpu is None:
            raise _lib.TcbnnError("Error: NULL pointer (input_gpu)")
        return self

    def get_output_gpu(self):
        return self.output_gpu

    def _desc(self):
        return _lib.Out128Desc(self.input_gpu.ptr, self.weight_gpu.ptr, self.bn_scale_gpu.ptr,
                               self.bn_bias_gpu.ptr, self.output_gpu.ptr, self.input_height,
                               self.input_width, self.weight_width, self.variant)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_out128_forward(C.byref(d), _stream_handle(stream)))

    def kernel_name(self):
        buf = C.create_string_buffer(128)
        d = self._desc()
        check(lib.tcbnn_out128_kernel_name(C.byref(d), buf, 128))
        return buf.value.decode()

    def download_output(self):
        return self.output_gpu.to_numpy(np.float32, (self.output_height, self.output_width))

    def release(self):
        self._release_ref_bufs()
        for b in (self.weight_gpu, self.bn_scale_gpu, self.bn_bias_gpu, self.output_gpu):
            if b is not None:
                b.free()
        self.weight_gpu = self.bn_scale_gpu = self.bn_bias_gpu = self.output_gpu = None


class _ConvGeometry(_ReferenceLayoutIO):
    """Derived geometry shared by both conv constructors (param.h:719-728, 897-906)."""

    def _derive(self):
        self.pad_h = lib.tcbnn_conv_pad(self.input_height, self.filter_height, self.stride_height, int(self.padding))
        self.pad_w = lib.tcbnn_conv_pad(self.input_width, self.filter_width, self.stride_width, int(self.padding))
        self.buf_height = lib.tcbnn_conv_out(self.input_height, self.filter_height, self.stride_height, int(self.padding), 1)
        self.buf_width = lib.tcbnn_conv_out(self.input_width, self.filter_width, self.stride_width, int(self.padding), 1)
        self.output_height = lib.tcbnn_conv_out(self.input_height, self.filter_height, self.stride_height,
                                                int(self.padding), self.pool_height)
        self.output_width = lib.tcbnn_conv_out(self.input_width, self.filter_width, self.stride_width,
                                               int(self.padding), self.pool_width)

    def filter_size(self):
        return self.output_channels * self.input_channels * self.filter_height * self.filter_width

    def bn_size(self):
        return self.output_channels

    def output_bit_size(self):
        return STEP128(self.output_channels) * self.output_height * self.output_width * PAD8(self.batch)

    def residual_size(self):
        return PAD128(self.output_channels) * PAD8(self.batch) * self.output_height * self.output_width

    def get_output_gpu(self):
        return self.output_gpu

    def get_output_residual_gpu(self):
        """The saved residual, for a consumer's initialize().  (Every hand-out is counted: as long as each one
        is matched by a Conv128 consumer that registers with residual_pool, nobody else can be reading the
        tensor, and the producer may store its 2x2 maximum alone.)"""
        if self.output_residual_gpu is not None:
            self.output_residual_gpu.handed_out += 1
        return self.output_residual_gpu

    def _pooled_save_now(self):
        return False  # (only Conv128 layers can store the window maximum)

    def _residual_dependency(self):
        """(saved residual that depends on the injected one, what this layer adds to its bound), or (None, 0)."""
        return None, 0

    def _want_full_residual(self, stream=None):
        """The full P x Q tensor is asked for: from now on it is what forward() saves, and if the buffer holds
        the 2x2 maximum from the last forward(), the layer is run again (its inputs are still in place)."""
        buf = self.output_residual_gpu
        buf.observed = True
        if buf.pooled:
            self.forward(stream)

    def download_residual(self):
        """Saved residual as int32 [P][Q][B][O] (host transpose of the engine's layouts)."""
        self._want_full_residual()
        _lib.device_synchronize()
        return _unpack_residual(self.output_residual_gpu, self.buf_height, self.buf_width, self.output_channels,
                                self.batch)

    def download_saved_residual(self):
        """What the buffer holds since the last forward(), without asking for anything: (int32 [P'][Q'][B][O],
        pooled) with P' x Q' = P/2 x Q/2 and every value the maximum over a 2x2 window when `pooled`."""
        buf = self.output_residual_gpu
        _lib.device_synchronize()
        k = 2 if buf.pooled else 1
        return _unpack_residual(buf, self.buf_height // k, self.buf_width // k, self.output_channels, self.batch), \
            buf.pooled

    def download_residual_reference(self):
        """Saved residual in the reference layout int32 [P][Q][PAD8(B)][PAD128(O)]."""
        self._want_full_residual()
        shape = (self.buf_height, self.buf_width, PAD8(self.batch), PAD128(self.output_channels))
        tmp = DeviceBuffer(4 * int(np.prod(shape)))
        check(lib.tcbnn_residual_to_reference(self.output_residual_gpu.ptr, tmp.ptr, self.buf_height,
                                              self.buf_width, self.batch, self.output_channels,
                                              self.output_residual_gpu.format, None))
        _lib.device_synchronize()
        return tmp.to_numpy(np.int32, shape)

    def _is_fc_ready(self):
        return bool(getattr(self, "ahead_fc", False))

    def download_packed(self):
        if self._is_fc_ready():
            eng = self.output_gpu.to_numpy(
                np.uint32, (self.output_height * self.output_width * 4 * STEP128(self.output_channels), self.batch))
            return np.ascontiguousarray(eng.T)
        eng = self.output_gpu.to_numpy(
            np.uint32, (self.output_height, self.output_width, STEP32(self.output_channels), self.batch))
        return np.ascontiguousarray(eng.transpose(0, 1, 3, 2))

    def download_output(self):
        if self._is_fc_ready():
            feats = self.output_height * self.output_width * PAD128(self.output_channels)
            return _fc_download_fmt(self.output_gpu, self.batch, feats)
        words = self.output_bit_size() * 4
        tmp = DeviceBuffer(4 * words)
        check(lib.tcbnn_conv_to_reference_fmt(self.output_gpu.ptr, tmp.ptr, self.output_height,
                                              self.output_width, self.batch, self.output_channels, None))
        _lib.device_synchronize()
        return tmp.to_numpy(np.uint32, (words,))

    def download_full_output(self):
        """+-1.0f, NHWC [B][OH][OW][O] (UnpackConvOutput32FMT, param.h:661-688)."""
        if self._is_fc_ready():
            feats = self.output_height * self.output_width * PAD128(self.output_channels)
            full = _fc_download_full(self.output_gpu, self.batch, feats)
            full = full.reshape(self.batch, self.output_height, self.output_width, PAD128(self.output_channels))
            return np.ascontiguousarray(full[..., :self.output_channels])
        shape = (self.batch, self.output_height, self.output_width, self.output_channels)
        tmp = DeviceBuffer(4 * int(np.prod(shape)))
        check(lib.tcbnn_unpack_conv_output(self.output_gpu.ptr, tmp.ptr, self.output_height, self.output_width,
                                           self.output_channels, self.batch, None))
        _lib.device_synchronize()
        return tmp.to_numpy(np.float32, shape)


class InConv128LayerParam(_ConvGeometry):
    """param.h:701-870; forward = InConv128LayerFMT (kernel.cuh:578-672)."""

    def __init__(self, name, input_height, input_width, filter_height, filter_width, input_channels,
                 output_channels, batch, stride_height=1, stride_width=1, padding=True, pool_height=1,
                 pool_width=1, save_residual=False, residual_format=None, input_layout=None):
        self.name = name
        self.residual_format = residual_format  # None: narrowest exact format; or _lib.RES_I32 / RES_I16
        # None / _lib.INCONV_INPUT_NCHW: the layer reads the uploaded [batch][3][H][W] array (the reference's device
        # layout, kernel.cuh:620-625).  _lib.INCONV_INPUT_PACKED: initialize / set_input also make a zero-padded,
        # batch-innermost copy on the device and the (un-pooled) layer reads that with a kernel that needs no
        # staging; the upload then costs one more pass over the input, the forward pass less.
        self.input_layout = input_layout
        self.input_height, self.input_width = input_height, input_width
        self.filter_height, self.filter_width = filter_height, filter_width
        self.input_channels, self.output_channels, self.batch = input_channels, output_channels, batch
        self.stride_height, self.stride_width = stride_height, stride_width
        self.padding, self.pool_height, self.pool_width = padding, pool_height, pool_width
        self.save_residual = save_residual
        self.filter = self.bn = None
        self.input_gpu = self.filter_gpu = self.bn_gpu = self.output_gpu = self.output_residual_gpu = None
        self.input_packed_gpu = None
        self._derive()

    def input_size(self):
        return self.input_channels * self.input_height * self.input_width * self.batch

    def _packed_floats(self):
        """Size of the zero-padded, batch-innermost copy of the input that the un-pooled first layer reads
        (tcbnn_inconv_pack_input), or 0 where the layer reads the uploaded [batch][3][H][W] array itself."""
        if self.pool_height != 1 or self.pool_width != 1 or self.input_layout != _lib.INCONV_INPUT_PACKED:
            return 0
        n = lib.tcbnn_inconv_packed_input_floats(
            self.batch, self.input_height, self.input_width, self.filter_height, self.filter_width,
            self.stride_height, self.stride_width, int(self.padding))
        return n if 0 < 4 * n < (1 << 31) else 0

    def _pack_input(self):
        if self.input_packed_gpu is None:
            return
        check(lib.tcbnn_inconv_pack_input(
            self.input_gpu.ptr, self.input_packed_gpu.ptr, self.batch, self.input_height, self.input_width,
            self.filter_height, self.filter_width, self.stride_height, self.stride_width, int(self.padding), None))
        _lib.device_synchronize()

    def initialize(self, input, config_file):
        if input is None:
            raise _lib.TcbnnError("Error: NULL pointer (input)")
        x = np.ascontiguousarray(input, dtype=np.float32)
        assert x.size == self.input_size(), (x.size, self.input_size())
        self.input_gpu = DeviceBuffer.from_numpy(x)
        if self._packed_floats():
            self.input_packed_gpu = DeviceBuffer(4 * self._packed_floats())
            self._pack_input()
        self.input_abs_max = float(np.max(np.abs(x))) if x.size else 0.0
        self.filter = np.array(config_file.launch_array(self.filter_size()), dtype=np.float32)
        self.filter_gpu = DeviceBuffer(4 * lib.tcbnn_inconv_filter_words(
            self.filter_height, self.filter_width, self.input_channels, self.output_channels))
        ff = DeviceBuffer.from_numpy(self.filter)
        check(lib.tcbnn_pack_inconv_filter(ff.ptr, self.filter_gpu.ptr, self.filter_height, self.filter_width,
                                           self.input_channels, self.output_channels, None))
        _lib.device_synchronize()
        ff.free()
        self.bn = np.array(config_file.launch_array(self.bn_size()), dtype=np.float32)
        self.bn_gpu = DeviceBuffer.from_numpy(self.bn)
        self.output_gpu = DeviceBuffer(4 * lib.tcbnn_conv_act_words(
            self.output_height, self.output_width, self.batch, self.output_channels))
        if self.save_residual:
            bound = self._residual_bound(x)
            self.output_residual_gpu = _residual_buffer(self.output_channels, self.buf_height, self.buf_width,
                                                        self.batch, bound, self.residual_format)
        return self

    def _residual_bound(self, x):
        """Upper bound of |first-layer sum| for this batch: the largest sum of |x| under any filter window."""
        return lib.tcbnn_inconv_residual_bound_of_input(
            x.ctypes.data, self.batch, self.input_height, self.input_width, self.filter_height, self.filter_width,
            self.stride_height, self.stride_width, int(self.padding))

    def set_input(self, input):
        """A new batch.  The residual formats downstream were chosen from the first batch's bound; a batch whose
        sums can be larger is accepted as long as every one of those tensors still holds its values (the recorded
        bounds are raised), and refused only when a format would have to change.  The window scan of the batch is
        skipped when R*S*3*max|x| already fits."""
        x = np.ascontiguousarray(input, dtype=np.float32)
        assert x.size == self.input_size(), (x.size, self.input_size())
        if self.save_residual:
            buf = self.output_residual_gpu
            coarse = lib.tcbnn_inconv_residual_bound(self.filter_height, self.filter_width,
                                                     lib.tcbnn_host_abs_max(x.ctypes.data, x.size))
            limit = _residual_bound_limit(buf)
            if coarse > buf.bound:
                bound = coarse if coarse <= limit else self._residual_bound(x)
                if bound > limit:
                    raise _lib.TcbnnError("input magnitude (window sums of |x| up to %d) exceeds what the residual "
                                          "formats chosen at initialize() hold (up to %d)" % (bound, limit))
                _raise_residual_bound(buf, bound)
        self.input_gpu.upload(x)
        self._pack_input()

    def _desc(self):
        packed = self.input_packed_gpu is not None
        return _lib.InConv128Desc(
            (self.input_packed_gpu if packed else self.input_gpu).ptr, self.filter_gpu.ptr, self.bn_gpu.ptr, self.output_gpu.ptr,
            self.output_residual_gpu.ptr if self.output_residual_gpu is not None else None,
            self.input_height, self.input_width, self.input_channels, self.filter_height, self.filter_width,
            self.output_channels, self.batch, self.stride_height, self.stride_width, int(self.padding),
            self.pool_height, self.pool_width, int(self.save_residual),
            self.output_residual_gpu.format if self.output_residual_gpu is not None else 0,
            _lib.INCONV_INPUT_PACKED if packed else _lib.INCONV_INPUT_NCHW)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_inconv128_forward(C.byref(d), _stream_handle(stream)))

    def kernel_name(self):
        buf = C.create_string_buffer(128)
        d = self._desc()
        check(lib.tcbnn_inconv128_kernel_name(C.byref(d), buf, 128))
        return buf.value.decode()

    def release(self):
        self._release_ref_bufs()
        for b in (self.input_gpu, self.input_packed_gpu, self.filter_gpu, self.bn_gpu, self.output_gpu,
                  self.output_residual_gpu):
            if b is not None:
                b.free()
        self.input_gpu = self.filter_gpu = self.bn_gpu = self.output_gpu = self.output_residual_gpu = None
        self.input_packed_gpu = None


class Conv128LayerParam(_ConvGeometry):
    """param.h:872-1065; forward = Conv128LayerFMT (kernel.cuh:676-827)."""

    def __init__(self, name, input_height, input_width, filter_height, filter_width, input_channels,
                 output_channels, batch, stride_height=1, stride_width=1, padding=True, pool_height=1,
                 pool_width=1, ahead_fc=False, save_residual=False, inject_residual=False,
                 residual_channels=0, residual_pool=False, variant=_lib.VARIANT_AUTO, residual_format=None):
        self.name = name
        self.residual_format = residual_format  # None: narrowest exact format; or _lib.RES_I32 / RES_I16
        self.input_height, self.input_width = input_height, input_width
        self.filter_height, self.filter_width = filter_height, filter_width
        self.input_channels, self.output_channels, self.batch = input_channels, output_channels, batch
        self.stride_height, self.stride_width = stride_height, stride_width
        self.padding, self.pool_height, self.pool_width = padding, pool_height, pool_width
        self.ahead_fc, self.save_residual, self.inject_residual = ahead_fc, save_residual, inject_residual
        self.residual_channels, self.residual_pool = residual_channels, residual_pool
        self.variant = variant
        self.filter = self.bn = None
        self.input_gpu = self.filter_gpu = self.bn_gpu = self.output_gpu = None
        self.output_residual_gpu = self.input_residual_gpu = None
        self._derive()

    def set_input_gpu(self, input_gpu):
        self.input_gpu = input_gpu

    def set_input_residual_gpu(self, input_residual_gpu):
        if input_residual_gpu is not None and not hasattr(input_residual_gpu, "bound"):
            # a residual that no layer of this library produced: int32 with the consumer's channel limit and
            # no known bound
            input_residual_gpu.channels, input_residual_gpu.format = self.residual_channels, _lib.RES_I32
            input_residual_gpu.bound = _lib.INT32_MAX
        out = self.output_residual_gpu
        if out is not None and input_residual_gpu is not None and self.inject_residual and \
                lib.tcbnn_conv_residual_bound(self.input_channels, self.filter_height, self.filter_width,
                                              min(input_residual_gpu.bound, _lib.INT32_MAX // 4)) > out.bound:
            raise _lib.TcbnnError("injected residual exceeds the bound the saved residual's format was chosen for")
        if self.inject_residual:
            _register_residual_consumer(self.input_residual_gpu, self.residual_pool, -1, self)
            _register_residual_consumer(input_residual_gpu, self.residual_pool, +1, self)
        self.input_residual_gpu = input_residual_gpu

    def initialize(self, config_file, prev_layer_gpu, input_residual_gpu=None):
        self.filter = np.array(config_file.launch_array(self.filter_size()), dtype=np.float32)
        self.filter_gpu = DeviceBuffer(4 * lib.tcbnn_conv_filter_words(
            self.filter_height, self.filter_width, self.input_channels, self.output_channels))
        ff = DeviceBuffer.from_numpy(self.filter)
        check(lib.tcbnn_pack_conv_filter(ff.ptr, self.filter_gpu.ptr, self.filter_height, self.filter_width,
                                         self.input_channels, self.output_channels, None))
        _lib.device_synchronize()
        ff.free()
        self.bn = np.array(config_file.launch_array(self.bn_size()), dtype=np.float32)
        self.bn_gpu = DeviceBuffer.from_numpy(self.bn)
        if self.ahead_fc:
            words = lib.tcbnn_fc_act_words(
                self.batch, self.output_height * self.output_width * PAD128(self.output_channels))
        else:
            words = lib.tcbnn_conv_act_words(self.output_height, self.output_width, self.batch,
                                             self.output_channels)
        self.output_gpu = DeviceBuffer(4 * words)
        self.set_input_gpu(prev_layer_gpu)
        if self.inject_residual:
            self.set_input_residual_gpu(input_residual_gpu)
            if self.input_residual_gpu is None:
                raise _lib.TcbnnError("Error: NULL pointer (input_residual_gpu)")
        if self.save_residual:
            injected = self.input_residual_gpu.bound if self.inject_residual else 0
            bound = lib.tcbnn_conv_residual_bound(self.input_channels, self.filter_height, self.filter_width,
                                                  injected) if injected < _lib.INT32_MAX else _lib.INT32_MAX
            self.output_residual_gpu = _residual_buffer(self.output_channels, self.buf_height, self.buf_width,
                                                        self.batch, bound, self.residual_format)
            self.output_residual_gpu.producer = self
        if self.input_gpu is None:
            raise _lib.TcbnnError("Error: NULL pointer (input_gpu)")
        return self

    def _residual_dependency(self):
        if self.inject_residual and self.output_residual_gpu is not None:
            return self.output_residual_gpu, self.input_channels * self.filter_height * self.filter_width
        return None, 0

    def _pooled_save_now(self):
        """Store only the 2x2 maximum of the saved residual?  Yes when that is all anybody reads: every hand-out of
        the pointer went to a Conv128 layer that injects it with residual_pool, nobody asked for the full tensor,
        and the kernel that serves this layer can do it."""
        out = self.output_residual_gpu
        if out is None or out.observed or out.other_consumers or not out.pool_consumers or \
                out.handed_out != out.pool_consumers:
            return False
        d = self._desc(decide_pool=False)
        return bool(lib.tcbnn_conv128_pooled_save_supported(C.byref(d)))

    def _desc(self, decide_pool=True):
        rin = self.input_residual_gpu if self.inject_residual else None
        # a source that holds the 2x2 maximum already is injected as it is
        pool_source = self.residual_pool and not _residual_holds_window_maximum(rin)
        pool_out = 2 if decide_pool and self._pooled_save_now() else 0
        return _lib.Conv128Desc(
            self.input_gpu.ptr, self.filter_gpu.ptr, self.bn_gpu.ptr, self.output_gpu.ptr,
            rin.ptr if rin is not None else None,
            self.output_residual_gpu.ptr if self.output_residual_gpu is not None else None,
            self.input_height, self.input_width, self.input_channels, self.filter_height, self.filter_width,
            self.output_channels, self.batch, self.stride_height, self.stride_width, int(self.padding),
            self.pool_height, self.pool_width, int(self.ahead_fc), int(self.save_residual),
            int(self.inject_residual), self.residual_channels, int(pool_source),
            rin.channels if rin is not None else 0, self.variant,
            rin.format if rin is not None else 0,
            self.output_residual_gpu.format if self.output_residual_gpu is not None else 0, pool_out)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_conv128_forward(C.byref(d), _stream_handle(stream)))
        if self.output_residual_gpu is not None:
            self.output_residual_gpu.pooled, self.output_residual_gpu.written = d.output_residual_pool == 2, True

    def kernel_name(self):
        buf = C.create_string_buffer(128)
        d = self._desc()
        check(lib.tcbnn_conv128_kernel_name(C.byref(d), buf, 128))
        return buf.value.decode()

    def release(self):
        self._release_ref_bufs()
        if self.inject_residual:
            _register_residual_consumer(self.input_residual_gpu, self.residual_pool, -1, self)
            self.input_residual_gpu = None
        for b in (self.filter_gpu, self.bn_gpu, self.output_gpu, self.output_residual_gpu):
            if b is not None:
                b.free()
        self.filter_gpu = self.bn_gpu = self.output_gpu = self.output_residual_gpu = None


class Pool128LayerParam:
    """Overlapping OR / max pooling of a packed activation tensor and, optionally, its residual (the
    3x3 stride-2 max-pool of the textbook ResNet wiring).  No counterpart among the reference's layer
    classes: its pooling is a non-overlapping window fused into the convolution (kernel.cuh:811-815)."""

    def __init__(self, name, input_height, input_width, channels, batch, window=3, stride=2, padding=1,
                 pool_residual=False):
        self.name = name
        self.input_height, self.input_width = input_height, input_width
        self.output_channels = channels
        self.batch = batch
        self.window, self.stride, self.padding = window, stride, padding
        self.pool_residual = pool_residual
        self.output_height = self.buf_height = lib.tcbnn_pool_out(input_height, window, stride, padding)
        self.output_width = self.buf_width = lib.tcbnn_pool_out(input_width, window, stride, padding)
        self.input_gpu = self.input_residual_gpu = self.output_gpu = self.output_residual_gpu = None

    def initialize(self, prev_layer_gpu, input_residual_gpu=None):
        if prev_layer_gpu is None:
            raise _lib.TcbnnError("Error: NULL pointer (input_gpu)")
        self.input_gpu = prev_layer_gpu
        self.output_gpu = DeviceBuffer(4 * lib.tcbnn_conv_act_words(self.output_height, self.output_width,
                                                                    self.batch, self.output_channels))
        if self.pool_residual:
            if input_residual_gpu is None:
                raise _lib.TcbnnError("Error: NULL pointer (input_residual_gpu)")
            self.input_residual_gpu = input_residual_gpu
            _register_residual_consumer(input_residual_gpu, False, +1, self)
            # a maximum never exceeds the bound of its operands: same bound, same format
            self.output_residual_gpu = _residual_buffer(self.output_channels, self.output_height, self.output_width,
                                                        self.batch, input_residual_gpu.bound,
                                                        input_residual_gpu.format)
        return self

    def get_output_gpu(self):
        return self.output_gpu

    get_output_residual_gpu = _ConvGeometry.get_output_residual_gpu
    _pooled_save_now = _ConvGeometry._pooled_save_now

    def _residual_dependency(self):
        return (self.output_residual_gpu, 0) if self.pool_residual else (None, 0)

    _want_full_residual = _ConvGeometry._want_full_residual
    download_saved_residual = _ConvGeometry.download_saved_residual

    def _desc(self):
        rin, rout = self.input_residual_gpu, self.output_residual_gpu
        return _lib.Pool128Desc(self.input_gpu.ptr, self.output_gpu.ptr, rin.ptr if rin is not None else None,
                                rout.ptr if rout is not None else None, self.input_height, self.input_width,
                                self.output_channels, self.batch, self.window, self.stride, self.padding,
                                rin.format if rin is not None else 0)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_pool128_forward(C.byref(d), _stream_handle(stream)))

    def kernel_name(self):
        return "pool128_kernel"

    download_packed = _ConvGeometry.download_packed
    download_residual = _ConvGeometry.download_residual
    _is_fc_ready = _ConvGeometry._is_fc_ready

    def release(self):
        if self.pool_residual:
            _register_residual_consumer(self.input_residual_gpu, False, -1, self)
            self.input_residual_gpu = None
        for b in (self.output_gpu, self.output_residual_gpu):
            if b is not None:
                b.free()
        self.output_gpu = self.output_residual_gpu = None


class AvgPoolFcLayerParam:
    """Global average pool over a residual tensor + fp32 fully connected layer (the head of the textbook
    ResNet wiring; the reference's head is a binarized FC layer, imagenet_resnet.cu:320-325).  Weight file
    order: the fp32 weight matrix [channels][out_features], then the bias."""

    def __init__(self, name, input_height, input_width, channels, batch, out_features):
        self.name = name
        self.input_height, self.input_width = input_height, input_width
        self.channels, self.batch, self.out_features = channels, batch, out_features
        self.input_residual_gpu = self.weight_gpu = self.bias_gpu = self.output_gpu = None

    def initialize(self, config_file, input_residual_gpu):
        if input_residual_gpu is None:
            raise _lib.TcbnnError("Error: NULL pointer (input_residual_gpu)")
        self.input_residual_gpu = input_residual_gpu
        _register_residual_consumer(input_residual_gpu, False)
        self.weight = np.array(config_file.launch_array(self.channels * self.out_features), dtype=np.float32)
        self.bias = np.array(config_file.launch_array(self.out_features), dtype=np.float32)
        self.weight_gpu = DeviceBuffer.from_numpy(self.weight)
        self.bias_gpu = DeviceBuffer.from_numpy(self.bias)
        self.output_gpu = DeviceBuffer(4 * self.batch * self.out_features)
        return self

    def get_output_gpu(self):
        return self.output_gpu

    def _desc(self):
        return _lib.AvgPoolFcDesc(self.input_residual_gpu.ptr, self.weight_gpu.ptr, self.bias_gpu.ptr,
                                  self.output_gpu.ptr, self.input_height, self.input_width, self.channels,
                                  self.batch, self.out_features, self.input_residual_gpu.format)

    def forward(self, stream=None):
        d = self._desc()
        check(lib.tcbnn_avgpool_fc_forward(C.byref(d), _stream_handle(stream)))

    def kernel_name(self):
        return "avgpool_fc_kernel"

    def download_output(self):
        return self.output_gpu.to_numpy(np.float32, (self.batch, self.out_features))

    def release(self):
        for b in (self.weight_gpu, self.bias_gpu, self.output_gpu):
            if b is not None:
                b.free()
        self.weight_gpu = self.bias_gpu = self.output_gpu = None
