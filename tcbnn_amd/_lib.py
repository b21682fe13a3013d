"""ctypes bindings of libtcbnn_hip.so (the C ABI in include/tcbnn_hip.h) and of the
few HIP runtime calls the Python host mirror needs (device memory, copies, events).

There is no CPU fallback: importing this module without the built library, or
calling into it without a GPU, raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtcbnn_hip.so")


class TcbnnError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise TcbnnError(
            "libtcbnn_hip.so is not built (%s missing): run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C tcbnn_amd/csrc`" % LIB_PATH)
    return C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)


lib = _load()

c_void_p, c_int, c_size_t, c_float_p = C.c_void_p, C.c_int, C.c_size_t, C.c_void_p


class In128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("output", c_void_p), ("input_height", c_int),
                ("input_width", c_int)]


class Fc128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("weight", c_void_p), ("bn", c_void_p), ("output", c_void_p),
                ("input_height", c_int), ("input_width", c_int), ("weight_width", c_int),
                ("variant", c_int), ("workspace", c_void_p), ("workspace_words", c_size_t)]


class Out128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("weight", c_void_p), ("bn_scale", c_void_p),
                ("bn_bias", c_void_p), ("output", c_void_p), ("input_height", c_int),
                ("input_width", c_int), ("weight_width", c_int), ("variant", c_int)]


class InConv128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("filter", c_void_p), ("bn", c_void_p), ("output", c_void_p),
                ("output_residual", c_void_p), ("input_height", c_int), ("input_width", c_int),
                ("input_channels", c_int), ("filter_height", c_int), ("filter_width", c_int),
                ("output_channels", c_int), ("batch", c_int), ("stride_height", c_int),
                ("stride_width", c_int), ("padding", c_int), ("pool_height", c_int),
                ("pool_width", c_int), ("save_residual", c_int), ("residual_format", c_int),
                ("input_layout", c_int)]


class Conv128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("filter", c_void_p), ("bn", c_void_p), ("output", c_void_p),
                ("input_residual", c_void_p), ("output_residual", c_void_p),
                ("input_height", c_int), ("input_width", c_int), ("input_channels", c_int),
                ("filter_height", c_int), ("filter_width", c_int), ("output_channels", c_int),
                ("batch", c_int), ("stride_height", c_int), ("stride_width", c_int),
                ("padding", c_int), ("pool_height", c_int), ("pool_width", c_int),
                ("ahead_fc", c_int), ("save_residual", c_int), ("inject_residual", c_int),
                ("residual_channels", c_int), ("residual_pool", c_int),
                ("input_residual_channels", c_int), ("variant", c_int),
                ("input_residual_format", c_int), ("output_residual_format", c_int),
                ("output_residual_pool", c_int)]


class Pool128Desc(C.Structure):
    _fields_ = [("input", c_void_p), ("output", c_void_p), ("input_residual", c_void_p),
                ("output_residual", c_void_p), ("input_height", c_int), ("input_width", c_int),
                ("channels", c_int), ("batch", c_int), ("window", c_int), ("stride", c_int),
                ("padding", c_int), ("residual_format", c_int)]


class AvgPoolFcDesc(C.Structure):
    _fields_ = [("input_residual", c_void_p), ("weight", c_void_p), ("bias", c_void_p), ("output", c_void_p),
                ("input_height", c_int), ("input_width", c_int), ("channels", c_int), ("batch", c_int),
                ("out_features", c_int), ("residual_format", c_int)]


# name -> (restype, argtypes); the complete list of symbols include/tcbnn_hip.h declares.
ABI = {
    "tcbnn_abi_version": (c_int, []),
    "tcbnn_last_error": (C.c_char_p, []),
    "tcbnn_set_default_variant": (c_int, [c_int]),
    "tcbnn_get_default_variant": (c_int, []),
    "tcbnn_conv_pad": (c_int, [c_int] * 4),
    "tcbnn_conv_out": (c_int, [c_int] * 5),
    "tcbnn_pool_out": (c_int, [c_int] * 4),
    "tcbnn_pool128_forward": (c_int, [C.POINTER(Pool128Desc), c_void_p]),
    "tcbnn_avgpool_fc_forward": (c_int, [C.POINTER(AvgPoolFcDesc), c_void_p]),
    "tcbnn_fc_act_words": (c_size_t, [c_int] * 2),
    "tcbnn_conv_act_words": (c_size_t, [c_int] * 4),
    "tcbnn_fc_weight_words": (c_size_t, [c_int] * 2),
    "tcbnn_conv_filter_words": (c_size_t, [c_int] * 4),
    "tcbnn_inconv_filter_words": (c_size_t, [c_int] * 4),
    "tcbnn_residual_bytes": (c_size_t, [c_int] * 5),
    "tcbnn_inconv_residual_bound": (c_int, [c_int, c_int, C.c_float]),
    "tcbnn_host_abs_max": (C.c_float, [c_void_p, c_size_t]),
    "tcbnn_conv_residual_bound": (c_int, [c_int] * 4),
    "tcbnn_residual_format_for_bound": (c_int, [c_int]),
    "tcbnn_residual_format_narrowest": (c_int, [c_int, c_int]),
    "tcbnn_inconv_residual_bound_of_input": (c_int, [c_void_p] + [c_int] * 8),
    "tcbnn_pack_fc_weight": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tcbnn_pack_conv_filter": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_pack_inconv_filter": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_pack_rows": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_pack_cols": (c_int, [c_void_p, c_void_p] + [c_int] * 3 + [c_void_p]),
    "tcbnn_pack_conv_input_nhwc": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_in128_forward": (c_int, [C.POINTER(In128Desc), c_void_p]),
    "tcbnn_fc128_forward": (c_int, [C.POINTER(Fc128Desc), c_void_p]),
    "tcbnn_fc128_forward_static_scratch": (c_int, [C.POINTER(Fc128Desc), c_void_p]),
    "tcbnn_out128_forward": (c_int, [C.POINTER(Out128Desc), c_void_p]),
    "tcbnn_inconv128_forward": (c_int, [C.POINTER(InConv128Desc), c_void_p]),
    "tcbnn_inconv_packed_input_floats": (c_size_t, [c_int] * 8),
    "tcbnn_inconv_pack_input": (c_int, [c_void_p, c_void_p] + [c_int] * 8 + [c_void_p]),
    "tcbnn_conv128_forward": (c_int, [C.POINTER(Conv128Desc), c_void_p]),
    "tcbnn_conv128_pooled_save_supported": (c_int, [C.POINTER(Conv128Desc)]),
    "tcbnn_conv128_kernel_name": (c_int, [C.POINTER(Conv128Desc), C.c_char_p, c_size_t]),
    "tcbnn_fc128_kernel_name": (c_int, [C.POINTER(Fc128Desc), C.c_char_p, c_size_t]),
    "tcbnn_out128_kernel_name": (c_int, [C.POINTER(Out128Desc), C.c_char_p, c_size_t]),
    "tcbnn_inconv128_kernel_name": (c_int, [C.POINTER(InConv128Desc), C.c_char_p, c_size_t]),
    "tcbnn_shader_clock_probe": (c_int, [c_void_p, c_int, C.POINTER(c_int), c_void_p]),
    "tcbnn_bmm": (c_int, [c_void_p] * 3 + [c_int] * 4 + [c_void_p]),
    "tcbnn_bconv": (c_int, [c_void_p] * 3 + [c_int] * 14 + [c_void_p]),
    "tcbnn_unpack_fc_output": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tcbnn_unpack_conv_output": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_fc_to_reference_fmt": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tcbnn_fc_from_reference_fmt": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "tcbnn_conv_to_reference_fmt": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_conv_from_reference_fmt": (c_int, [c_void_p, c_void_p] + [c_int] * 4 + [c_void_p]),
    "tcbnn_residual_to_reference": (c_int, [c_void_p, c_void_p] + [c_int] * 5 + [c_void_p]),
    "tcbnn_residual_from_reference": (c_int, [c_void_p, c_void_p] + [c_int] * 5 + [c_void_p]),
}

for _name, (_res, _args) in ABI.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args

VARIANT_AUTO, VARIANT_POPC, VARIANT_MFMA_I8, VARIANT_MFMA_F4 = 0, 1, 2, 3
VARIANTS = {"auto": 0, "popc": 1, "mfma_i8": 2, "mfma_f4": 3}
RES_I32, RES_I16, RES_I12 = 0, 1, 2
INCONV_INPUT_NCHW, INCONV_INPUT_PACKED = 0, 1
INT32_MAX = 2 ** 31 - 1


def check(rc):
    """Raise TcbnnError with the library's message for a non-zero return code."""
    if rc != 0:
        raise TcbnnError("tcbnn error %d: %s" % (rc, lib.tcbnn_last_error().decode()))


# --------------------------------------------------------------------------- HIP runtime
# The runtime the library itself is linked against (resolved by soname, so this is the
# already-loaded copy, not a second runtime).
_hip = C.CDLL("libamdhip64.so", mode=C.RTLD_GLOBAL)
_hip.hipGetErrorString.restype = C.c_char_p
_hip.hipGetErrorString.argtypes = [c_int]
_hip.hipMalloc.argtypes = [C.POINTER(c_void_p), c_size_t]
_hip.hipFree.argtypes = [c_void_p]
_hip.hipMemcpy.argtypes = [c_void_p, c_void_p, c_size_t, c_int]
_hip.hipMemset.argtypes = [c_void_p, c_int, c_size_t]
_hip.hipMemsetAsync.argtypes = [c_void_p, c_int, c_size_t, c_void_p]
_hip.hipGetDeviceCount.argtypes = [C.POINTER(c_int)]
_hip.hipSetDevice.argtypes = [c_int]
_hip.hipStreamCreate.argtypes = [C.POINTER(c_void_p)]
_hip.hipStreamDestroy.argtypes = [c_void_p]
_hip.hipStreamSynchronize.argtypes = [c_void_p]
_hip.hipEventCreate.argtypes = [C.POINTER(c_void_p)]
_hip.hipEventDestroy.argtypes = [c_void_p]
_hip.hipEventRecord.argtypes = [c_void_p, c_void_p]
_hip.hipEventSynchronize.argtypes = [c_void_p]
_hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), c_void_p, c_void_p]
_hip.hipStreamBeginCapture.argtypes = [c_void_p, c_int]
_hip.hipStreamEndCapture.argtypes = [c_void_p, C.POINTER(c_void_p)]
_hip.hipGraphInstantiate.argtypes = [C.POINTER(c_void_p), c_void_p, c_void_p, c_void_p, c_size_t]
_hip.hipGraphLaunch.argtypes = [c_void_p, c_void_p]
_hip.hipGraphExecDestroy.argtypes = [c_void_p]
_hip.hipGraphDestroy.argtypes = [c_void_p]

H2D, D2H, D2D = 1, 2, 3


def hip_check(rc, what="hip call"):
    if rc != 0:
        raise TcbnnError("%s failed: %s" % (what, _hip.hipGetErrorString(rc).decode()))


def device_count():
    n = c_int(0)
    rc = _hip.hipGetDeviceCount(C.byref(n))
    return n.value if rc == 0 else 0


def set_device(i):
    hip_check(_hip.hipSetDevice(i), "hipSetDevice")


def device_synchronize():
    hip_check(_hip.hipDeviceSynchronize(), "hipDeviceSynchronize")


hip = _hip
