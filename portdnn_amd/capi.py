"""ctypes binding of the libsnn_hip.so C ABI (include/snn_hip.h).

Pointers are raw device addresses (e.g. ``torch.Tensor.data_ptr()``); the
stream argument is a ``hipStream_t`` handle as an integer (0 = default).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsnn_hip.so")


class SnnHipError(RuntimeError):
    pass


class STATUS:
    OK = 0
    INVALID_ALGORITHM = 1
    INDEX_EXCEEDED = 2
    INSUFFICIENT_WORKSPACE = 3
    ALLOCATION_PROBLEM = 4
    INVALID_PARAMETER = 5
    DEVICE_ERROR = 6


class ALGO:
    NOT_SUPPORTED = 0
    DIRECT = 1
    TILED = 2
    IM2COL = 3
    WINOGRAD = 4
    WINOGRAD_LARGE = 5
    MATMUL = 6


class DIRECTION:
    FORWARD = 0
    INPUT_BACKPROP = 1
    FILTER_BACKPROP = 2


class DTYPE:
    F32 = 0
    F16 = 1


class POOL_OP:
    MAX = 0
    MAX_WITH_NAN = 1
    AVERAGE = 2


class POINTWISE_OP:
    RELU = 0
    TANH = 1
    EXP = 2
    LOG = 3
    FLOOR = 4
    SQRT = 5


class BINARY_OP:
    ADD = 0
    SUB = 1
    MUL = 2
    DIV = 3


def _struct(name, fields, defaults):
    class S(ctypes.Structure):
        _fields_ = [(f, ctypes.c_int) for f in fields]

        def __init__(self, **kw):
            super().__init__()
            for f in fields:
                setattr(self, f, kw.pop(f, defaults.get(f, 0)))
            if kw:
                raise TypeError("unknown fields: %s" % sorted(kw))

        def __repr__(self):
            return name + "(" + ", ".join(
                "%s=%d" % (f, getattr(self, f)) for f in fields) + ")"
    S.__name__ = name
    return S


ConvParams = _struct(
    "ConvParams",
    ["channels", "features", "batch", "in_rows", "in_cols", "window_rows",
     "window_cols", "stride_rows", "stride_cols", "out_rows", "out_cols",
     "pad_rows", "pad_cols", "dilation_rows", "dilation_cols", "groups",
     "input_format", "filter_format", "group_format"],
    {"dilation_rows": 1, "dilation_cols": 1, "groups": 1})

DepthwiseParams = _struct(
    "DepthwiseParams",
    ["channels", "channel_multiplier", "batch", "in_rows", "in_cols",
     "window_rows", "window_cols", "stride_rows", "stride_cols", "out_rows",
     "out_cols", "pad_rows", "pad_cols", "input_format", "filter_format"], {})

PoolParams = _struct(
    "PoolParams",
    ["in_rows", "in_cols", "out_rows", "out_cols", "window_rows",
     "window_cols", "stride_rows", "stride_cols", "batch", "channels",
     "pad_rows", "pad_cols", "input_format"], {})

_P = ctypes.c_void_p
_SZ = ctypes.c_size_t
_I = ctypes.c_int

# name -> argtypes; every symbol include/snn_hip.h declares.
SIGNATURES = {
    "snn_hip_version": [],
    "snn_hip_status_string": [_I],
    "snn_hip_last_error": [],
    "snn_hip_temporary_memory_stats": [
        ctypes.POINTER(ctypes.c_ulonglong), ctypes.POINTER(ctypes.c_ulonglong),
        _I],
    "snn_hip_kernel_timing_enable": [_I],
    "snn_hip_kernel_timing_read": [ctypes.POINTER(ctypes.c_double),
                                   ctypes.POINTER(ctypes.c_int)],
    "snn_hip_conv2d_forward_f32": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_input_backprop_f32": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_filter_backprop_f32": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_forward_f16": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_input_backprop_f16": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_filter_backprop_f16": [_P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_forward_bias_act_f32": [_P, _P, _P, _P, _P, _I, _I, _P,
                                            _SZ, _P],
    "snn_hip_conv2d_deterministic_f32": [_I, _P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_prepare_filter_f32": [_I, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_prepared_f32": [_I, _P, _P, _P, _P, _I, _P, _SZ, _P],
    "snn_hip_conv2d_workspace_size": [_P, _I, _I, ctypes.POINTER(_SZ),
                                      ctypes.POINTER(_SZ)],
    "snn_hip_conv2d_algorithm_supports": [_P, _I, _I],
    "snn_hip_conv2d_default_algorithm": [_P, _I],
    "snn_hip_conv2d_default_algorithm_for": [_P, _I, _I],
    "snn_hip_conv2d_workspace_size_for": [_P, _I, _I, _I, ctypes.POINTER(_SZ),
                                          ctypes.POINTER(_SZ)],
    "snn_hip_depthwise_conv2d_forward_f32": [_P, _P, _P, _P, _P],
    "snn_hip_depthwise_conv2d_input_backprop_f32": [_P, _P, _P, _P, _P],
    "snn_hip_depthwise_conv2d_filter_backprop_f32": [_P, _P, _P, _P, _P],
    "snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32": [_P, _P, _P, _P,
                                                             _P],
    "snn_hip_depthwise_conv2d_forward_f16": [_P, _P, _P, _P, _P],
    "snn_hip_depthwise_conv2d_input_backprop_f16": [_P, _P, _P, _P, _P],
    "snn_hip_depthwise_conv2d_filter_backprop_f16": [_P, _P, _P, _P, _P],
    "snn_hip_pooling_forward_f32": [_P, _P, _P, _I, _P],
    "snn_hip_pooling_forward_f16": [_P, _P, _P, _I, _P],
    "snn_hip_pooling_max_grad_f32": [_P, _P, _P, _P, _P, _I, _P],
    "snn_hip_pooling_avg_grad_f32": [_P, _P, _P, _P],
    "snn_hip_pooling_max_grad_f16": [_P, _P, _P, _P, _P, _I, _P],
    "snn_hip_pooling_avg_grad_f16": [_P, _P, _P, _P],
    "snn_hip_matmul_f32": [_P, _P, _P, _I, _I, _I, _I, _I, _I,
                           ctypes.c_float, _P],
    "snn_hip_matmul_f16": [_P, _P, _P, _I, _I, _I, _I, _I, _I,
                           ctypes.c_float, _P],
    "snn_hip_scale_blend_f32": [_P, _P, ctypes.c_float, ctypes.c_float, _SZ,
                                _P],
    "snn_hip_pointwise_forward_f32": [_P, _P, _SZ, _I, _P],
    "snn_hip_pointwise_forward_f16": [_P, _P, _SZ, _I, _P],
    "snn_hip_pointwise_grad_f32": [_P, _P, _P, _SZ, _I, _P],
    "snn_hip_pointwise_grad_f16": [_P, _P, _P, _SZ, _I, _P],
    "snn_hip_binaryop_f32": [_P, _P, _P, ctypes.POINTER(_I), _I,
                             ctypes.POINTER(_I), _I, _I, _P],
    "snn_hip_binaryop_f16": [_P, _P, _P, ctypes.POINTER(_I), _I,
                             ctypes.POINTER(_I), _I, _I, _P],
}

_lib = None


def lib_path():
    return _LIB_PATH


def lib():
    """Loads libsnn_hip.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise SnnHipError(
                "libsnn_hip.so is missing: build it with "
                "`python -m portdnn_amd.build` (there is no CPU fallback)")
        # torch bundles its own libamdhip64; load it first so that this
        # library binds to the same HIP runtime the tensors live in (two
        # runtimes in one process do not see each other's devices).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(_LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = argtypes
            fn.restype = _I
        L.snn_hip_status_string.restype = ctypes.c_char_p
        L.snn_hip_last_error.restype = ctypes.c_char_p
        _lib = L
    return _lib


def status_string(code):
    return lib().snn_hip_status_string(int(code)).decode()


def check(code):
    """Raises SnnHipError for a non-OK status."""
    if code != STATUS.OK:
        raise SnnHipError("%s (%d) %s" % (
            status_string(code), code, lib().snn_hip_last_error().decode()))
    return code
