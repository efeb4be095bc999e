"""ctypes front-end of the CPU oracle (oracle.c).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg; the shipped package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with gcc (a few seconds)."""
    if force:
        subprocess.check_call(["make", "-s", "-C", _HERE, "clean"])
    subprocess.check_call(["make", "-s", "-C", _HERE, "CC=gcc"])


class Params(ctypes.Structure):
    """Mirror of struct oracle_params."""
    _fields_ = [(n, ctypes.c_int) for n in (
        "channels", "features", "batch", "in_rows", "in_cols", "window_rows",
        "window_cols", "stride_rows", "stride_cols", "out_rows", "out_cols",
        "pad_rows", "pad_cols")]


_lib = None
_FP = ctypes.POINTER(ctypes.c_float)
_PP = ctypes.POINTER(Params)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        L = _lib
        L.oracle_calculate_padding.argtypes = [ctypes.c_int] * 4 + [
            ctypes.POINTER(ctypes.c_int)] * 2
        for name in ("conv2d_forward", "conv2d_input_backprop",
                     "conv2d_filter_backprop", "depthwise_forward",
                     "depthwise_input_backprop", "depthwise_filter_backprop"):
            getattr(L, "oracle_" + name).argtypes = [_FP, _FP, _FP, _PP,
                                                     ctypes.c_int]
        L.oracle_conv2d_winograd_forward.argtypes = [_FP, _FP, _FP, _PP,
                                                     ctypes.c_int,
                                                     ctypes.c_int]
        L.oracle_conv2d_winograd_forward.restype = ctypes.c_int
        L.oracle_conv2d_tiled_forward.argtypes = [_FP, _FP, _FP, _PP,
                                                  ctypes.c_int]
        L.oracle_conv2d_tiled_forward.restype = ctypes.c_int
        L.oracle_pool_max_forward.argtypes = [_FP, _FP, _PP, ctypes.c_int]
        L.oracle_pool_avg_forward.argtypes = [_FP, _FP, _PP, ctypes.c_int]
        L.oracle_pool_max_grad.argtypes = [_FP, _FP, _FP, _FP, _PP,
                                           ctypes.c_int]
        L.oracle_pool_avg_grad.argtypes = [_FP, _FP, _PP, ctypes.c_int]
        L.oracle_matmul.argtypes = [_FP, _FP, _FP] + [ctypes.c_int] * 6 + [
            ctypes.c_float, ctypes.c_int]
        L.oracle_pointwise_forward.argtypes = [ctypes.c_int, _FP, _FP,
                                               ctypes.c_long]
        L.oracle_pointwise_grad.argtypes = [ctypes.c_int, _FP, _FP, _FP,
                                            ctypes.c_long]
        _IP = ctypes.POINTER(ctypes.c_int)
        L.oracle_binaryop.argtypes = [ctypes.c_int, _FP, _FP, _FP, _IP,
                                      ctypes.c_int, _IP, ctypes.c_int]
        L.oracle_set_threads.argtypes = [ctypes.c_int]
        L.oracle_set_threads.restype = ctypes.c_int
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_FP)


def calculate_padding(inp, window, stride, same):
    pad, out = ctypes.c_int(), ctypes.c_int()
    lib().oracle_calculate_padding(inp, window, stride, int(bool(same)),
                                   ctypes.byref(pad), ctypes.byref(out))
    return pad.value, out.value


def make_params(batch, in_rows, in_cols, channels, features, window, stride,
                same, window_cols=None, stride_cols=None):
    """Shape record with out_* / pad_* filled in the way
    helpers::add_padding_to does (include/portdnn/helpers/padding.h:80-92)."""
    wr, wc = window, window if window_cols is None else window_cols
    sr, sc = stride, stride if stride_cols is None else stride_cols
    pr, orows = calculate_padding(in_rows, wr, sr, same)
    pc, ocols = calculate_padding(in_cols, wc, sc, same)
    return Params(channels, features, batch, in_rows, in_cols, wr, wc, sr, sc,
                  orows, ocols, pr, pc)


def set_threads(n):
    return lib().oracle_set_threads(int(n))


def _three(name, a, b, out_size, p, acc64):
    a, ap = _f(a)
    b, bp = _f(b)
    out = np.empty(out_size, dtype=np.float32)
    getattr(lib(), "oracle_" + name)(ap, bp, out.ctypes.data_as(_FP),
                                     ctypes.byref(p), int(acc64))
    return out


def conv2d_forward(x, w, p, acc64=True):
    n = p.batch * p.out_rows * p.out_cols * p.features
    return _three("conv2d_forward", x, w, n, p, acc64)


def conv2d_input_backprop(dy, w, p, acc64=True):
    n = p.batch * p.in_rows * p.in_cols * p.channels
    return _three("conv2d_input_backprop", dy, w, n, p, acc64)


def conv2d_filter_backprop(x, dy, p, acc64=True):
    n = p.window_rows * p.window_cols * p.channels * p.features
    return _three("conv2d_filter_backprop", x, dy, n, p, acc64)


def conv2d_winograd_forward(x, w, p, tile, acc64=False):
    """Forward convolution by Winograd F(tile x tile, 3x3), tile 2 or 4, every
    stage in float (or double): the fp32 behaviour of the algorithm."""
    x, xp = _f(x)
    w, wp = _f(w)
    out = np.empty(p.batch * p.out_rows * p.out_cols * p.features,
                   dtype=np.float32)
    rc = lib().oracle_conv2d_winograd_forward(
        xp, wp, out.ctypes.data_as(_FP), ctypes.byref(p), int(tile),
        int(acc64))
    if rc != 0:
        raise ValueError("Winograd restatement: 3x3 stride 1, tile 2 or 4")
    return out


def conv2d_tiled_forward(x, w, p, threads=0):
    x, xp = _f(x)
    w, wp = _f(w)
    out = np.empty(p.batch * p.out_rows * p.out_cols * p.features,
                   dtype=np.float32)
    rc = lib().oracle_conv2d_tiled_forward(xp, wp, out.ctypes.data_as(_FP),
                                           ctypes.byref(p), int(threads))
    if rc != 0:
        raise ValueError("shape not covered by the reference tiled tile list")
    return out


def depthwise_forward(x, w, p, acc64=True):
    n = p.batch * p.out_rows * p.out_cols * p.channels * p.features
    return _three("depthwise_forward", x, w, n, p, acc64)


def depthwise_input_backprop(dy, w, p, acc64=True):
    n = p.batch * p.in_rows * p.in_cols * p.channels
    return _three("depthwise_input_backprop", dy, w, n, p, acc64)


def depthwise_filter_backprop(x, dy, p, acc64=True):
    n = p.window_rows * p.window_cols * p.channels * p.features
    return _three("depthwise_filter_backprop", x, dy, n, p, acc64)


def pool_max_forward(x, p, nan_mode=False):
    x, xp = _f(x)
    out = np.empty(p.batch * p.out_rows * p.out_cols * p.channels,
                   dtype=np.float32)
    lib().oracle_pool_max_forward(xp, out.ctypes.data_as(_FP), ctypes.byref(p),
                                  int(nan_mode))
    return out


def pool_avg_forward(x, p, acc64=True):
    x, xp = _f(x)
    out = np.empty(p.batch * p.out_rows * p.out_cols * p.channels,
                   dtype=np.float32)
    lib().oracle_pool_avg_forward(xp, out.ctypes.data_as(_FP), ctypes.byref(p),
                                  int(acc64))
    return out


def pool_max_grad(x, y, dy, p, nan_mode=False):
    x, xp = _f(x)
    y, yp = _f(y)
    dy, dyp = _f(dy)
    dx = np.empty(p.batch * p.in_rows * p.in_cols * p.channels,
                  dtype=np.float32)
    lib().oracle_pool_max_grad(xp, yp, dyp, dx.ctypes.data_as(_FP),
                               ctypes.byref(p), int(nan_mode))
    return dx


def pool_avg_grad(dy, p, acc64=True):
    dy, dyp = _f(dy)
    dx = np.empty(p.batch * p.in_rows * p.in_cols * p.channels,
                  dtype=np.float32)
    lib().oracle_pool_avg_grad(dyp, dx.ctypes.data_as(_FP), ctypes.byref(p),
                               int(acc64))
    return dx


def matmul(a, b, batches, m, k, n, trans_a=False, trans_b=False, beta=0.0,
           c=None, acc64=True):
    a, ap = _f(a)
    b, bp = _f(b)
    out = (np.zeros(batches * m * n, dtype=np.float32) if c is None else
           np.array(c, dtype=np.float32).reshape(-1).copy())
    lib().oracle_matmul(ap, bp, out.ctypes.data_as(_FP), batches, m, k, n,
                        int(trans_a), int(trans_b), float(beta), int(acc64))
    return out


def iota(size, max_val):
    """1, 2, ..., max_val, 1, 2, ...  (test/gen/iota_initialised_data.h:74-79;
    max_val < 1 means no wrap)."""
    idx = np.arange(size, dtype=np.int64)
    if max_val >= 1:
        idx = idx % int(max_val)
    return (idx + 1).astype(np.float32)


POINTWISE_OPS = {"relu": 0, "tanh": 1, "exp": 2, "log": 3, "floor": 4,
                 "sqrt": 5}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def pointwise_forward(op, x):
    x, xp = _f(x)
    out = np.empty_like(x)
    rc = lib().oracle_pointwise_forward(POINTWISE_OPS[op], xp,
                                        out.ctypes.data_as(_FP), x.size)
    assert rc == 0, op
    return out


def pointwise_grad(op, val, err):
    """`val` is the forward output (the forward input for log)."""
    val, vp = _f(val)
    err, ep = _f(err)
    out = np.empty_like(val)
    rc = lib().oracle_pointwise_grad(POINTWISE_OPS[op], vp, ep,
                                     out.ctypes.data_as(_FP), val.size)
    assert rc == 0, op
    return out


def binaryop_out_dims(lhs_dims, rhs_dims):
    """include/portdnn/internal/binaryop/launch.h:40-62; None when the shapes
    do not broadcast."""
    n = max(len(lhs_dims), len(rhs_dims), 1)
    l = [1] * (n - len(lhs_dims)) + list(lhs_dims)
    r = [1] * (n - len(rhs_dims)) + list(rhs_dims)
    out = []
    for a, b in zip(l, r):
        if a != b and a != 1 and b != 1:
            return None
        out.append(max(a, b))
    return out


def binaryop(op, lhs, rhs, lhs_dims, rhs_dims):
    lhs, lp = _f(lhs)
    rhs, rp = _f(rhs)
    out_dims = binaryop_out_dims(lhs_dims, rhs_dims)
    assert out_dims is not None
    out = np.empty(int(np.prod(out_dims)), dtype=np.float32)
    ld = (ctypes.c_int * max(len(lhs_dims), 1))(*lhs_dims)
    rd = (ctypes.c_int * max(len(rhs_dims), 1))(*rhs_dims)
    rc = lib().oracle_binaryop(BINARY_OPS[op], lp, rp,
                               out.ctypes.data_as(_FP), ld, len(lhs_dims), rd,
                               len(rhs_dims))
    assert rc == 0, (op, lhs_dims, rhs_dims)
    return out


def iota_signed(size):
    """-ceil(size / 2), ..., size - 1 - ceil(size / 2)
    (test/gen/iota_initialised_data.h:89-97)."""
    half = (size + 1) // 2
    return (np.arange(size, dtype=np.int64) - half).astype(np.float32)
