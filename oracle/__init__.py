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
