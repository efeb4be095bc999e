"""Torch-tensor conveniences over the C ABI, used by the tests and bench.py.

torch is plumbing here (device memory and the current HIP stream); every
computation happens in libsnn_hip.so.  There is no fallback path.
"""
import ctypes

import torch

from . import capi
from .capi import ALGO, BINARY_OP, DIRECTION, POINTWISE_OP, POOL_OP, STATUS, \
    ConvParams, DepthwiseParams, PoolParams


def calculate_padding(inp, window, stride, same):
    """helpers::calculate_padding (include/portdnn/helpers/padding.h:51-69):
    returns (padding, output)."""
    if same:
        out = (inp + stride - 1) // stride
        needed = (out - 1) * stride + window - inp
        return int(needed / 2), out  # C++ integer division truncates
    num = inp - window + 1
    q = int(num / stride)
    return 0, (q if num < 0 else q + (1 if num % stride else 0))


def add_padding_to(params, same):
    """helpers::add_padding_to (include/portdnn/helpers/padding.h:80-92)."""
    params.pad_rows, params.out_rows = calculate_padding(
        params.in_rows, params.window_rows, params.stride_rows, same)
    params.pad_cols, params.out_cols = calculate_padding(
        params.in_cols, params.window_cols, params.stride_cols, same)
    return params


def conv_params(batch, in_rows, in_cols, channels, features, window, stride,
                same):
    return add_padding_to(ConvParams(
        channels=channels, features=features, batch=batch, in_rows=in_rows,
        in_cols=in_cols, window_rows=window, window_cols=window,
        stride_rows=stride, stride_cols=stride), same)


def depthwise_params(batch, in_rows, in_cols, channels, multiplier, window,
                     stride, same):
    return add_padding_to(DepthwiseParams(
        channels=channels, channel_multiplier=multiplier, batch=batch,
        in_rows=in_rows, in_cols=in_cols, window_rows=window,
        window_cols=window, stride_rows=stride, stride_cols=stride), same)


def pool_params(batch, in_rows, in_cols, channels, window, stride, same):
    return add_padding_to(PoolParams(
        in_rows=in_rows, in_cols=in_cols, window_rows=window,
        window_cols=window, stride_rows=stride, stride_cols=stride,
        batch=batch, channels=channels), same)


def conv_sizes(p, direction):
    """(input, filter, output) element counts, conv2d/sizes.h:166-179."""
    x = p.batch * p.in_rows * p.in_cols * p.channels
    w = p.window_rows * p.window_cols * p.channels * p.features
    y = p.batch * p.out_rows * p.out_cols * p.features
    if direction == DIRECTION.FORWARD:
        return x, w, y
    if direction == DIRECTION.INPUT_BACKPROP:
        return y, w, x
    return x, y, w


def conv_flops(p, direction):
    """bench/conv2d/base_convolution_fixture.h:81-109."""
    if direction == DIRECTION.FORWARD:
        pix = p.batch * p.out_rows * p.out_cols
    else:
        pix = p.batch * p.in_rows * p.in_cols
    return 2 * pix * p.window_rows * p.window_cols * p.channels * p.features


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def workspace_size(p, direction, algorithm, dtype=None):
    """(required, recommended) elements; with a capi.DTYPE the element type's
    own answer (snn_hip_conv2d_workspace_size_for)."""
    req, rec = ctypes.c_size_t(), ctypes.c_size_t()
    if dtype is None:
        capi.check(capi.lib().snn_hip_conv2d_workspace_size(
            ctypes.byref(p), direction, algorithm, ctypes.byref(req),
            ctypes.byref(rec)))
    else:
        capi.check(capi.lib().snn_hip_conv2d_workspace_size_for(
            ctypes.byref(p), direction, algorithm, dtype, ctypes.byref(req),
            ctypes.byref(rec)))
    return req.value, rec.value


def default_algorithm(p, direction, dtype=None):
    """The library's default selector's choice (for a capi.DTYPE when given)."""
    if dtype is None:
        return capi.lib().snn_hip_conv2d_default_algorithm(ctypes.byref(p),
                                                           direction)
    return capi.lib().snn_hip_conv2d_default_algorithm_for(
        ctypes.byref(p), direction, dtype)


_CONV_FN = {
    (DIRECTION.FORWARD, torch.float32): "snn_hip_conv2d_forward_f32",
    (DIRECTION.INPUT_BACKPROP, torch.float32):
        "snn_hip_conv2d_input_backprop_f32",
    (DIRECTION.FILTER_BACKPROP, torch.float32):
        "snn_hip_conv2d_filter_backprop_f32",
    (DIRECTION.FORWARD, torch.float16): "snn_hip_conv2d_forward_f16",
    (DIRECTION.INPUT_BACKPROP, torch.float16):
        "snn_hip_conv2d_input_backprop_f16",
    (DIRECTION.FILTER_BACKPROP, torch.float16):
        "snn_hip_conv2d_filter_backprop_f16",
}


def conv2d_raw(inp, fil, out, p, direction, algorithm, workspace=None):
    """Calls the entry point and returns its status code (no exception)."""
    fn = getattr(capi.lib(), _CONV_FN[(direction, inp.dtype)])
    ws_elems = 0 if workspace is None else workspace.numel()
    return fn(_ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p), algorithm,
              _ptr(workspace), ws_elems, _stream())


def conv2d(inp, fil, p, direction=DIRECTION.FORWARD, algorithm=ALGO.DIRECT,
           workspace=None, out=None):
    """inp / fil are flat or shaped device tensors with the operand roles of
    include/snn_hip.h; returns the flat output tensor."""
    n_in, n_fil, n_out = conv_sizes(p, direction)
    assert inp.numel() == n_in and fil.numel() == n_fil, (inp.shape, fil.shape)
    assert inp.is_contiguous() and fil.is_contiguous()
    if out is None:
        out = torch.empty(n_out, dtype=inp.dtype, device=inp.device)
    if (workspace is None and inp.dtype == torch.float32 and
            algorithm in (ALGO.WINOGRAD, ALGO.WINOGRAD_LARGE)):
        _, rec = workspace_size(p, direction, algorithm)
        workspace = torch.empty(rec, dtype=inp.dtype, device=inp.device)
    capi.check(conv2d_raw(inp, fil, out, p, direction, algorithm, workspace))
    return out


def _bind(fn, *cargs):
    """A zero-argument callable that makes one C ABI call with arguments
    converted once: timing loops over kernels of a few microseconds would
    otherwise measure the per-call conversions of the wrappers above (6-7 us
    against 2 for the call itself).  The stream is the one current now."""
    def call():
        code = fn(*cargs)
        if code:
            capi.check(code)
    return call


def conv2d_bound(inp, fil, out, p, direction, algorithm, workspace=None):
    """conv2d with everything fixed: returns the callable that launches it."""
    n_in, n_fil, n_out = conv_sizes(p, direction)
    assert (inp.numel(), fil.numel(), out.numel()) == (n_in, n_fil, n_out)
    assert inp.is_contiguous() and fil.is_contiguous() and out.is_contiguous()
    fn = getattr(capi.lib(), _CONV_FN[(direction, inp.dtype)])
    return _bind(fn, _ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p),
                 algorithm, _ptr(workspace),
                 0 if workspace is None else workspace.numel(),
                 ctypes.c_void_p(_stream()))


def conv2d_prepared_bound(inp, fil, out, p, direction, algorithm, workspace):
    """conv2d_prepared with everything fixed."""
    return _bind(capi.lib().snn_hip_conv2d_prepared_f32, direction, _ptr(inp),
                 _ptr(fil), _ptr(out), ctypes.byref(p), algorithm,
                 _ptr(workspace),
                 0 if workspace is None else workspace.numel(),
                 ctypes.c_void_p(_stream()))


def conv2d_prepare_filter(fil, p, direction, algorithm, workspace):
    """snn_hip_conv2d_prepare_filter_f32: what the launch derives from the
    filter alone goes into `workspace`."""
    capi.check(capi.lib().snn_hip_conv2d_prepare_filter_f32(
        direction, _ptr(fil), ctypes.byref(p), algorithm, _ptr(workspace),
        0 if workspace is None else workspace.numel(), _stream()))


def conv2d_prepared(inp, fil, p, direction, algorithm, workspace, out=None):
    """snn_hip_conv2d_prepared_f32: the launch that trusts a prepared
    workspace."""
    _, _, n_out = conv_sizes(p, direction)
    if out is None:
        out = torch.empty(n_out, dtype=inp.dtype, device=inp.device)
    capi.check(capi.lib().snn_hip_conv2d_prepared_f32(
        direction, _ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p), algorithm,
        _ptr(workspace), 0 if workspace is None else workspace.numel(),
        _stream()))
    return out


def conv2d_deterministic(inp, fil, p, direction, algorithm, workspace=None,
                         out=None):
    """snn_hip_conv2d_deterministic_f32: fixed order of additions."""
    n_in, n_fil, n_out = conv_sizes(p, direction)
    assert inp.numel() == n_in and fil.numel() == n_fil
    if out is None:
        out = torch.empty(n_out, dtype=inp.dtype, device=inp.device)
    if workspace is None:
        _, rec = workspace_size(p, direction, algorithm)
        if rec:
            workspace = torch.empty(rec, dtype=inp.dtype, device=inp.device)
    capi.check(capi.lib().snn_hip_conv2d_deterministic_f32(
        direction, _ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p), algorithm,
        _ptr(workspace), 0 if workspace is None else workspace.numel(),
        _stream()))
    return out


def conv2d_bias_act(inp, fil, bias, p, algorithm, relu=True, workspace=None,
                    out=None):
    """snn_hip_conv2d_forward_bias_act_f32: act(conv(inp, fil) + bias)."""
    _, _, n_out = conv_sizes(p, DIRECTION.FORWARD)
    if out is None:
        out = torch.empty(n_out, dtype=inp.dtype, device=inp.device)
    if workspace is None and algorithm in (ALGO.WINOGRAD, ALGO.WINOGRAD_LARGE):
        _, rec = workspace_size(p, DIRECTION.FORWARD, algorithm)
        workspace = torch.empty(rec, dtype=inp.dtype, device=inp.device)
    ws_elems = 0 if workspace is None else workspace.numel()
    capi.check(capi.lib().snn_hip_conv2d_forward_bias_act_f32(
        _ptr(inp), _ptr(fil), _ptr(bias), _ptr(out), ctypes.byref(p),
        algorithm, 1 if relu else 0, _ptr(workspace), ws_elems, _stream()))
    return out


_DW_FN = {
    (DIRECTION.FORWARD, torch.float32): "snn_hip_depthwise_conv2d_forward_f32",
    (DIRECTION.INPUT_BACKPROP, torch.float32):
        "snn_hip_depthwise_conv2d_input_backprop_f32",
    (DIRECTION.FILTER_BACKPROP, torch.float32):
        "snn_hip_depthwise_conv2d_filter_backprop_f32",
    (DIRECTION.FORWARD, torch.float16): "snn_hip_depthwise_conv2d_forward_f16",
    (DIRECTION.INPUT_BACKPROP, torch.float16):
        "snn_hip_depthwise_conv2d_input_backprop_f16",
    (DIRECTION.FILTER_BACKPROP, torch.float16):
        "snn_hip_depthwise_conv2d_filter_backprop_f16",
}


def depthwise_sizes(p, direction):
    x = p.batch * p.in_rows * p.in_cols * p.channels
    w = p.window_rows * p.window_cols * p.channels * p.channel_multiplier
    y = p.batch * p.out_rows * p.out_cols * p.channels * p.channel_multiplier
    if direction == DIRECTION.FORWARD:
        return x, w, y
    if direction == DIRECTION.INPUT_BACKPROP:
        return y, w, x
    return x, y, w


def depthwise_conv2d(inp, fil, p, direction=DIRECTION.FORWARD, out=None):
    n_in, n_fil, n_out = depthwise_sizes(p, direction)
    assert inp.numel() == n_in and fil.numel() == n_fil
    if out is None:
        out = torch.empty(n_out, dtype=inp.dtype, device=inp.device)
    fn = getattr(capi.lib(), _DW_FN[(direction, inp.dtype)])
    capi.check(fn(_ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p), _stream()))
    return out


def depthwise_conv2d_bound(inp, fil, out, p, direction=DIRECTION.FORWARD):
    """depthwise_conv2d with everything fixed (see _bind)."""
    n_in, n_fil, n_out = depthwise_sizes(p, direction)
    assert (inp.numel(), fil.numel(), out.numel()) == (n_in, n_fil, n_out)
    fn = getattr(capi.lib(), _DW_FN[(direction, inp.dtype)])
    return _bind(fn, _ptr(inp), _ptr(fil), _ptr(out), ctypes.byref(p),
                 ctypes.c_void_p(_stream()))


def pooling_forward_bound(inp, out, p, op):
    """pooling_forward with everything fixed (see _bind)."""
    assert inp.numel() == p.batch * p.in_rows * p.in_cols * p.channels
    assert out.numel() == p.batch * p.out_rows * p.out_cols * p.channels
    name = ("snn_hip_pooling_forward_f32" if inp.dtype == torch.float32 else
            "snn_hip_pooling_forward_f16")
    return _bind(getattr(capi.lib(), name), _ptr(inp), _ptr(out),
                 ctypes.byref(p), op, ctypes.c_void_p(_stream()))


def pooling_forward(inp, p, op, out=None):
    assert inp.numel() == p.batch * p.in_rows * p.in_cols * p.channels
    if out is None:
        out = torch.empty(p.batch * p.out_rows * p.out_cols * p.channels,
                          dtype=inp.dtype, device=inp.device)
    name = ("snn_hip_pooling_forward_f32" if inp.dtype == torch.float32 else
            "snn_hip_pooling_forward_f16")
    capi.check(getattr(capi.lib(), name)(_ptr(inp), _ptr(out), ctypes.byref(p),
                                         op, _stream()))
    return out


def pooling_max_grad(inp, out, dy, p, op=POOL_OP.MAX, dx=None):
    if dx is None:
        dx = torch.empty_like(inp)
    name = ("snn_hip_pooling_max_grad_f32" if inp.dtype == torch.float32 else
            "snn_hip_pooling_max_grad_f16")
    capi.check(getattr(capi.lib(), name)(
        _ptr(inp), _ptr(out), _ptr(dy), _ptr(dx), ctypes.byref(p), op,
        _stream()))
    return dx


def pooling_avg_grad(dy, p, dx=None):
    if dx is None:
        dx = torch.empty(p.batch * p.in_rows * p.in_cols * p.channels,
                         dtype=dy.dtype, device=dy.device)
    name = ("snn_hip_pooling_avg_grad_f32" if dy.dtype == torch.float32 else
            "snn_hip_pooling_avg_grad_f16")
    capi.check(getattr(capi.lib(), name)(
        _ptr(dy), _ptr(dx), ctypes.byref(p), _stream()))
    return dx


def matmul(a, b, batches, m, k, n, trans_a=False, trans_b=False, beta=0.0,
           out=None):
    assert a.numel() == batches * m * k and b.numel() == batches * k * n
    if out is None:
        out = torch.zeros(batches * m * n, dtype=a.dtype, device=a.device)
    name = ("snn_hip_matmul_f32" if a.dtype == torch.float32 else
            "snn_hip_matmul_f16")
    capi.check(getattr(capi.lib(), name)(
        _ptr(a), _ptr(b), _ptr(out), batches, m, k, n, int(trans_a),
        int(trans_b), float(beta), _stream()))
    return out


def _suffix(t):
    return "_f32" if t.dtype == torch.float32 else "_f16"


def pointwise_forward(x, op, out=None):
    """sycldnn::pointwise::launch<T, Op, Forward>; `out` may be `x`."""
    if out is None:
        out = torch.empty_like(x)
    fn = getattr(capi.lib(), "snn_hip_pointwise_forward" + _suffix(x))
    capi.check(fn(_ptr(x), _ptr(out), x.numel(), op, _stream()))
    return out


def pointwise_forward_bound(x, out, op):
    """pointwise_forward with everything fixed (see _bind)."""
    assert out.numel() == x.numel()
    fn = getattr(capi.lib(), "snn_hip_pointwise_forward" + _suffix(x))
    return _bind(fn, _ptr(x), _ptr(out), x.numel(), op,
                 ctypes.c_void_p(_stream()))


def pointwise_grad(val, err, op, out=None):
    """sycldnn::pointwise::launch<T, Op, Gradient>: `val` is the forward
    output (the forward input for LOG), `err` the incoming gradient."""
    if out is None:
        out = torch.empty_like(val)
    fn = getattr(capi.lib(), "snn_hip_pointwise_grad" + _suffix(val))
    capi.check(fn(_ptr(val), _ptr(err), _ptr(out), val.numel(), op, _stream()))
    return out


def binaryop_raw(lhs, rhs, out, lhs_dims, rhs_dims, op):
    """Calls the entry point and returns its status code (no exception)."""
    ld = (ctypes.c_int * max(len(lhs_dims), 1))(*lhs_dims)
    rd = (ctypes.c_int * max(len(rhs_dims), 1))(*rhs_dims)
    fn = getattr(capi.lib(), "snn_hip_binaryop" + _suffix(lhs))
    return fn(_ptr(lhs), _ptr(rhs), _ptr(out), ld, len(lhs_dims), rd,
              len(rhs_dims), op, _stream())


def binaryop(lhs, rhs, lhs_dims, rhs_dims, op, out=None):
    """sycldnn::binaryop::launch<T, Op> with BinaryParams{lhs_dims, rhs_dims};
    `out` may be either operand when that operand has the output's shape."""
    n = max(len(lhs_dims), len(rhs_dims), 1)
    l = [1] * (n - len(lhs_dims)) + list(lhs_dims)
    r = [1] * (n - len(rhs_dims)) + list(rhs_dims)
    size = 1
    for a, b in zip(l, r):
        size *= max(a, b)
    if out is None:
        out = torch.empty(size, dtype=lhs.dtype, device=lhs.device)
    capi.check(binaryop_raw(lhs, rhs, out, lhs_dims, rhs_dims, op))
    return out


__all__ = [
    "ALGO", "BINARY_OP", "DIRECTION", "POINTWISE_OP", "POOL_OP", "STATUS",
    "ConvParams", "DepthwiseParams", "PoolParams", "add_padding_to",
    "binaryop", "binaryop_raw", "calculate_padding", "conv2d",
    "conv2d_bias_act", "conv2d_prepare_filter", "conv2d_prepared",
    "conv2d_raw", "conv_flops", "conv_params", "conv_sizes",
    "default_algorithm",
    "depthwise_conv2d", "depthwise_params", "depthwise_sizes", "matmul",
    "pointwise_forward", "pointwise_grad", "pool_params", "pooling_avg_grad",
    "pooling_forward", "pooling_max_grad",
    "workspace_size",
]


class kernel_timing:
    """Context manager around snn_hip_kernel_timing_*: times the dominant
    kernel of every convolution launched inside it with HIP events on the
    launch stream.  After exit `.total_ms` and `.kernels` hold the result."""

    def __enter__(self):
        capi.check(capi.lib().snn_hip_kernel_timing_enable(1))
        self.total_ms = 0.0
        self.kernels = 0
        return self

    def __exit__(self, *exc):
        lib = capi.lib()
        capi.check(lib.snn_hip_kernel_timing_enable(0))
        ms = ctypes.c_double(0.0)
        n = ctypes.c_int(0)
        capi.check(lib.snn_hip_kernel_timing_read(ctypes.byref(ms),
                                                  ctypes.byref(n)))
        self.total_ms = ms.value
        self.kernels = n.value
        return False
