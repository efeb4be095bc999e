"""The depthwise filter gradient entry point that allocates nothing
(snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32) against the ordinary
entry point and the CPU oracle, through the C ABI.

The entry point keeps the work-groups' partial filters in a device array
inside the library, shared by every call on a GPU and never cleared, so the
calls run back to back: a large input first, then smaller ones whose plans
use fewer work-groups and fewer channels (stale partial filters of the first
call stay in the array behind them), then shapes for the path that needs no
partial filters at all.

fp32 bar: |a - b| <= 1e-4 * |b| + 1e-5 * max(1, rms(b)) (dF sums N*OH*OW
products, so its magnitude grows with the input size).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from portdnn_amd import capi, ops
from portdnn_amd.capi import DIRECTION

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def assert_close(got, ref, what):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, what
    scale = max(1.0, float(np.sqrt(np.mean(ref * ref))))
    err = np.abs(got - ref)
    bad = np.flatnonzero(~(err <= RTOL * np.abs(ref) + ATOL * scale))
    assert bad.size == 0, (what, bad.size, float(err.max()))


def noalloc(x, dy, p):
    out = torch.empty(9 * p.channels, dtype=torch.float32, device=x.device)
    fn = capi.lib().snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    capi.check(fn(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(dy.data_ptr()),
                  ctypes.c_void_p(out.data_ptr()), ctypes.byref(p), stream))
    return out


# (batch, rows, cols, channels, stride).  The first three take the path with
# partial filters (many channels: more float atomics into dF than the launcher
# allows), each with fewer work-groups or channels than the one before; the
# last three have few enough sums to add them into dF directly.
CALLS = [(32, 56, 56, 256, 1), (32, 56, 56, 128, 1), (20, 55, 57, 128, 2),
         (24, 112, 112, 32, 1), (11, 111, 109, 64, 2), (4, 56, 56, 128, 2)]


def temporary_memory(reset):
    reserved, high = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    capi.check(capi.lib().snn_hip_temporary_memory_stats(
        ctypes.byref(reserved), ctypes.byref(high), 1 if reset else 0))
    return reserved.value, high.value


def test_noalloc_filter_backprop_matches_allocating_entry():
    rng = np.random.default_rng(0x5EED + 77)
    pending = []
    # Nothing may come out of the pools stream-ordered temporaries are taken
    # from while the entry point runs: clear their high-water marks, and make
    # sure the check can see a temporary at all (the allocating entry on the
    # first shape takes one).
    warm = ops.depthwise_params(*CALLS[0][:4], 1, 3, CALLS[0][4], True)
    wx = torch.zeros(warm.batch * warm.in_rows * warm.in_cols * warm.channels,
                     device="cuda")
    wdy = torch.zeros(warm.batch * warm.out_rows * warm.out_cols *
                      warm.channels, device="cuda")
    ops.depthwise_conv2d(wx, wdy, warm, DIRECTION.FILTER_BACKPROP)
    torch.cuda.synchronize()
    assert temporary_memory(reset=True)[1] > 0
    del wx, wdy
    torch.cuda.synchronize()
    temporary_memory(reset=True)
    reserved_before, high_before = temporary_memory(reset=False)
    # every call is enqueued before any result is read, so the calls really
    # run in a row on the stream and share the scratch array
    for batch, rows, cols, ch, stride in CALLS:
        p = ops.depthwise_params(batch, rows, cols, ch, 1, 3, stride, True)
        x = rng.standard_normal(batch * rows * cols * ch).astype(np.float32)
        dy = rng.standard_normal(
            batch * p.out_rows * p.out_cols * ch).astype(np.float32)
        dx, ddy = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
        got = noalloc(dx, ddy, p)
        pending.append((p, x, dy, dx, ddy, got))
    torch.cuda.synchronize()
    reserved_after, used_high = temporary_memory(reset=False)
    assert used_high == high_before and reserved_after == reserved_before, (
        "the no-allocation entry took a temporary", high_before, used_high,
        reserved_before, reserved_after)
    for p, x, dy, dx, ddy, got in pending:
        want = ops.depthwise_conv2d(dx, ddy, p, DIRECTION.FILTER_BACKPROP)
        assert_close(got.cpu().numpy(), want.cpu().numpy(),
                     ("noalloc vs allocating entry", repr(p)))
        op = oracle.Params(p.channels, 1, p.batch, p.in_rows, p.in_cols, 3, 3,
                           p.stride_rows, p.stride_cols, p.out_rows,
                           p.out_cols, p.pad_rows, p.pad_cols)
        assert_close(got.cpu().numpy(),
                     oracle.depthwise_filter_backprop(x, dy, op),
                     ("noalloc vs oracle", repr(p)))


def test_noalloc_rejects_bad_arguments():
    p = ops.depthwise_params(2, 8, 8, 8, 1, 3, 1, True)
    fn = capi.lib().snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32
    assert fn(None, None, None, ctypes.byref(p), None) == \
        capi.STATUS.INVALID_PARAMETER
    p.channels = 0
    x = torch.zeros(16, device="cuda")
    assert fn(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(x.data_ptr()),
              ctypes.c_void_p(x.data_ptr()), ctypes.byref(p), None) == \
        capi.STATUS.INVALID_PARAMETER
