"""GPU parity against the reference's golden vectors, through the C ABI.

Every case of tests/golden/*.npz (the reference's own generated tests, exact
integers) is run through libsnn_hip.so with every algorithm whose selector
accepts it; the bar is the reference's own: exact for conv / depthwise / max
pooling (all values are integers below 2^24, so any correct fp32 evaluation
order is exact), 4 ULP for average pooling, 8 ULP for its gradient
(test/pooling/pooling_fixture.h:107-125).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from golden_cases import load, load_binaryop, load_matmul, load_pointwise
from portdnn_amd import capi, ops
from portdnn_amd.capi import ALGO, BINARY_OP, DIRECTION, POINTWISE_OP, POOL_OP

pytestmark = pytest.mark.gpu

ALGOS = [ALGO.DIRECT, ALGO.TILED, ALGO.IM2COL, ALGO.WINOGRAD, ALGO.MATMUL]
ALGO_NAME = {1: "direct", 2: "tiled", 3: "im2col", 4: "winograd", 6: "matmul"}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def supported(p, direction, algo):
    return capi.lib().snn_hip_conv2d_algorithm_supports(
        ctypes.byref(p), direction, algo) == algo


def run_conv_group(group, direction, algo):
    n_run = 0
    for case in load(group):
        p = ops.conv_params(case.n, case.h, case.w, case.c, case.k,
                            case.window, case.stride, case.same)
        if not supported(p, direction, algo):
            continue
        n_in, n_fil, _ = ops.conv_sizes(p, direction)
        a = dev(oracle.iota(n_in, case.max_val))
        b = dev(oracle.iota(n_fil, case.max_val))
        got = ops.conv2d(a, b, p, direction, algo).cpu().numpy()
        exp = case.expected.astype(np.float32)
        assert got.size == exp.size
        bad = np.flatnonzero(got != exp)
        assert bad.size == 0, (group, ALGO_NAME[algo], case[:9], bad[:4],
                               got[bad[:4]], exp[bad[:4]])
        n_run += 1
    return n_run


@pytest.mark.parametrize("algo", ALGOS, ids=lambda a: ALGO_NAME[a])
def test_conv2d_forward_golden(algo):
    n = run_conv_group("conv2d_forward", DIRECTION.FORWARD, algo)
    expected = {ALGO.DIRECT: 2592, ALGO.IM2COL: 2592, ALGO.TILED: 5 * 324,
                ALGO.WINOGRAD: 324, ALGO.MATMUL: 162 + 6}
    assert n >= expected[algo] - 200 and n > 0, n


@pytest.mark.parametrize("algo", [ALGO.DIRECT, ALGO.IM2COL, ALGO.WINOGRAD,
                                  ALGO.MATMUL], ids=lambda a: ALGO_NAME[a])
def test_conv2d_input_backprop_golden(algo):
    assert run_conv_group("conv2d_input_backprop", DIRECTION.INPUT_BACKPROP,
                          algo) > 0


@pytest.mark.parametrize("algo", [ALGO.DIRECT, ALGO.IM2COL, ALGO.WINOGRAD,
                                  ALGO.MATMUL], ids=lambda a: ALGO_NAME[a])
def test_conv2d_filter_backprop_golden(algo):
    assert run_conv_group("conv2d_filter_backprop", DIRECTION.FILTER_BACKPROP,
                          algo) > 0


@pytest.mark.parametrize("group,direction", [
    ("depthwise_forward", DIRECTION.FORWARD),
    ("depthwise_input_backprop", DIRECTION.INPUT_BACKPROP),
    ("depthwise_filter_backprop", DIRECTION.FILTER_BACKPROP)])
def test_depthwise_golden(group, direction):
    n_run = 0
    for case in load(group):
        p = ops.depthwise_params(case.n, case.h, case.w, case.c, case.k,
                                 case.window, case.stride, case.same)
        n_in, n_fil, _ = ops.depthwise_sizes(p, direction)
        a = dev(oracle.iota(n_in, case.max_val))
        b = dev(oracle.iota(n_fil, case.max_val))
        got = ops.depthwise_conv2d(a, b, p, direction).cpu().numpy()
        exp = case.expected.astype(np.float32)
        bad = np.flatnonzero(got != exp)
        assert bad.size == 0, (group, case[:9], bad[:4], got[bad[:4]],
                               exp[bad[:4]])
        n_run += 1
    assert n_run == 1620


@pytest.mark.parametrize("op", [POOL_OP.MAX, POOL_OP.MAX_WITH_NAN])
def test_pool_max_forward_golden(op):
    n_run = 0
    for case in load("pool_max_forward"):
        p = ops.pool_params(case.n, case.h, case.w, case.c, case.window,
                            case.stride, case.same)
        x = dev(oracle.iota(case.n * case.h * case.w * case.c, case.max_val))
        got = ops.pooling_forward(x, p, op).cpu().numpy()
        assert np.array_equal(got, case.expected.astype(np.float32)), case[:9]
        n_run += 1
    assert n_run == 972


def test_pool_avg_forward_golden():
    n_run = 0
    for case in load("pool_avg_forward"):
        p = ops.pool_params(case.n, case.h, case.w, case.c, case.window,
                            case.stride, case.same)
        x = dev(oracle.iota(case.n * case.h * case.w * case.c, case.max_val))
        got = ops.pooling_forward(x, p, POOL_OP.AVERAGE).cpu().numpy()
        exp = case.expected
        tol = 4 * np.spacing(np.abs(exp).astype(np.float32))
        assert np.all(np.abs(got.astype(np.float64) - exp) <= tol), case[:9]
        n_run += 1
    assert n_run == 972


def test_pool_max_grad_golden():
    n_run = 0
    for case in load("pool_max_grad"):
        p = ops.pool_params(case.n, case.h, case.w, case.c, case.window,
                            case.stride, case.same)
        x = dev(oracle.iota(case.n * case.h * case.w * case.c, case.max_val))
        y = ops.pooling_forward(x, p, POOL_OP.MAX)
        dy = dev(oracle.iota(y.numel(), case.max_val))
        got = ops.pooling_max_grad(x, y, dy, p).cpu().numpy()
        assert np.array_equal(got, case.expected.astype(np.float32)), case[:9]
        n_run += 1
    assert n_run == 432


def test_pool_avg_grad_golden():
    n_run = 0
    for case in load("pool_avg_grad"):
        p = ops.pool_params(case.n, case.h, case.w, case.c, case.window,
                            case.stride, case.same)
        dy = dev(oracle.iota(p.batch * p.out_rows * p.out_cols * case.c,
                             case.max_val))
        got = ops.pooling_avg_grad(dy, p).cpu().numpy()
        exp = case.expected
        tol = 8 * np.spacing(np.abs(exp).astype(np.float32))
        assert np.all(np.abs(got.astype(np.float64) - exp) <= tol), case[:9]
        n_run += 1
    assert n_run == 432


def test_matmul_golden():
    """The reference's matmul cases through snn_hip_matmul_f32, offsets into
    the buffers included (test/matmul/fixture.h:37-76); exact."""
    for c in load_matmul():
        lhs = dev(oracle.iota(c.batches * c.m * c.k + c.lhs_offset, c.max_val))
        rhs = dev(oracle.iota(c.batches * c.k * c.n + c.rhs_offset, c.max_val))
        out = dev(oracle.iota(c.batches * c.m * c.n + c.out_offset, c.max_val))
        ops.matmul(lhs[c.lhs_offset:], rhs[c.rhs_offset:], c.batches, c.m, c.k,
                   c.n, c.trans_lhs, c.trans_rhs, c.beta,
                   out=out[c.out_offset:])
        assert np.array_equal(out.cpu().numpy(),
                              c.expected.astype(np.float32)), c[:11]


def ulp_close(got, exp, ulps=10):
    """SNN_ALMOST_EQUAL(exp, got, 10u) of test/helpers/float_comparison.h."""
    got = np.asarray(got, dtype=np.float32)
    exp = np.asarray(exp, dtype=np.float32)
    tol = ulps * np.spacing(np.maximum(np.abs(exp), np.abs(got)))
    return np.all(np.abs(got.astype(np.float64) - exp.astype(np.float64))
                  <= tol.astype(np.float64))


def test_pointwise_golden():
    """test/pointwise/<op>_{forward,grad}.cc through snn_hip_pointwise_*,
    driven as test/pointwise/pointwise_fixture.h drives the reference."""
    n_cases = 0
    for c in load_pointwise():
        op = getattr(POINTWISE_OP, c.op.upper())
        x = dev(oracle.iota_signed(c.size) if c.signed
                else oracle.iota(c.size, c.max_val))
        if not c.is_grad:
            got = ops.pointwise_forward(x, op).cpu().numpy()
            assert ulp_close(got, c.expected), (c.op, c.size)
        else:
            val = x if c.op == "log" else ops.pointwise_forward(x, op)
            got = ops.pointwise_grad(val, x, op).cpu().numpy()
            assert np.allclose(got, c.expected, rtol=0, atol=1e-5), \
                (c.op, c.size)
        n_cases += 1
    assert n_cases == 36


def test_binaryop_golden():
    """test/binaryop/binaryop_{add,sub,mul,div}.cc through snn_hip_binaryop_f32
    (test/binaryop/fixture.h:37-76, 10 ULP)."""
    n_cases = 0
    for c in load_binaryop():
        lhs = dev(oracle.iota(int(np.prod(c.lhs_dims)), c.max_val))
        rhs = dev(oracle.iota(int(np.prod(c.rhs_dims)), c.max_val))
        got = ops.binaryop(lhs, rhs, c.lhs_dims, c.rhs_dims,
                           getattr(BINARY_OP, c.op.upper())).cpu().numpy()
        assert ulp_close(got, c.expected), (c.op, c.lhs_dims, c.rhs_dims)
        n_cases += 1
    assert n_cases == 52
