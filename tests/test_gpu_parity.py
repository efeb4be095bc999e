"""GPU parity on seeded random data at the benchmark shapes, through the C ABI.

Floating-point bar (fp32): |gpu - oracle| <= 1e-4 * |oracle| + 1e-5 * S, where
the oracle accumulates in double and S = max(1, rms(oracle)).  S is 1 -- i.e.
the bar is exactly "1e-4 relative / 1e-5 absolute" -- whenever the outputs are
O(1); for the deep reductions of the ResNet layers (up to 4608 products of
U[-1,1] values, output rms up to ~23) the absolute term scales with the output
magnitude, because no fp32 accumulation (the reference's included) can hold
1e-5 absolute on an output that cancels to ~0 out of terms that large.
f16: 1e-2 relative to S against the double-precision result of the
f16-rounded operands.

Shapes are the benchmark configurations at a batch the CPU oracle finishes in
seconds; the full batch-32 shapes are covered by sampled outputs recomputed in
float64 and by linearity.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from portdnn_amd import capi, ops
from portdnn_amd.capi import ALGO, BINARY_OP, DIRECTION, POINTWISE_OP, POOL_OP, \
    STATUS

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5
ALGO_NAME = {1: "direct", 2: "tiled", 3: "im2col", 4: "winograd", 6: "matmul"}
FWD_ALGOS = [ALGO.DIRECT, ALGO.TILED, ALGO.IM2COL, ALGO.WINOGRAD, ALGO.MATMUL]
BK_ALGOS = [ALGO.DIRECT, ALGO.IM2COL, ALGO.WINOGRAD, ALGO.MATMUL]

RESNET_3X3 = [(56, 64), (28, 128), (14, 256), (7, 512)]


def assert_close(got, ref, what, rtol=RTOL, atol=ATOL):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, what
    scale = max(1.0, float(np.sqrt(np.mean(ref * ref))))
    err = np.abs(got - ref)
    tol = rtol * np.abs(ref) + atol * scale
    bad = np.flatnonzero(~(err <= tol))
    assert bad.size == 0, (what, "n_bad=%d of %d" % (bad.size, ref.size),
                           "worst err %.3e tol %.3e" % (
                               err[bad].max(), tol[bad[np.argmax(err[bad])]]),
                           bad[:4], got[bad[:4]], ref[bad[:4]])


def uniform(rng, n):
    return rng.uniform(-1.0, 1.0, size=n).astype(np.float32)


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda().to(dtype)


def supported(p, direction, algo):
    return capi.lib().snn_hip_conv2d_algorithm_supports(
        ctypes.byref(p), direction, algo) == algo


def oracle_params(p, features):
    return oracle.Params(p.channels, features, p.batch, p.in_rows, p.in_cols,
                         p.window_rows, p.window_cols, p.stride_rows,
                         p.stride_cols, p.out_rows, p.out_cols, p.pad_rows,
                         p.pad_cols)


ORACLE_FN = {DIRECTION.FORWARD: oracle.conv2d_forward,
             DIRECTION.INPUT_BACKPROP: oracle.conv2d_input_backprop,
             DIRECTION.FILTER_BACKPROP: oracle.conv2d_filter_backprop}


def conv_case(p, direction, algos, seed):
    rng = np.random.default_rng(seed)
    n_in, n_fil, _ = ops.conv_sizes(p, direction)
    a, b = uniform(rng, n_in), uniform(rng, n_fil)
    ref = ORACLE_FN[direction](a, b, oracle_params(p, p.features), acc64=True)
    da, db = dev(a), dev(b)
    ran = 0
    for algo in algos:
        if not supported(p, direction, algo):
            continue
        got = ops.conv2d(da, db, p, direction, algo).cpu().numpy()
        assert_close(got, ref, (ALGO_NAME[algo], direction, repr(p)))
        ran += 1
    assert ran > 0


@pytest.mark.parametrize("size,ch", RESNET_3X3)
@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
def test_resnet_3x3(size, ch, direction):
    p = ops.conv_params(2, size, size, ch, ch, 3, 1, True)
    algos = FWD_ALGOS if direction == DIRECTION.FORWARD else BK_ALGOS
    conv_case(p, direction, algos, seed=100 + size + direction)


@pytest.mark.parametrize("size,ch", RESNET_3X3)
@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
def test_resnet_1x1_expand(size, ch, direction):
    p = ops.conv_params(2, size, size, ch, 4 * ch, 1, 1, False)
    algos = FWD_ALGOS if direction == DIRECTION.FORWARD else BK_ALGOS
    conv_case(p, direction, algos, seed=200 + size + direction)


@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
def test_stem_7x7_stride2(direction):
    p = ops.conv_params(1, 224, 224, 3, 64, 7, 2, True)
    assert (p.out_rows, p.pad_rows) == (112, 2)
    conv_case(p, direction, [ALGO.DIRECT, ALGO.IM2COL], seed=300 + direction)


@pytest.mark.parametrize("batch,rows,cols,same", [
    (5, 97, 61, True),      # ragged pixel block, odd rows
    (6, 85, 100, False),    # no padding
    (2, 224, 224, True),    # the stem layer itself
])
def test_stem_in_half_precision(batch, rows, cols, same):
    """A binary16 launch of the 7x7 stride-2 three-channel stem runs the fp32
    stem kernels: forward, the image and the filter widened into a temporary
    and the output rounded to binary16 by the kernel's own store; the
    gradients through fp32 copies.  Against the oracle in double precision on the same
    binary16-rounded operands; nothing written past the result."""
    p = ops.conv_params(batch, rows, cols, 3, 64, 7, 2, same)
    rng = np.random.default_rng(331 + rows + cols)
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP,
                      DIRECTION.FILTER_BACKPROP):
        n_a, n_b, n_o = ops.conv_sizes(p, direction)
        a = uniform(rng, n_a).astype(np.float16)
        b = uniform(rng, n_b).astype(np.float16)
        ref = ORACLE_FN[direction](a.astype(np.float32), b.astype(np.float32),
                                   oracle_params(p, 64), acc64=True)
        out = torch.full((n_o + 16,), 7.0, dtype=torch.float16, device="cuda")
        got = ops.conv2d(dev(a, torch.float16), dev(b, torch.float16), p,
                         direction, ALGO.IM2COL, out=out[:n_o])
        assert_close_f16(got.float().cpu().numpy(), ref,
                         ("f16 stem", direction, batch, rows, cols))
        assert torch.all(out[n_o:] == 7.0)


@pytest.mark.parametrize("batch,rows,cols,same", [
    (40, 64, 64, True),     # bands of three steps, two-row last band
    (5, 97, 61, True),      # 49 x 31 output: ragged pixel block, odd rows
    (6, 85, 100, False),    # no padding
    (3, 223, 221, True),    # odd image, padding 3
    (9, 224, 224, True),    # the stem layer itself, bands of two steps
])
def test_stem_rows_in_lds_kernel(batch, rows, cols, same):
    """The 7x7 stride-2, 3 -> 64 channel forward and filter-gradient kernels
    that keep a band of input rows in LDS (used from 224 output rows over the
    batch upwards)."""
    p = ops.conv_params(batch, rows, cols, 3, 64, 7, 2, same)
    assert batch * p.out_rows >= 224
    conv_case(p, DIRECTION.FORWARD, [ALGO.IM2COL, ALGO.TILED],
              seed=350 + batch + rows)
    conv_case(p, DIRECTION.FILTER_BACKPROP, [ALGO.IM2COL],
              seed=360 + batch + rows)


@pytest.mark.parametrize("batch,rows,cols,same", [
    (60, 64, 64, True),     # bands of three steps, two-row last band
    (40, 97, 61, True),     # 49 x 31 output: ragged pixel block, odd rows
    (45, 85, 100, False),   # no padding
    (46, 86, 100, False),   # ... and a last input row that no window reads
    (17, 223, 221, True),   # odd image, padding 3
    (16, 224, 224, True),   # the stem layer itself
])
def test_stem_input_backprop_rows_in_lds_kernel(batch, rows, cols, same):
    """The 7x7 stride-2, 3 <- 64 channel input-gradient kernel that adds the
    products into a band of input rows in LDS (used from 1792 output rows over
    the batch upwards)."""
    p = ops.conv_params(batch, rows, cols, 3, 64, 7, 2, same)
    assert batch * p.out_rows >= 1792
    conv_case(p, DIRECTION.INPUT_BACKPROP, [ALGO.IM2COL],
              seed=370 + batch + rows)
    # The kernel stores most rows, adds into the rows two bands share and
    # writes nothing where no window reaches: whatever dX held before must be
    # gone everywhere.
    rng = np.random.default_rng(371 + batch + rows)
    n_dy, n_fil, n_dx = ops.conv_sizes(p, DIRECTION.INPUT_BACKPROP)
    dy, w = uniform(rng, n_dy), uniform(rng, n_fil)
    ref = oracle.conv2d_input_backprop(dy, w, oracle_params(p, 64), acc64=True)
    out = torch.full((n_dx,), float("nan"), device="cuda")
    ops.conv2d(dev(dy), dev(w), p, DIRECTION.INPUT_BACKPROP, ALGO.IM2COL,
               out=out)
    assert_close(out.cpu().numpy(), ref, ("stem input gradient over NaN", p))


def test_config0_single_image_tiled():
    """Benchmark configuration 0: N=1, 56x56x64 -> 64, 3x3 s1 SAME, Tiled;
    also checked against the reference-loop-nest restatement in fp32."""
    p = ops.conv_params(1, 56, 56, 64, 64, 3, 1, True)
    rng = np.random.default_rng(0x5EED)
    x, w = uniform(rng, 56 * 56 * 64), uniform(rng, 9 * 64 * 64)
    op = oracle_params(p, 64)
    ref = oracle.conv2d_forward(x, w, op, acc64=True)
    tiled = oracle.conv2d_tiled_forward(x, w, op)
    assert_close(tiled, ref, "tiled restatement vs direct oracle")
    got = ops.conv2d(dev(x), dev(w), p, DIRECTION.FORWARD,
                     ALGO.TILED).cpu().numpy()
    assert_close(got, ref, "config0 tiled")


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, same
    (1, 56, 56, 64, 64, 3, 1, True),      # configuration 0
    (1, 50, 50, 64, 64, 3, 1, True),      # pixel count not a multiple of 16
    (2, 27, 29, 128, 128, 3, 1, True),    # two channel groups, two feature blocks
    (4, 56, 56, 64, 64, 3, 2, True),      # stride 2 (asymmetric padding)
    (1, 58, 58, 64, 128, 3, 1, False),    # VALID
    (1, 56, 56, 64, 64, 1, 1, False),     # 1x1: a single step
    (1, 52, 52, 64, 64, 5, 1, True),      # 25 taps: beyond its step limit
])
def test_small_problem_kernel(shape):
    """Few-tile forward convolutions (below 128 tiles of 64x64) run on the
    kernel whose waves split the reduction inside a work-group -- one launch,
    no atomics -- through the Tiled and Im2col tags; the same with bias and
    ReLU folded in; and twice, bit for bit (its additions have a fixed
    order).  The last shape has too long a reduction for it and must still be
    right on the kernels that take it instead."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(1500 + rows + ch + window)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = uniform(rng, n_in), uniform(rng, n_fil)
    bias = uniform(rng, feats)
    ref = oracle.conv2d_forward(x, w, oracle_params(p, feats), acc64=True)
    dx, dw = dev(x), dev(w)
    for algo in (ALGO.TILED, ALGO.IM2COL):
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        got = ops.conv2d(dx, dw, p, DIRECTION.FORWARD, algo)
        assert_close(got.cpu().numpy(), ref, ("small", ALGO_NAME[algo], shape))
        if window != 5:
            again = ops.conv2d(dx, dw, p, DIRECTION.FORWARD, algo)
            assert torch.equal(got.view(torch.int32), again.view(torch.int32))
        fused = ops.conv2d_bias_act(dx, dw, dev(bias), p, algo, relu=True)
        want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64), 0)
        assert_close(fused.cpu().numpy(), want.reshape(-1),
                     ("small + bias + relu", ALGO_NAME[algo], shape))


@pytest.mark.parametrize("shape", [
    (16, 56, 56, 16, 128, 3, 3, True),   # one channel block, 13 pixel blocks a wave
    (32, 28, 28, 32, 128, 3, 3, True),   # two channel blocks, 7 pixel blocks
    (24, 40, 40, 48, 128, 3, 3, True),   # 10 pixel blocks
    (16, 56, 56, 64, 64, 3, 3, True),    # the input gradient qualifies as well
    (16, 56, 56, 16, 128, 5, 5, True),   # 25 taps: the loop over any window
    (16, 58, 58, 32, 128, 3, 3, False),  # VALID
    (8, 100, 250, 16, 64, 3, 3, True),   # tiles longer than a row, across images
    (16, 56, 56, 32, 128, 1, 3, True),   # fewer taps than filter loads in flight
])
def test_input_rows_in_lds_kernel(shape):
    """Large stride-1 convolutions through the Tiled and Im2col tags run on the
    kernel that keeps the input rows of a run of output pixels in LDS (16
    channels at a time) and reads the filter straight from the HWCF tensor:
    forward, and the input gradient as a forward convolution over dY with
    mirrored taps (the kernel takes it when the channel count is a multiple of
    64, other shapes fall to the gather kernel and must be right all the
    same); bias and ReLU folded into the store; twice, bit for bit."""
    batch, rows, cols, ch, feats, wr, wc, same = shape
    p = ops.ConvParams(channels=ch, features=feats, batch=batch, in_rows=rows,
                       in_cols=cols, window_rows=wr, window_cols=wc,
                       stride_rows=1, stride_cols=1)
    ops.add_padding_to(p, same)
    rng = np.random.default_rng(2600 + rows + ch + wr)
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
        n_in, n_fil, _ = ops.conv_sizes(p, direction)
        a, w = uniform(rng, n_in), uniform(rng, n_fil)
        ref = ORACLE_FN[direction](a, w, oracle_params(p, feats), acc64=True)
        da, dw = dev(a), dev(w)
        for algo in (ALGO.TILED, ALGO.IM2COL):
            if not supported(p, direction, algo):
                continue
            got = ops.conv2d(da, dw, p, direction, algo)
            assert_close(got.cpu().numpy(), ref,
                         ("rows in LDS", ALGO_NAME[algo], direction, shape))
            if direction == DIRECTION.FORWARD or ch % 64 == 0:
                again = ops.conv2d(da, dw, p, direction, algo)
                assert torch.equal(got.view(torch.int32),
                                   again.view(torch.int32)), (direction, shape)
        if direction == DIRECTION.FORWARD:
            bias = uniform(rng, feats)
            fused = ops.conv2d_bias_act(da, dw, dev(bias), p, ALGO.IM2COL,
                                        relu=True)
            want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64),
                              0)
            assert_close(fused.cpu().numpy(), want.reshape(-1),
                         ("rows in LDS + bias + relu", shape))
            # operands that are not 16-byte aligned go to the kernels that
            # load word by word, with the same result
            pad_a = torch.empty(a.size + 1, device="cuda")
            pad_w = torch.empty(w.size + 3, device="cuda")
            pad_a[1:].copy_(da)
            pad_w[3:].copy_(dw)
            got = ops.conv2d(pad_a[1:], pad_w[3:], p, direction, ALGO.IM2COL)
            assert_close(got.cpu().numpy(), ref,
                         ("rows in LDS, unaligned operands", shape))


@pytest.mark.parametrize("shape", [
    (32, 14, 14, 256, 256, 3, 3, True),  # 4 feature blocks a wave, 2 channel
                                         # blocks a wave
    (32, 7, 7, 512, 512, 3, 3, True),    # 2 feature blocks a wave, tiles that
                                         # span images, 4 channel blocks a wave
    (40, 14, 14, 128, 96, 3, 3, True),   # 96 features: three slices of 32
    (64, 14, 14, 128, 128, 5, 5, True),  # 25 taps, tiles of whole rows
    (64, 16, 16, 128, 128, 3, 3, False), # VALID
    (32, 14, 14, 1024, 256, 1, 1, False),  # 1x1 with a long reduction, forward
    (32, 7, 7, 512, 2048, 1, 1, False),  # ... and as the input gradient
])
def test_reduction_split_over_waves_kernel(shape):
    """Deep stride-1 layers with few pixels (channels a multiple of 128) run on
    the kernel whose eight waves each hold the whole output tile and split the
    channel blocks among themselves, meeting in LDS at the end: forward and
    the input gradient (a forward convolution over dY with mirrored taps),
    against the oracle over the whole tensor; bias and ReLU folded into the
    store; no atomics, so twice gives the same bits.  1x1 windows take it
    from 1024 reduction channels on (in the other direction the two 1x1
    shapes run on the kernels for short reductions)."""
    batch, rows, cols, ch, feats, wr, wc, same = shape
    p = ops.ConvParams(channels=ch, features=feats, batch=batch, in_rows=rows,
                       in_cols=cols, window_rows=wr, window_cols=wc,
                       stride_rows=1, stride_cols=1)
    ops.add_padding_to(p, same)
    rng = np.random.default_rng(2700 + rows + ch + wr)
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
        n_in, n_fil, _ = ops.conv_sizes(p, direction)
        a, w = uniform(rng, n_in), uniform(rng, n_fil)
        ref = ORACLE_FN[direction](a, w, oracle_params(p, feats), acc64=True)
        da, dw = dev(a), dev(w)
        for algo in (ALGO.TILED, ALGO.IM2COL):
            if not supported(p, direction, algo):
                continue
            got = ops.conv2d(da, dw, p, direction, algo)
            assert_close(got.cpu().numpy(), ref,
                         ("reduction split over waves", ALGO_NAME[algo],
                          direction, shape))
            # (the gradient of the 96-feature and of the VALID shape falls to
            # kernels that add partial sums atomically)
            if wr == 1:
                continue
            if direction == DIRECTION.FORWARD or (same and feats % 128 == 0):
                again = ops.conv2d(da, dw, p, direction, algo)
                assert torch.equal(got.view(torch.int32),
                                   again.view(torch.int32)), (direction, shape)
        if direction == DIRECTION.FORWARD:
            bias = uniform(rng, feats)
            fused = ops.conv2d_bias_act(da, dw, dev(bias), p, ALGO.IM2COL,
                                        relu=True)
            want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64),
                              0)
            assert_close(fused.cpu().numpy(), want.reshape(-1),
                         ("reduction split over waves + bias + relu", shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, SAME
    (32, 7, 7, 512, 2048, 1, 1, 1, 1, False),   # one work-group per tile
    (32, 14, 14, 256, 1024, 1, 1, 1, 1, False), # four work-groups per tile
    (5, 9, 11, 64, 128, 1, 1, 1, 1, False),     # pixel count not a multiple of 4
    (3, 20, 20, 192, 64, 1, 1, 1, 1, False),    # waves past the end, no pixels
    (2, 12, 12, 64, 64, 1, 1, 1, 1, False),     # one tile, 9 steps a wave
    (8, 28, 28, 128, 512, 1, 1, 1, 1, False),
    (8, 14, 14, 128, 64, 3, 3, 1, 1, True),     # 3x3 SAME: 9 taps, padding
    (4, 28, 28, 64, 128, 3, 3, 2, 2, True),     # 3x3 stride 2
    (4, 28, 28, 128, 256, 1, 1, 2, 2, False),   # 1x1 stride 2
    (6, 20, 18, 64, 64, 5, 3, 1, 2, False),     # VALID, 5x3 window, strides 1x2
    (40, 7, 3, 64, 64, 3, 3, 1, 1, True),       # rows shorter than a step
    (8, 7, 7, 256, 128, 3, 3, 1, 1, True),
    # channel counts that are neither multiples of 64 nor few enough for the
    # one-work-group kernel: ragged tiles
    (4, 14, 14, 96, 80, 3, 3, 1, 1, True),
    (6, 10, 10, 36, 100, 3, 3, 2, 2, True),
    (8, 12, 12, 200, 72, 1, 1, 1, 1, False),
])
def test_filter_gradient_from_registers(shape):
    """The filter gradient of layers with channels and features in multiples
    of 64 (behind the Tiled / Im2col / Matmul tags) runs on the kernel that
    feeds both NHWC operands straight into the matrix instruction -- one (tap,
    64 x 64 tile) unit per work-group, the pixel range split over its waves
    and, for few units, over work-groups whose partial filters a second kernel
    adds: against the oracle over the whole tensor, through every tag that
    reaches it; partial filters in a temporary, in a workspace of the size the
    query recommends and past one too small or misaligned; everything is added
    in a fixed order, so every call gives the same bits, the reproducible
    entry point included."""
    batch, rows, cols, ch, feats, wr, wc, sr, sc, same = shape
    p = ops.ConvParams(channels=ch, features=feats, batch=batch, in_rows=rows,
                       in_cols=cols, window_rows=wr, window_cols=wc,
                       stride_rows=sr, stride_cols=sc)
    ops.add_padding_to(p, same)
    rng = np.random.default_rng(3100 + rows + ch + wr)
    direction = DIRECTION.FILTER_BACKPROP
    n_in, n_fil, _ = ops.conv_sizes(p, direction)
    a, w = uniform(rng, n_in), uniform(rng, n_fil)
    ref = ORACLE_FN[direction](a, w, oracle_params(p, feats), acc64=True)
    da, dw = dev(a), dev(w)
    first, tag = None, None
    for algo in (ALGO.MATMUL, ALGO.TILED, ALGO.IM2COL):
        if not supported(p, direction, algo):
            continue
        got = ops.conv2d(da, dw, p, direction, algo)
        assert_close(got.cpu().numpy(), ref,
                     ("filter gradient", ALGO_NAME[algo], shape))
        if first is None:
            first, tag = got, algo
        assert torch.equal(got.view(torch.int32), first.view(torch.int32))
    assert first is not None
    _, rec = ops.workspace_size(p, direction, tag)
    # (one work-group per unit -- as many units as compute units, or too few
    # steps of 4 pixels to split further than over the 8 waves -- needs none)
    units = wr * wc * ((ch + 63) // 64) * ((feats + 63) // 64)
    steps = (batch * p.out_rows * p.out_cols + 3) // 4
    if max(1, min(256 // units, steps // 64)) > 1:
        assert rec >= 2 * wr * wc * ch * feats, rec
    room = torch.full((rec + 8,), float("nan"), device="cuda")
    for ws in (room[:rec], room[1:rec + 1], room[:max(rec // 2 - 4, 0)]):
        got = ops.conv2d(da, dw, p, direction, tag, workspace=ws)
        assert torch.equal(got.view(torch.int32), first.view(torch.int32))
    got = ops.conv2d_deterministic(da, dw, p, direction, tag)
    assert torch.equal(got.view(torch.int32), first.view(torch.int32))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, SAME
    # (from 2^30 multiply-adds on; smaller launches keep the general kernel)
    (16, 56, 56, 128, 128, 3, 2, True),  # a ResNet 3x3 stride-2 layer
    (16, 57, 55, 128, 128, 3, 2, True),  # odd image
    (16, 57, 55, 128, 144, 3, 2, False), # VALID
    (8, 40, 40, 128, 128, 5, 2, True),   # 5x5: classes of 3x3, 3x2, 2x3, 2x2 taps
    (18, 45, 45, 128, 256, 3, 3, True),  # stride 3: one tap per class
    (4, 64, 64, 64, 96, 7, 2, True),     # 7x7 stride 2 over 64 channels
    (48, 40, 40, 128, 256, 2, 3, False), # stride above the window: empty classes
    (4, 28, 28, 256, 256, 3, 2, True),   # below the threshold: general kernel
])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_strided_input_gradient_by_stride_classes(shape, dtype):
    """A strided input gradient is computed class by class of input pixels
    modulo the strides -- each a dense stride-1 forward convolution of dY with
    the sub-filter of the taps that reach the class, on the stride-1 kernels
    (binary16: on the binary16 ones when the feature count is a multiple of
    64, else through fp32 copies) -- and interleaved into dX in one pass:
    against the oracle over the whole tensor, every element of dX written (the
    output starts as NaN)."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(2950 + rows + ch + window)
    direction = DIRECTION.INPUT_BACKPROP
    n_dy, n_fil, n_dx = ops.conv_sizes(p, direction)
    half = dtype == "f16"
    tdt = torch.float16 if half else torch.float32
    dy, w = uniform(rng, n_dy), uniform(rng, n_fil)
    if half:
        dy, w = dy.astype(np.float16), w.astype(np.float16)
    ref = ORACLE_FN[direction](dy.astype(np.float32), w.astype(np.float32),
                               oracle_params(p, feats), acc64=True)
    out = torch.full((n_dx + 16,), float("nan"), dtype=tdt, device="cuda")
    out[n_dx:] = 7.0
    for algo in (ALGO.IM2COL, ALGO.TILED):
        if not supported(p, direction, algo):
            continue
        out[:n_dx] = float("nan")
        got = ops.conv2d(dev(dy, tdt), dev(w, tdt), p, direction, algo,
                         out=out[:n_dx])
        if half:
            assert_close_f16(got.float().cpu().numpy(), ref,
                             ("f16 strided input gradient", shape))
        else:
            assert_close(got.cpu().numpy(), ref,
                         ("strided input gradient", ALGO_NAME[algo], shape))
        assert torch.all(out[n_dx:] == 7.0)


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, stride
    (8, 56, 56, 256, 512, 2),    # a ResNet shortcut
    (4, 28, 28, 512, 1024, 2),
    (3, 57, 55, 64, 128, 2),     # odd image: the last row and column count
    (6, 40, 40, 32, 64, 3),      # stride 3
])
def test_input_gradient_of_strided_1x1_layers(shape):
    """The input gradient of a strided 1x1 unpadded layer is the stride-1
    gradient over the output pixels, written to the input pixels at multiples
    of the stride, zeros elsewhere: computed dense on the stride-1 kernels and
    scattered in one pass; against the oracle over the whole tensor, every
    element of dX written (the output starts as NaN).  The forward layer
    gathers the pixels it reads and runs on the stride-1 kernels too, bias
    and ReLU included."""
    batch, rows, cols, ch, feats, stride = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 1, stride, False)
    rng = np.random.default_rng(2900 + rows + ch)
    direction = DIRECTION.INPUT_BACKPROP
    n_dy, n_fil, n_dx = ops.conv_sizes(p, direction)
    dy, w = uniform(rng, n_dy), uniform(rng, n_fil)
    ref = ORACLE_FN[direction](dy, w, oracle_params(p, feats), acc64=True)
    out = torch.full((n_dx + 16,), float("nan"), device="cuda")
    out[n_dx:] = 7.0
    for algo in (ALGO.MATMUL, ALGO.IM2COL, ALGO.TILED):
        if not supported(p, direction, algo):
            continue
        out[:n_dx] = float("nan")
        got = ops.conv2d(dev(dy), dev(w), p, direction, algo, out=out[:n_dx])
        assert_close(got.cpu().numpy(), ref,
                     ("strided 1x1 input gradient", ALGO_NAME[algo], shape))
        assert torch.all(out[n_dx:] == 7.0)
    n_x, n_w, n_y = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, bias = uniform(rng, n_x), uniform(rng, feats)
    ref = oracle.conv2d_forward(x, w, oracle_params(p, feats), acc64=True)
    for algo in (ALGO.MATMUL, ALGO.IM2COL, ALGO.TILED):
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        got = ops.conv2d(dev(x), dev(w), p, DIRECTION.FORWARD, algo)
        assert_close(got.cpu().numpy(), ref,
                     ("strided 1x1 forward", ALGO_NAME[algo], shape))
    fused = ops.conv2d_bias_act(dev(x), dev(w), dev(bias), p, ALGO.IM2COL,
                                relu=True)
    want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64), 0)
    assert_close(fused.cpu().numpy(), want.reshape(-1),
                 ("strided 1x1 forward + bias + relu", shape))


@pytest.mark.parametrize("shape", [
    # ragged / edge shapes: odd sizes, C and K not multiples of the tiles,
    # non-square windows and strides, VALID padding
    (3, 13, 17, 5, 7, 3, 3, 1, 1, True),
    (2, 9, 11, 3, 130, 3, 3, 2, 2, True),
    (1, 16, 16, 70, 9, 5, 5, 1, 1, False),
    (2, 12, 10, 8, 8, 3, 1, 1, 1, True),
    (2, 12, 10, 8, 8, 1, 3, 1, 1, True),
    (1, 20, 20, 33, 65, 3, 3, 1, 2, True),
    (2, 7, 7, 16, 16, 7, 7, 1, 1, False),
    (1, 1, 1, 1, 1, 1, 1, 1, 1, False),
    (4, 5, 5, 2, 3, 11, 11, 4, 4, True),
])
@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
def test_ragged_shapes(shape, direction):
    n, h, w, c, k, wr, wc, sr, sc, same = shape
    p = ops.ConvParams(channels=c, features=k, batch=n, in_rows=h, in_cols=w,
                       window_rows=wr, window_cols=wc, stride_rows=sr,
                       stride_cols=sc)
    ops.add_padding_to(p, same)
    algos = FWD_ALGOS if direction == DIRECTION.FORWARD else BK_ALGOS
    conv_case(p, direction, algos, seed=sum(shape[:9]) + direction)


@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP])
@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, same
    (3, 13, 11, 32, 64, True),    # odd sizes: clipped tiles on both edges
    (2, 9, 10, 16, 32, False),    # VALID, single chunk
    (1, 7, 7, 512, 512, True),    # channel range split across work-groups
    (5, 6, 5, 48, 96, True),      # three chunks, three feature blocks
    (2, 30, 4, 64, 32, False),    # narrow image
    # persistent work-groups that walk several units: 680 units of two
    # chunks (a unit boundary every other chunk), clipped tiles, a ragged
    # last tile block
    (40, 33, 31, 32, 64, True),
    (21, 45, 47, 96, 64, False),  # 666 units of six chunks, VALID
])
def test_winograd_fused_shapes(shape, direction):
    batch, rows, cols, ch, feats, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 3, 1, same)
    conv_case(p, direction, [ALGO.WINOGRAD], seed=1300 + rows + ch)


@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP])
@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, win_rows, win_cols, same
    (3, 9, 20, 64, 96, 1, 3, True),     # along columns, MFMA GEMMs
    (3, 20, 9, 64, 96, 3, 1, True),     # along rows
    (2, 7, 13, 32, 64, 1, 3, False),    # VALID, odd output length
    (2, 13, 7, 32, 64, 3, 1, False),
    (4, 6, 11, 5, 7, 1, 3, True),       # channel counts off the MFMA path
    (4, 11, 6, 5, 7, 3, 1, True),
])
def test_winograd_one_dimensional_windows(shape, direction):
    """F(2,3) along the window's axis for 1x3 / 3x1 windows, with the
    recommended workspace (all images in one pass) and with the required one
    (one image per pass)."""
    batch, rows, cols, ch, feats, wr, wc, same = shape
    p = ops.add_padding_to(ops.ConvParams(
        channels=ch, features=feats, batch=batch, in_rows=rows, in_cols=cols,
        window_rows=wr, window_cols=wc, stride_rows=1, stride_cols=1), same)
    rng = np.random.default_rng(1360 + rows * cols + ch)
    n_a, n_b, n_out = ops.conv_sizes(p, direction)
    a, b = uniform(rng, n_a), uniform(rng, n_b)
    ref = ORACLE_FN[direction](a, b, oracle_params(p, feats), acc64=True)
    required, recommended = ops.workspace_size(p, direction, ALGO.WINOGRAD)
    assert 0 < required < recommended
    for elems in (recommended, required):
        ws = torch.empty(elems, dtype=torch.float32, device="cuda")
        got = ops.conv2d(dev(a), dev(b), p, direction, ALGO.WINOGRAD,
                         workspace=ws).cpu().numpy()
        assert_close(got, ref, ("winograd 1-D", shape, direction, elems))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, same
    (3, 13, 11, 32, 64, True),    # odd sizes: clipped dY tiles on both edges
    (2, 9, 10, 16, 32, False),    # VALID, half-empty channel and feature blocks
    (1, 7, 7, 512, 512, True),    # 128 filter blocks, tile range in two slices
    (5, 6, 5, 48, 96, True),      # ragged channel block, ragged feature block
    (2, 30, 4, 64, 36, False),    # narrow image, features not a multiple of 32
    (7, 33, 29, 64, 64, True),    # many slices, ragged last step of a slice
    (4, 16, 16, 18, 20, True),    # channels x2 only, features x4 only
])
def test_winograd_filter_backprop_shapes(shape):
    """The fused F(3x3,2x2) filter gradient: tile-range slices, partial
    channel / feature blocks, images with odd sizes."""
    batch, rows, cols, ch, feats, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 3, 1, same)
    conv_case(p, DIRECTION.FILTER_BACKPROP, [ALGO.WINOGRAD],
              seed=1350 + rows + ch)


@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, same
    (3, 17, 13, 3, 64, 7, 2, True),     # stem-like, ragged image
    (2, 9, 9, 5, 36, 3, 1, True),       # 45 (tap, channel) pairs
    (2, 12, 10, 20, 40, 3, 1, False),   # 180 pairs, features not x64
    (4, 8, 8, 6, 128, 5, 2, True),      # 150 pairs, two feature groups
    (1, 6, 7, 1, 4, 3, 1, True),        # a single channel
    (2, 30, 30, 3, 32, 7, 4, False),    # stride 4
])
def test_small_channel_counts_on_mfma(shape, direction):
    """Channel counts that are not multiples of 4 (forward: scalar gather),
    (tap, channel) ranges that fit one work-group (filter backprop) and
    fewer than 16 channels (input backprop: GEMM per output pixel + tap
    gather when the feature count is a multiple of 32)."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    conv_case(p, direction, [ALGO.IM2COL], seed=1400 + rows + ch)


# ---- full batch-32 shapes: sampled float64 recomputation + linearity --------

def sampled_forward_reference(x, w, p, samples):
    """float64 value of the chosen (n, oy, ox, k) outputs by definition."""
    X = x.reshape(p.batch, p.in_rows, p.in_cols, p.channels).astype(np.float64)
    W = w.reshape(p.window_rows, p.window_cols, p.channels,
                  p.features).astype(np.float64)
    out = np.zeros(len(samples))
    for i, (n, oy, ox, k) in enumerate(samples):
        acc = 0.0
        for r in range(p.window_rows):
            y = oy * p.stride_rows - p.pad_rows + r
            if not 0 <= y < p.in_rows:
                continue
            for s in range(p.window_cols):
                xx = ox * p.stride_cols - p.pad_cols + s
                if not 0 <= xx < p.in_cols:
                    continue
                acc += X[n, y, xx] @ W[r, s, :, k]
        out[i] = acc
    return out


@pytest.mark.parametrize("size,ch,window", [(56, 64, 3), (28, 128, 3),
                                            (14, 256, 3), (7, 512, 3),
                                            (56, 64, 1), (28, 128, 1),
                                            (14, 256, 1), (7, 512, 1)])
def test_full_batch_forward_sampled_and_linear(size, ch, window):
    feats = ch if window == 3 else 4 * ch
    p = ops.conv_params(32, size, size, ch, feats, window, 1, window == 3)
    rng = np.random.default_rng(1000 + size + window)
    n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
    x1, x2, w = uniform(rng, n_in), uniform(rng, n_in), uniform(rng, n_fil)
    samples = np.stack([rng.integers(0, p.batch, 600),
                        rng.integers(0, p.out_rows, 600),
                        rng.integers(0, p.out_cols, 600),
                        rng.integers(0, feats, 600)], axis=1)
    # force image corners and edges into the sample
    samples[:8, 1] = [0, 0, p.out_rows - 1, p.out_rows - 1, 0, p.out_rows - 1,
                      p.out_rows // 2, p.out_rows // 2]
    samples[:8, 2] = [0, p.out_cols - 1, 0, p.out_cols - 1, p.out_cols // 2,
                      p.out_cols // 2, 0, p.out_cols - 1]
    ref = sampled_forward_reference(x1, w, p, samples)
    flat = ((samples[:, 0] * p.out_rows + samples[:, 1]) * p.out_cols +
            samples[:, 2]) * feats + samples[:, 3]
    d1, d2, dw = dev(x1), dev(x2), dev(w)
    scale = max(1.0, float(np.sqrt(np.mean(ref * ref))))
    outs = {}
    for algo in FWD_ALGOS:
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        y1 = ops.conv2d(d1, dw, p, DIRECTION.FORWARD, algo)
        got = y1.cpu().numpy()[flat]
        err = np.abs(got - ref)
        assert np.all(err <= RTOL * np.abs(ref) + ATOL * scale), (
            ALGO_NAME[algo], err.max())
        # linearity: conv(2*x1 - x2) == 2*conv(x1) - conv(x2)
        y2 = ops.conv2d(d2, dw, p, DIRECTION.FORWARD, algo)
        y3 = ops.conv2d(2 * d1 - d2, dw, p, DIRECTION.FORWARD, algo)
        lin = (y3 - (2 * y1 - y2)).abs().max().item()
        assert lin <= 20 * ATOL * scale, (ALGO_NAME[algo], lin)
        outs[algo] = y1
    # every algorithm agrees with Direct over the whole tensor
    base = outs[ALGO.DIRECT]
    for algo, y in outs.items():
        diff = (y - base).abs()
        tol = 2 * (RTOL * base.abs() + ATOL * scale)
        assert bool((diff <= tol).all()), (ALGO_NAME[algo], diff.max().item())


# ---- depthwise ---------------------------------------------------------------

MOBILENET = [(112, 32, 1), (112, 64, 2), (56, 128, 1), (28, 256, 2),
             (14, 512, 1), (7, 1024, 1)]


@pytest.mark.parametrize("size,ch,stride", MOBILENET)
def test_depthwise_mobilenet_all_directions(size, ch, stride):
    p = ops.depthwise_params(2, size, size, ch, 1, 3, stride, True)
    op = oracle_params(p, 1)
    rng = np.random.default_rng(400 + size)
    x = rng.standard_normal(2 * size * size * ch).astype(np.float32)
    w = rng.standard_normal(9 * ch).astype(np.float32)
    dy = rng.standard_normal(2 * p.out_rows * p.out_cols * ch).astype(
        np.float32)
    got = ops.depthwise_conv2d(dev(x), dev(w), p).cpu().numpy()
    assert_close(got, oracle.depthwise_forward(x, w, op), ("dw fwd", size, ch))
    got = ops.depthwise_conv2d(dev(dy), dev(w), p,
                               DIRECTION.INPUT_BACKPROP).cpu().numpy()
    assert_close(got, oracle.depthwise_input_backprop(dy, w, op),
                 ("dw inbk", size, ch))
    got = ops.depthwise_conv2d(dev(x), dev(dy), p,
                               DIRECTION.FILTER_BACKPROP).cpu().numpy()
    assert_close(got, oracle.depthwise_filter_backprop(x, dy, op),
                 ("dw filbk", size, ch))


@pytest.mark.parametrize("shape", [(3, 9, 7, 5, 3, 3, 2, True),
                                   (1, 12, 12, 6, 1, 5, 1, False),
                                   (2, 8, 8, 4, 2, 3, 1, True),
                                   (2, 6, 6, 7, 1, 7, 4, True)])
def test_depthwise_ragged(shape):
    n, h, w_, c, m, win, st, same = shape
    p = ops.depthwise_params(n, h, w_, c, m, win, st, same)
    op = oracle_params(p, m)
    rng = np.random.default_rng(sum(shape[:7]))
    x = rng.standard_normal(n * h * w_ * c).astype(np.float32)
    w = rng.standard_normal(win * win * c * m).astype(np.float32)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c * m).astype(
        np.float32)
    assert_close(ops.depthwise_conv2d(dev(x), dev(w), p).cpu().numpy(),
                 oracle.depthwise_forward(x, w, op), ("dw fwd", shape))
    assert_close(ops.depthwise_conv2d(dev(dy), dev(w), p,
                                      DIRECTION.INPUT_BACKPROP).cpu().numpy(),
                 oracle.depthwise_input_backprop(dy, w, op), ("dw inbk", shape))
    assert_close(ops.depthwise_conv2d(dev(x), dev(dy), p,
                                      DIRECTION.FILTER_BACKPROP).cpu().numpy(),
                 oracle.depthwise_filter_backprop(x, dy, op),
                 ("dw filbk", shape))


@pytest.mark.parametrize("shape", [(2, 13, 11, 8, 1, True),
                                   (3, 14, 14, 64, 2, True),
                                   (1, 12, 10, 4, 2, False),
                                   (2, 12, 12, 8, 2, False),
                                   (2, 33, 20, 12, 1, False),
                                   (5, 5, 37, 16, 2, True),
                                   (1, 3, 3, 256, 1, True),
                                   (2, 29, 6, 132, 1, True)])
def test_depthwise_filter_backprop_row_strips(shape):
    """3x3 filter gradient with four channels per lane: row blocks that run
    past the last output row, odd sizes, both strides and paddings."""
    n, h, w_, c, st, same = shape
    p = ops.depthwise_params(n, h, w_, c, 1, 3, st, same)
    op = oracle_params(p, 1)
    rng = np.random.default_rng(900 + h * w_ + c)
    x = rng.standard_normal(n * h * w_ * c).astype(np.float32)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float32)
    # rows and columns no window touches must not leak in, whatever they hold
    if not same and st == 2:
        xv = x.reshape(n, h, w_, c)
        last_r = (p.out_rows - 1) * st + 3
        last_c = (p.out_cols - 1) * st + 3
        xv[:, last_r:, :, :] = np.inf
        xv[:, :, last_c:, :] = np.inf
    got = ops.depthwise_conv2d(dev(x), dev(dy), p,
                               DIRECTION.FILTER_BACKPROP).cpu().numpy()
    assert_close(got, oracle.depthwise_filter_backprop(x, dy, op),
                 ("dw filbk strips", shape))


@pytest.mark.parametrize("shape", [(2, 9, 7, 8, True),      # pad 1
                                   (3, 14, 14, 64, True),    # pad 0
                                   (1, 12, 10, 4, False),    # unused last row
                                   (2, 33, 21, 12, False),
                                   (5, 5, 37, 16, True),
                                   (1, 3, 3, 256, True),
                                   (40, 30, 31, 128, True)])  # 4-row strips
def test_depthwise_input_backprop_stride2_blocks(shape):
    """3x3 stride-2 input gradient, one 2 x 2 block of dX pixels at a time."""
    n, h, w_, c, same = shape
    p = ops.depthwise_params(n, h, w_, c, 1, 3, 2, same)
    op = oracle_params(p, 1)
    rng = np.random.default_rng(950 + h * w_ + c)
    w = rng.standard_normal(9 * c).astype(np.float32)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float32)
    got = ops.depthwise_conv2d(dev(dy), dev(w), p,
                               DIRECTION.INPUT_BACKPROP).cpu().numpy()
    assert_close(got, oracle.depthwise_input_backprop(dy, w, op),
                 ("dw inbk s2", shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, stride, same
    (64, 50, 45, 64, 1, True),     # ragged last strip, ragged last wave column
    (64, 50, 45, 64, 1, False),    # VALID: window starts at its own column
    (40, 44, 64, 32, 1, True),     # two full wave columns of 32 pixels
    (72, 30, 28, 128, 1, True),    # two pixel lanes per wave
    (48, 61, 59, 32, 2, True),     # stride 2, odd size: padding 1
    (48, 60, 58, 128, 2, False),   # stride 2, VALID
    (32, 57, 57, 64, 2, True),
])
@pytest.mark.parametrize("half", [False, True])
def test_depthwise_tall_strip_kernel(shape, half):
    """Shapes that reach the tall-strip forward kernel (every input vector
    loaded by one lane, window columns of the neighbours read across lanes):
    ragged strips and wave columns, both strides, every padding, and its
    mirrored-tap form as the stride-1 input gradient; fp32 and half (eight
    channels per lane, twice the pixel lanes per wave)."""
    n, h, w_, c, st, same = shape
    p = ops.depthwise_params(n, h, w_, c, 1, 3, st, same)
    op = oracle_params(p, 1)
    rng = np.random.default_rng(sum(shape[:5]) + 5)
    x = rng.standard_normal(n * h * w_ * c).astype(np.float32)
    w = rng.standard_normal(9 * c).astype(np.float32)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float32)
    if half:
        x, w, dy = (a.astype(np.float16).astype(np.float32)
                    for a in (x, w, dy))
        dtype, check = torch.float16, assert_close_f16
    else:
        dtype, check = torch.float32, assert_close
    got = ops.depthwise_conv2d(dev(x, dtype), dev(w, dtype), p)
    check(got.float().cpu().numpy(), oracle.depthwise_forward(x, w, op),
          ("dw tall fwd", shape, half))
    if st == 1:
        got = ops.depthwise_conv2d(dev(dy, dtype), dev(w, dtype), p,
                                   DIRECTION.INPUT_BACKPROP)
        check(got.float().cpu().numpy(),
              oracle.depthwise_input_backprop(dy, w, op),
              ("dw tall inbk", shape, half))


@pytest.mark.parametrize("size,ch,stride", MOBILENET)
def test_depthwise_full_batch_matches_oracle(size, ch, stride):
    """Batch 32: the depthwise oracle is cheap enough to run in full."""
    p = ops.depthwise_params(32, size, size, ch, 1, 3, stride, True)
    rng = np.random.default_rng(500 + size)
    x = rng.standard_normal(32 * size * size * ch).astype(np.float32)
    w = rng.standard_normal(9 * ch).astype(np.float32)
    got = ops.depthwise_conv2d(dev(x), dev(w), p).cpu().numpy()
    assert_close(got, oracle.depthwise_forward(x, w, oracle_params(p, 1)),
                 ("dw fwd b32", size, ch))


# ---- pooling -----------------------------------------------------------------

def test_maxpool_resnet_full_batch_bit_exact():
    """3x3 s2 SAME max pool on [32,112,112,64]: values must be bit-identical;
    so must the argmax implied by them (checked through the gradient)."""
    p = ops.pool_params(32, 112, 112, 64, 3, 2, True)
    assert (p.out_rows, p.pad_rows) == (56, 0)
    rng = np.random.default_rng(600)
    x = rng.standard_normal(32 * 112 * 112 * 64).astype(np.float32)
    op = oracle_params(p, 0)
    dx_ = dev(x)
    y = ops.pooling_forward(dx_, p, POOL_OP.MAX)
    ref = oracle.pool_max_forward(x, op)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    dy = rng.standard_normal(ref.size).astype(np.float32)
    got = ops.pooling_max_grad(dx_, y, dev(dy), p).cpu().numpy()
    # overlapping windows add two or more dY terms; the oracle adds them in
    # output order as the kernel does, so the sums are bit-identical too
    ref_dx = oracle.pool_max_grad(x, ref, dy, op)
    assert np.array_equal(got.view(np.uint32), ref_dx.view(np.uint32))


def test_maxpool_ties_take_first_maximum():
    p = ops.pool_params(1, 6, 6, 4, 3, 2, True)
    x = np.zeros(6 * 6 * 4, dtype=np.float32)  # every window is all ties
    op = oracle_params(p, 0)
    y = ops.pooling_forward(dev(x), p, POOL_OP.MAX)
    dy = np.arange(1, y.numel() + 1, dtype=np.float32)
    got = ops.pooling_max_grad(dev(x), y, dev(dy), p).cpu().numpy()
    assert np.array_equal(got, oracle.pool_max_grad(x, y.cpu().numpy(), dy, op))


def test_avgpool_resnet_full_batch():
    p = ops.pool_params(32, 7, 7, 2048, 7, 1, False)
    assert (p.out_rows, p.out_cols) == (1, 1)
    rng = np.random.default_rng(601)
    x = rng.standard_normal(32 * 7 * 7 * 2048).astype(np.float32)
    got = ops.pooling_forward(dev(x), p, POOL_OP.AVERAGE).cpu().numpy()
    assert_close(got, oracle.pool_avg_forward(x, oracle_params(p, 0)),
                 "avg 7x7 global")
    dy = rng.standard_normal(32 * 2048).astype(np.float32)
    assert_close(ops.pooling_avg_grad(dev(dy), p).cpu().numpy(),
                 oracle.pool_avg_grad(dy, oracle_params(p, 0)), "avg grad")


@pytest.mark.parametrize("shape", [(32, 75, 70, 64, 3, 2, True),
                                   (16, 61, 59, 64, 3, 2, False),
                                   (24, 40, 40, 128, 5, 1, True),
                                   (20, 30, 33, 256, 2, 2, False),
                                   (32, 112, 112, 64, 3, 2, True)])
def test_avgpool_grad_row_strips(shape):
    """Average-pool gradient on tensors large enough for the kernel that
    gives a lane a strip of input rows (8 or 4 rows, ragged last strip)."""
    n, h, w_, c, win, st, same = shape
    p = ops.pool_params(n, h, w_, c, win, st, same)
    rng = np.random.default_rng(700 + h + c)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float32)
    got = ops.pooling_avg_grad(dev(dy), p).cpu().numpy()
    assert_close(got, oracle.pool_avg_grad(dy, oracle_params(p, 0)),
                 ("avg grad strips", shape))


@pytest.mark.parametrize("shape", [(32, 112, 112, 64, True),
                                   (16, 61, 59, 64, False),
                                   (3, 75, 70, 8, True),
                                   (2, 8, 9, 4, True),
                                   (2, 7, 7, 12, False),
                                   (1, 3, 3, 4, False),
                                   (5, 30, 31, 32, True)])
def test_avgpool_grad_3x3_stride2_bit_exact(shape):
    """The block-row kernel for the 3x3 stride-2 average gradient adds the
    window terms in the reference's order, so it must reproduce the oracle's
    fp32 reference-order mode bit for bit (even / odd sizes, SAME and VALID
    padding, both strip heights, signed zeros in dY)."""
    n, h, w_, c, same = shape
    p = ops.pool_params(n, h, w_, c, 3, 2, same)
    rng = np.random.default_rng(900 + h + w_ + c)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float32)
    dy[::97] = 0.0
    dy[5::89] = -0.0
    got = ops.pooling_avg_grad(dev(dy), p).cpu().numpy()
    ref = oracle.pool_avg_grad(dy, oracle_params(p, 0), acc64=False)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), shape


@pytest.mark.parametrize("shape", [(2, 9, 7, 5, 3, 2, True),
                                   (1, 11, 11, 3, 5, 1, True),
                                   (3, 8, 8, 8, 2, 2, False),
                                   (2, 13, 13, 6, 11, 4, True)])
def test_pooling_ragged(shape):
    n, h, w_, c, win, st, same = shape
    p = ops.pool_params(n, h, w_, c, win, st, same)
    op = oracle_params(p, 0)
    rng = np.random.default_rng(sum(shape[:6]))
    x = rng.standard_normal(n * h * w_ * c).astype(np.float32)
    y = ops.pooling_forward(dev(x), p, POOL_OP.MAX)
    assert np.array_equal(y.cpu().numpy(), oracle.pool_max_forward(x, op))
    assert_close(ops.pooling_forward(dev(x), p, POOL_OP.AVERAGE).cpu().numpy(),
                 oracle.pool_avg_forward(x, op), ("avg", shape))
    dy = rng.standard_normal(y.numel()).astype(np.float32)
    assert_close(ops.pooling_max_grad(dev(x), y, dev(dy), p).cpu().numpy(),
                 oracle.pool_max_grad(x, y.cpu().numpy(), dy, op),
                 ("max grad", shape))
    assert_close(ops.pooling_avg_grad(dev(dy), p).cpu().numpy(),
                 oracle.pool_avg_grad(dy, op), ("avg grad", shape))


@pytest.mark.parametrize("channels", [8, 6])
def test_pooling_window_wholly_outside_the_image(channels):
    """Output sizes larger than the input implies are not rejected (nor are
    they by the reference's validation, include/portdnn/pooling/launch.h:56-88),
    so the last output row and column here own windows that lie outside the
    image on both axes.  Such a window has no elements: the reference's
    operators leave Max at lowest() and divide 0 by 0 for Average
    (src/pooling/operators_impl.h:27-87).  Eight channels take the kernel that
    deals window taps to lanes (16 taps), six the generic one."""
    p = ops.pool_params(2, 7, 7, channels, 4, 4, False)
    p.out_rows = p.out_cols = 3      # third window starts at row / column 8
    op = oracle_params(p, 0)
    rng = np.random.default_rng(77 + channels)
    x = rng.standard_normal(2 * 7 * 7 * channels).astype(np.float32)
    got = ops.pooling_forward(dev(x), p, POOL_OP.MAX).cpu().numpy()
    ref = oracle.pool_max_forward(x, op)
    assert np.array_equal(got, ref)
    assert ref.reshape(2, 3, 3, channels)[0, 2, 2, 0] == \
        np.finfo(np.float32).min
    got = ops.pooling_forward(dev(x), p, POOL_OP.AVERAGE).cpu().numpy()
    with np.errstate(invalid="ignore"):
        ref = oracle.pool_avg_forward(x, op)
    assert np.isnan(ref.reshape(2, 3, 3, channels)[:, 2, :, :]).all()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    ok = ~np.isnan(ref)
    assert_close(got[ok], ref[ok], "avg outside")


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, same
    (48, 61, 59, 32, True),     # odd size: padding 1, ragged strip and wave column
    (40, 60, 58, 128, False),   # VALID, two pixel lanes per wave
    (32, 57, 57, 64, True),
    (32, 112, 112, 64, True),   # the benchmark layer
])
def test_pooling_3x3_stride2_tall_strip_kernel(shape):
    """Shapes that reach the tall-strip 3x3 stride-2 forward kernel (a lane
    loads two window columns and reads the third from the next pixel lane):
    maxima bit-exact with and without NaNs in the data under both NaN rules,
    the average against the oracle."""
    n, h, w_, c, same = shape
    p = ops.pool_params(n, h, w_, c, 3, 2, same)
    op = oracle_params(p, 0)
    rng = np.random.default_rng(sum(shape[:4]) + 9)
    x = rng.standard_normal(n * h * w_ * c).astype(np.float32)
    got = ops.pooling_forward(dev(x), p, POOL_OP.MAX).cpu().numpy()
    assert np.array_equal(got, oracle.pool_max_forward(x, op)), shape
    assert_close(ops.pooling_forward(dev(x), p, POOL_OP.AVERAGE).cpu().numpy(),
                 oracle.pool_avg_forward(x, op), ("avg tall", shape))
    if n * h * w_ * c < 30_000_000:
        x[rng.integers(0, x.size, x.size // 50)] = np.nan
        for pool_op, nan_mode in ((POOL_OP.MAX, False),
                                  (POOL_OP.MAX_WITH_NAN, True)):
            got = ops.pooling_forward(dev(x), p, pool_op).cpu().numpy()
            ref = oracle.pool_max_forward(x, op, nan_mode=nan_mode)
            assert np.array_equal(got, ref, equal_nan=True), (shape, nan_mode)
            assert np.isnan(ref).any() == nan_mode


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, window, stride, same
    (2, 37, 41, 12, 3, 2, True),     # ragged 16 x 16 tiles, 3 channel vectors
    (1, 33, 17, 72, 3, 2, False),    # two channel groups, VALID
    (3, 19, 23, 8, 3, 1, True),      # stride 1: every element in 9 windows
    (2, 30, 18, 20, 2, 2, False),    # disjoint windows
    (1, 16, 16, 4, 3, 2, True),      # exactly one tile
    (32, 90, 75, 64, 3, 2, True),    # 3x3 s2 with four block rows per lane
    (64, 90, 90, 64, 3, 2, False),   # ... with fourteen, VALID
    (16, 91, 78, 128, 3, 2, True),   # ... odd rows, ragged last strip
    (3, 21, 20, 16, 3, 2, False),    # 3x3 s2 VALID, unused last column
])
@pytest.mark.parametrize("nan_mode", [False, True])
def test_maxpool_grad_tiled_kernel(shape, nan_mode):
    """The specialised max gradients (3x3 s2 by 2 x 2 blocks of dX pixels,
    3x3 s1 and 2x2 s2 by work-group tiles, channels % 4 == 0): small integers
    make most windows tie, some NaNs test both NaN rules; results must equal
    the oracle exactly."""
    n, h, w_, c, win, st, same = shape
    p = ops.pool_params(n, h, w_, c, win, st, same)
    op = oracle_params(p, 0)
    rng = np.random.default_rng(1300 + h * w_ + c)
    x = rng.integers(-2, 3, n * h * w_ * c).astype(np.float32)
    x[rng.integers(0, x.size, x.size // 50)] = np.nan
    gpu_op = POOL_OP.MAX_WITH_NAN if nan_mode else POOL_OP.MAX
    y = ops.pooling_forward(dev(x), p, gpu_op)
    ref_y = oracle.pool_max_forward(x, op, nan_mode)
    assert np.array_equal(y.cpu().numpy(), ref_y, equal_nan=True)
    dy = rng.integers(1, 9, ref_y.size).astype(np.float32)
    got = ops.pooling_max_grad(dev(x), y, dev(dy), p, gpu_op).cpu().numpy()
    assert np.array_equal(got, oracle.pool_max_grad(x, ref_y, dy, op, nan_mode))


def test_maxpool_nan_rules():
    """test/pooling/max_pooling_with_nan.cc: Max drops NaNs, MaxWithNan
    propagates them (forward and gradient)."""
    p = ops.pool_params(1, 4, 4, 4, 2, 2, False)
    op = oracle_params(p, 0)
    rng = np.random.default_rng(9)
    x = rng.standard_normal(64).astype(np.float32)
    x[[3, 17, 18, 40, 41, 44, 45]] = np.nan
    for gpu_op, nan_mode in ((POOL_OP.MAX, False), (POOL_OP.MAX_WITH_NAN, True)):
        y = ops.pooling_forward(dev(x), p, gpu_op)
        ref = oracle.pool_max_forward(x, op, nan_mode)
        assert np.array_equal(y.cpu().numpy(), ref, equal_nan=True)
        assert np.isnan(ref).any() == nan_mode
        dy = np.arange(1, 17, dtype=np.float32)
        got = ops.pooling_max_grad(dev(x), y, dev(dy), p, gpu_op).cpu().numpy()
        assert np.array_equal(got, oracle.pool_max_grad(x, ref, dy, op,
                                                        nan_mode))


@pytest.mark.parametrize("shape", [(2, 13, 11, 8, 3, 2, True),
                                   (1, 12, 12, 5, 2, 2, False),
                                   (2, 9, 9, 16, 3, 1, True)])
def test_f16_pooling_gradients(shape):
    """Half-precision pooling gradients: the maximum is exact in half, so the
    max gradient must equal the oracle on the same half values bit for bit;
    the average gradient within the half tolerance."""
    n, h, w_, c, win, st, same = shape
    p = ops.pool_params(n, h, w_, c, win, st, same)
    op = oracle_params(p, 0)
    rng = np.random.default_rng(1400 + h + c)
    x = rng.integers(-3, 4, n * h * w_ * c).astype(np.float16)
    y = ops.pooling_forward(dev(x, torch.float16), p, POOL_OP.MAX)
    ref_y = oracle.pool_max_forward(x.astype(np.float32), op)
    assert np.array_equal(y.float().cpu().numpy(), ref_y)
    dy = rng.integers(1, 9, ref_y.size).astype(np.float16)
    got = ops.pooling_max_grad(dev(x, torch.float16), y,
                               dev(dy, torch.float16), p)
    assert np.array_equal(got.float().cpu().numpy(),
                          oracle.pool_max_grad(x.astype(np.float32), ref_y,
                                               dy.astype(np.float32), op))
    got = ops.pooling_avg_grad(dev(dy, torch.float16), p)
    assert_close_f16(got.float().cpu().numpy(),
                     oracle.pool_avg_grad(dy.astype(np.float32), op),
                     ("f16 avg grad", shape))


# ---- matmul ------------------------------------------------------------------

@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("shape", [(1, 64, 64, 64), (3, 37, 29, 53),
                                   (1, 1568, 512, 2048), (2, 130, 7, 258),
                                   (16, 200, 64, 64), (3, 100, 96, 50),
                                   (1, 4096, 1024, 1024), (2, 33, 32, 3),
                                   # large and odd: repacked for the
                                   # matrix-core kernel (k -> 32s, n -> 4s)
                                   (1, 2047, 1023, 1001), (1, 512, 4096, 30),
                                   (1, 4096, 512, 10)])
def test_matmul(trans_a, trans_b, shape):
    b_, m, k, n = shape
    rng = np.random.default_rng(sum(shape))
    a, b = uniform(rng, b_ * m * k), uniform(rng, b_ * k * n)
    c0 = uniform(rng, b_ * m * n)
    for beta in (0.0, 1.0, -0.5):
        ref = oracle.matmul(a, b, b_, m, k, n, trans_a, trans_b, beta, c=c0)
        got = ops.matmul(dev(a), dev(b), b_, m, k, n, trans_a, trans_b, beta,
                         out=dev(c0).clone()).cpu().numpy()
        assert_close(got, ref, ("matmul", shape, trans_a, trans_b, beta))


@pytest.mark.parametrize("shape", [
    # m, k, n of A^T B with A stored [k x m]
    (64, 25088, 256),    # one row of tiles, the reduction split 64 ways
    (128, 1001, 192),    # k not a multiple of 4
    (64, 263, 64),       # a single tile
    (1024, 2048, 1024),  # more tiles than compute units
])
def test_matmul_transposed_lhs_on_the_filter_gradient_kernel(shape):
    """A^T * B with m and n multiples of 64 is the filter gradient of a 1x1
    convolution over k pixels and runs on its matrix-core kernel; nothing is
    written past the result."""
    m, k, n = shape
    rng = np.random.default_rng(sum(shape) + 23)
    a, b = uniform(rng, k * m), uniform(rng, k * n)
    ref = oracle.matmul(a, b, 1, m, k, n, True, False, 0.0)
    out = torch.full((m * n + 64,), 7.0, device="cuda")
    got = ops.matmul(dev(a), dev(b), 1, m, k, n, True, False, 0.0,
                     out=out[:m * n])
    assert_close(got.cpu().numpy(), ref, ("matmul A^T B", shape))
    assert torch.all(out[m * n:] == 7.0)
    again = ops.matmul(dev(a), dev(b), 1, m, k, n, True, False, 0.0)
    assert torch.equal(got.view(torch.int32), again.view(torch.int32))


@pytest.mark.parametrize("shape", [
    # batches, m, k, n: shapes that take the plain-rows kernel
    (1, 6390, 256, 1000),   # 112-row tiles: 57 full + 6 rows, 24 columns short
    (1, 16390, 64, 252),    # 64-row tiles, ragged last row tile and column tile
    (3, 6272, 128, 128),    # batched, short LDS stages
    (1, 25088, 96, 512),    # three chunks
])
def test_matmul_plain_rows_kernel(shape):
    """The 16x16x4 MFMA kernel behind A * B with 16-byte fetches and stores:
    both tilings, ragged rows and columns, batches."""
    b_, m, k, n = shape
    rng = np.random.default_rng(sum(shape) + 11)
    a, b = uniform(rng, b_ * m * k), uniform(rng, b_ * k * n)
    ref = oracle.matmul(a, b, b_, m, k, n, False, False, 0.0)
    got = ops.matmul(dev(a), dev(b), b_, m, k, n, False, False, 0.0)
    assert_close(got.cpu().numpy(), ref, ("matmul rows", shape))


@pytest.mark.parametrize("shape", [
    # m, k, n -> (pixel blocks per tile, feature blocks per wave) of the plan
    (16390, 64, 256),    # (2, 1), ragged last tile
    (40000, 64, 512),    # (2, 2)
    (12005, 128, 256),   # (1, 1), ragged
    (28923, 128, 128),   # (2, 1)
    (14965, 128, 256),   # (1, 2)
    (20000, 128, 512),   # (2, 2)
    (4100, 256, 1024),   # (1, 1), eight feature slices
    (28923, 256, 128),   # (2, 1)
    (14965, 256, 256),   # (1, 2)
    (30917, 256, 256),   # (2, 2)
    (3000, 512, 1024),   # 512 reduction steps
    (3137, 128, 2048),   # sixteen feature slices
])
def test_matmul_filter_in_registers_kernel(shape):
    """A * B with k = 64 / 128 / 256 / 512 and n in whole feature slices runs on
    the persistent kernel that keeps B in registers: every tiling it builds,
    row counts that end inside a tile, 1 to 16 feature slices."""
    m, k, n = shape
    rng = np.random.default_rng(sum(shape) + 17)
    a, b = uniform(rng, m * k), uniform(rng, k * n)
    ref = oracle.matmul(a, b, 1, m, k, n, False, False, 0.0)
    out = torch.full((m * n + 64,), 7.0, device="cuda")
    got = ops.matmul(dev(a), dev(b), 1, m, k, n, False, False, 0.0,
                     out=out[:m * n])
    assert_close(got.cpu().numpy(), ref, ("matmul, filter in registers", shape))
    # nothing is written past the last row
    assert torch.all(out[m * n:] == 7.0)


@pytest.mark.parametrize("shape", [
    (12, 56, 56, 256, 64),   # 64 features: four feature waves x two pixel halves
    (12, 55, 57, 64, 64),    # ... with a row count that ends inside a tile
    (13, 56, 56, 128, 64),
    (32, 28, 28, 512, 128),  # its input gradient: reduction 128, 512 columns
    (16, 56, 56, 64, 256),   # input gradient: reduction 256, 64 columns
])
def test_conv1x1_narrow_filters_and_input_gradient_in_registers(shape):
    """1x1 convolutions with 64 features, and the input gradient of 1x1
    convolutions with up to 256 features (dX = dY * W^T, the filter read with
    its feature index as the reduction), run on the filter-in-registers kernel
    too: against the oracle, forward also with bias and ReLU folded in."""
    batch, rows, cols, ch, feats = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 1, 1, False)
    rng = np.random.default_rng(6262 + ch + feats)
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
        n_in, n_fil, _ = ops.conv_sizes(p, direction)
        a, w = uniform(rng, n_in), uniform(rng, n_fil)
        ref = ORACLE_FN[direction](a, w, oracle_params(p, feats), acc64=True)
        da, dw = dev(a), dev(w)
        for algo in (ALGO.MATMUL, ALGO.IM2COL):
            got = ops.conv2d(da, dw, p, direction, algo)
            assert_close(got.cpu().numpy(), ref,
                         ("1x1", ALGO_NAME[algo], direction, shape))
        if direction == DIRECTION.FORWARD:
            bias = uniform(rng, feats) * 4
            got = ops.conv2d_bias_act(da, dw, dev(bias), p, ALGO.MATMUL,
                                      relu=True)
            want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64),
                              0)
            assert_close(got.cpu().numpy(), want.reshape(-1),
                         ("1x1 + bias + relu", shape))


@pytest.mark.parametrize("shape", [(4, 56, 56, 64, 256), (6, 28, 28, 128, 512),
                                   (12, 14, 14, 256, 1024),
                                   (32, 7, 7, 512, 2048)])
def test_conv1x1_filter_in_registers_bias_relu(shape):
    """1x1 convolutions on the same kernel with its fused epilogue: equal to
    the plain launch followed by the bias addition and the ReLU, and to the
    oracle."""
    batch, rows, cols, ch, feats = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 1, 1, False)
    rng = np.random.default_rng(5151 + ch)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = uniform(rng, n_in), uniform(rng, n_fil)
    bias = uniform(rng, feats) * 4
    dx, dw, db = dev(x), dev(w), dev(bias)
    plain = ops.conv2d(dx, dw, p, DIRECTION.FORWARD, ALGO.MATMUL)
    ref = oracle.conv2d_forward(x, w, oracle_params(p, feats), acc64=True)
    assert_close(plain.cpu().numpy(), ref, ("1x1, filter in registers", shape))
    want = torch.relu(plain.view(-1, feats) + db).view(-1)
    got = ops.conv2d_bias_act(dx, dw, db, p, ALGO.MATMUL, relu=True)
    assert torch.equal(got, want)
    got = ops.conv2d_bias_act(dx, dw, db, p, ALGO.MATMUL, relu=False)
    assert torch.equal(got, (plain.view(-1, feats) + db).view(-1))
    got = ops.conv2d_bias_act(dx, dw, None, p, ALGO.MATMUL, relu=True)
    assert torch.equal(got, torch.relu(plain))


def test_plain_rows_kernel_bias_relu_on_tall_tiles():
    """14x14x192 -> 1024 at batch 32 runs on 112-row tiles of the plain-rows
    kernel; the fused bias + ReLU epilogue must equal the convolution followed
    by the two steps."""
    p = ops.conv_params(32, 14, 14, 192, 1024, 1, 1, False)
    rng = np.random.default_rng(4343)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = uniform(rng, n_in), uniform(rng, n_fil)
    bias = uniform(rng, 1024) * 4
    dx, dw, db = dev(x), dev(w), dev(bias)
    plain = ops.conv2d(dx, dw, p, DIRECTION.FORWARD, ALGO.MATMUL)
    ref = oracle.conv2d_forward(x, w, oracle_params(p, 1024), acc64=True)
    assert_close(plain.cpu().numpy(), ref, "1x1 on tall tiles")
    want = torch.relu(plain.view(-1, 1024) + db).view(-1)
    got = ops.conv2d_bias_act(dx, dw, db, p, ALGO.MATMUL, relu=True)
    assert torch.equal(got, want)
    got = ops.conv2d_bias_act(dx, dw, db, p, ALGO.MATMUL, relu=False)
    assert torch.equal(got, (plain.view(-1, 1024) + db).view(-1))


def test_many_tiles_per_work_group_epilogue_and_accumulate():
    """Launches with thousands of 64 x 64 tiles make the implicit-GEMM
    work-groups walk several tiles each.  At that size: the fused bias + ReLU
    epilogue must equal the Direct convolution followed by the two element-wise
    steps, and a matmul that accumulates (beta = 1) must equal the plain
    product plus the previous contents; a small slice is checked against the
    oracle as well."""
    p = ops.conv_params(32, 56, 56, 64, 256, 1, 1, False)
    rng = np.random.default_rng(4242)
    n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = uniform(rng, n_in), uniform(rng, n_fil)
    bias = uniform(rng, 256) * 4
    dx, dw, db = dev(x), dev(w), dev(bias)
    base = ops.conv2d(dx, dw, p, DIRECTION.FORWARD, ALGO.DIRECT)
    want = torch.relu(base.view(-1, 256) + db).view(-1)
    scale = max(1.0, float(base.pow(2).mean().sqrt()))
    for algo in (ALGO.MATMUL, ALGO.IM2COL, ALGO.TILED):
        got = ops.conv2d_bias_act(dx, dw, db, p, algo, relu=True)
        diff = (got - want).abs()
        assert bool((diff <= 2 * (RTOL * want.abs() + ATOL * scale)).all()), (
            ALGO_NAME[algo], diff.max().item())
    # first 64 pixels against the oracle (1x1: rows of a GEMM)
    ref = oracle.matmul(x[:64 * 64], w, 1, 64, 64, 256, False, False, 0.0)
    ref = np.maximum(ref.reshape(64, 256) + bias, 0).reshape(-1)
    got = ops.conv2d_bias_act(dx, dw, db, p, ALGO.MATMUL, relu=True)
    assert_close(got[:64 * 256].cpu().numpy(), ref, "bias_act slice")

    m, k, n = 100352, 64, 256
    c0 = dev(uniform(rng, m * n))
    plain = ops.matmul(dx, dw, 1, m, k, n, False, False, 0.0,
                       out=torch.empty(m * n, device="cuda"))
    acc = ops.matmul(dx, dw, 1, m, k, n, False, False, 1.0, out=c0.clone())
    diff = (acc - (plain + c0)).abs()
    assert bool((diff <= 2 * (RTOL * (plain + c0).abs() + ATOL * scale)).all())
    assert_close(plain[:64 * 256].cpu().numpy(),
                 oracle.matmul(x[:64 * 64], w, 1, 64, 64, 256, False, False,
                               0.0), "matmul slice")


@pytest.mark.parametrize("shape", [
    # m, k, n -> (k / 32, pixel blocks per tile, feature blocks per wave)
    (50977, 64, 256),    # (2, 4, 2), ragged last tile
    (58973, 64, 512),    # (2, 4, 4)
    (24990, 128, 256),   # (4, 2, 2)
    (28988, 128, 512),   # (4, 2, 4)
    (12996, 256, 256),   # (8, 1, 2)
    (14995, 256, 512),   # (8, 1, 4)
    (28988, 256, 256),   # (8, 2, 2)
    (30987, 256, 512),   # (8, 2, 4)
    (12996, 512, 256),   # (16, 1, 2)
    (28988, 512, 256),   # (16, 2, 2)
    (6272, 512, 2048),   # eight feature slices, one XCD per slice
])
def test_matmul_f16_filter_in_registers_kernel(shape):
    """Half-precision A * B with k = 64 / 128 / 256 / 512 on the persistent kernel
    that keeps B in registers (transposed there from its feature-contiguous
    layout): every tiling it builds, row counts that end inside a tile."""
    m, k, n = shape
    rng = np.random.default_rng(sum(shape) + 23)
    a = uniform(rng, m * k).astype(np.float16)
    b = uniform(rng, k * n).astype(np.float16)
    ref = oracle.matmul(a.astype(np.float32), b.astype(np.float32), 1, m, k, n,
                        False, False, 0.0)
    out = torch.full((m * n + 64,), 7.0, device="cuda", dtype=torch.float16)
    got = ops.matmul(dev(a, torch.float16), dev(b, torch.float16), 1, m, k, n,
                     False, False, 0.0, out=out[:m * n])
    assert_close_f16(got.float().cpu().numpy(), ref,
                     ("matmul f16, filter in registers", shape))
    # nothing is written past the last row
    assert torch.all(out[m * n:] == 7.0)


@pytest.mark.parametrize("shape", [(1, 256, 128, 192), (1, 100, 64, 64),
                                   (3, 33, 20, 17), (1, 2048, 256, 512)])
@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
def test_matmul_f16(trans_a, trans_b, shape):
    """Half-precision matmul (fp32 accumulation): matrix-core shapes and the
    general kernel, against the oracle on the same half-rounded operands."""
    b_, m, k, n = shape
    rng = np.random.default_rng(sum(shape) + 7)
    a = uniform(rng, b_ * m * k).astype(np.float16)
    b = uniform(rng, b_ * k * n).astype(np.float16)
    c0 = uniform(rng, b_ * m * n).astype(np.float16)
    for beta in (0.0, 1.0):
        ref = oracle.matmul(a.astype(np.float32), b.astype(np.float32), b_, m,
                            k, n, trans_a, trans_b, beta,
                            c=c0.astype(np.float32))
        got = ops.matmul(dev(a, torch.float16), dev(b, torch.float16), b_, m,
                         k, n, trans_a, trans_b, beta,
                         out=dev(c0, torch.float16).clone())
        assert_close_f16(got.float().cpu().numpy(), ref,
                         ("matmul f16", shape, trans_a, trans_b, beta))


@pytest.mark.parametrize("shape", [
    # rows, reduction, columns of the row-major half-precision GEMM
    (6272, 64, 256),     # one slab, X kept in registers for both column groups
    (3136, 128, 512),    # two chunks resident, four column groups, tail jobs
    (1000, 128, 384),    # three column groups, rows not a multiple of 32
    (1568, 256, 1024),   # streamed X, four slabs
    (490, 512, 2048),    # sixteen slabs of 128 columns
    (777, 192, 192),     # 64-column groups (two interleaved features per lane)
    (65, 64, 64),        # a single 64-column group
    (1, 64, 128),        # one row
    (4097, 1024, 64),    # long reduction, narrow slab
])
def test_f16_rows_gemm_slab_kernel(shape):
    """1x1 stride-1 half-precision convolution / matmul on the kernel that
    keeps the filter slab in LDS: every driver (X resident for 64 and 128
    channels, streamed above), both column-group widths, ragged row counts and
    several slabs, against the fp64 product of the same half-rounded operands.
    Tolerance 1e-2 relative (rms-floored), the half-precision bar."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n)
    a = uniform(rng, m * k).astype(np.float16)
    b = uniform(rng, k * n).astype(np.float16)
    ref = (a.astype(np.float64).reshape(m, k) @
           b.astype(np.float64).reshape(k, n)).reshape(-1)
    got = ops.matmul(dev(a, torch.float16), dev(b, torch.float16), 1, m, k, n,
                     False, False, 0.0)
    assert_close_f16(got.float().cpu().numpy(), ref, ("rows f16 matmul", shape))
    # the same product as a convolution over an image of m pixels
    p = ops.conv_params(1, 1, m, k, n, 1, 1, False)
    out = ops.conv2d(dev(a, torch.float16), dev(b, torch.float16), p,
                     DIRECTION.FORWARD, ALGO.MATMUL)
    assert_close_f16(out.float().cpu().numpy(), ref, ("rows f16 conv", shape))


# ---- f16 ---------------------------------------------------------------------

def assert_close_f16(got, ref, what):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    scale = max(1.0, float(np.sqrt(np.mean(ref * ref))))
    err = np.abs(got - ref)
    assert np.all(err <= 1e-2 * np.maximum(np.abs(ref), scale)), (
        what, err.max())


@pytest.mark.parametrize("size,ch,window", [(56, 64, 3), (14, 256, 3),
                                            (7, 512, 3), (28, 128, 1)])
def test_f16_conv_forward(size, ch, window):
    feats = ch if window == 3 else 4 * ch
    p = ops.conv_params(2, size, size, ch, feats, window, 1, window == 3)
    rng = np.random.default_rng(700 + size)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x = uniform(rng, n_in).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    ref = oracle.conv2d_forward(x.astype(np.float32), w.astype(np.float32),
                                oracle_params(p, feats), acc64=True)
    for algo in FWD_ALGOS:
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        got = ops.conv2d(dev(x, torch.float16), dev(w, torch.float16), p,
                         DIRECTION.FORWARD, algo).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16", ALGO_NAME[algo], size, ch))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, same
    (3, 13, 11, 64, 40, 3, 1, True),     # ragged rows, features not x32
    (2, 17, 9, 128, 72, 3, 2, True),     # stride 2
    (1, 9, 9, 64, 200, 5, 1, False),     # VALID, 25 taps
    (5, 7, 7, 192, 8, 1, 1, False),      # 1x1, three chunks per tap
    (2, 33, 31, 64, 130, 3, 2, False),   # features just past two tiles
    (2, 17, 9, 128, 80, 3, 2, True),     # 16-byte stores, half a block masked
    (5, 7, 7, 192, 48, 1, 1, False),     # 1x1, 16-byte stores, ragged rows
    (3, 10, 10, 64, 272, 3, 2, True),    # 16-byte stores past two tiles
])
def test_f16_conv_forward_ragged(shape):
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(750 + rows)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x = uniform(rng, n_in).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    ref = oracle.conv2d_forward(x.astype(np.float32), w.astype(np.float32),
                                oracle_params(p, feats), acc64=True)
    for algo in (ALGO.IM2COL, ALGO.DIRECT):
        got = ops.conv2d(dev(x, torch.float16), dev(w, torch.float16), p,
                         DIRECTION.FORWARD, algo).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16 ragged", ALGO_NAME[algo], shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, win_rows, win_cols, same
    (5, 7, 7, 128, 64, 3, 3, True),      # tiles run over image boundaries
    (3, 14, 14, 64, 128, 3, 3, True),    # one channel block, two wave rows
    (2, 28, 28, 192, 192, 3, 3, True),   # three channel blocks, 64-wide slice
    (3, 12, 10, 128, 128, 5, 5, True),   # 25 taps, pad 2
    (2, 11, 13, 64, 64, 3, 3, False),    # VALID
    (2, 9, 20, 128, 256, 1, 3, True),    # 1 x 3 window
    (2, 20, 9, 128, 64, 3, 1, True),     # 3 x 1 window
    (7, 5, 5, 256, 320, 1, 1, False),    # 1x1, four channel blocks
    (1, 6, 200, 64, 64, 3, 3, True),     # rows wider than half a tile
    (130, 3, 3, 128, 128, 3, 3, True),   # many images per tile
])
def test_f16_conv_forward_lds_tile_kernel(shape):
    batch, rows, cols, ch, feats, wr, wc, same = shape
    p = ops.add_padding_to(ops.ConvParams(
        channels=ch, features=feats, batch=batch, in_rows=rows, in_cols=cols,
        window_rows=wr, window_cols=wc, stride_rows=1, stride_cols=1), same)
    rng = np.random.default_rng(770 + rows * cols)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x = uniform(rng, n_in).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    ref = oracle.conv2d_forward(x.astype(np.float32), w.astype(np.float32),
                                oracle_params(p, feats), acc64=True)
    got = ops.conv2d(dev(x, torch.float16), dev(w, torch.float16), p,
                     DIRECTION.FORWARD, ALGO.IM2COL).float().cpu().numpy()
    assert_close_f16(got, ref, ("f16 lds tile", shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, SAME
    (8, 28, 28, 144, 144, 3, 1, True),   # channels not a multiple of 64
    (4, 28, 28, 100, 100, 5, 1, True),
    (8, 32, 32, 16, 16, 3, 1, True),
    (8, 56, 56, 12, 20, 3, 2, True),
    (2, 56, 56, 64, 64, 7, 1, True),     # 49 taps
    (8, 17, 19, 40, 72, 1, 1, False),
])
def test_f16_conv_forward_general_kernel(shape):
    """Half-precision forward convolutions outside the binary16 kernels'
    shapes (channel counts that are not multiples of 64, more than 32 taps)
    run on the general implicit-GEMM kernel reading binary16 operands with
    fp32 accumulation, not one lane per output: against the oracle in double
    precision on the same half-rounded operands; nothing written past the
    result."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(770 + rows + ch + window)
    n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
    x = uniform(rng, n_in).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    ref = oracle.conv2d_forward(x.astype(np.float32), w.astype(np.float32),
                                oracle_params(p, feats), acc64=True)
    out = torch.full((n_out + 16,), 7.0, dtype=torch.float16, device="cuda")
    for algo in (ALGO.IM2COL, ALGO.TILED):
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        got = ops.conv2d(dev(x, torch.float16), dev(w, torch.float16), p,
                         DIRECTION.FORWARD, algo, out=out[:n_out])
        assert_close_f16(got.float().cpu().numpy(), ref,
                         ("f16 general forward", ALGO_NAME[algo], shape))
        assert torch.all(out[n_out:] == 7.0)


@pytest.mark.parametrize("size,ch,feats,window", [
    (28, 128, 128, 3),   # LDS-tile kernel, four channel blocks
    (56, 64, 64, 3),     # LDS-tile kernel, one channel block
    (7, 512, 512, 3),    # LDS-tile kernel, 64 x 64 wave tiles
    (28, 128, 512, 1),   # implicit-GEMM kernel, 128 x 128 work-group tile
])
def test_f16_conv_forward_full_batch_sampled(size, ch, feats, window):
    p = ops.conv_params(128, size, size, ch, feats, window, 1, window == 3)
    rng = np.random.default_rng(760 + size)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x = uniform(rng, n_in).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    got = ops.conv2d(dev(x, torch.float16), dev(w, torch.float16), p,
                     DIRECTION.FORWARD, ALGO.IM2COL).float().cpu().numpy()
    samples = np.stack([rng.integers(0, p.batch, 800),
                        rng.integers(0, p.out_rows, 800),
                        rng.integers(0, p.out_cols, 800),
                        rng.integers(0, p.features, 800)], axis=1)
    samples[:4, 1] = [0, 0, p.out_rows - 1, p.out_rows - 1]
    samples[:4, 2] = [0, p.out_cols - 1, 0, p.out_cols - 1]
    samples[:4, 0] = [0, p.batch - 1, p.batch - 1, 0]
    ref = sampled_forward_reference(x, w, p, samples)
    flat = ((samples[:, 0] * p.out_rows + samples[:, 1]) * p.out_cols +
            samples[:, 2]) * p.features + samples[:, 3]
    assert_close_f16(got[flat], ref, ("f16 batch 128 sampled", size, window))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, win_rows, win_cols, stride, same
    (3, 14, 14, 64, 128, 3, 3, 1, True),    # LDS-tile kernel on dY
    (2, 28, 28, 192, 64, 3, 3, 1, True),    # three feature blocks reduced
    (2, 11, 13, 64, 64, 3, 3, 1, False),    # VALID: padding 2 on dY
    (3, 12, 10, 128, 128, 5, 5, 1, True),   # 25 mirrored taps
    (2, 9, 20, 128, 256, 1, 3, 1, True),    # 1 x 3 window
    (7, 5, 5, 256, 320, 1, 1, 1, False),    # 1x1: implicit-GEMM kernel
    (2, 28, 28, 128, 512, 1, 1, 1, False),  # 1x1, 128 x 128 tiles
    (2, 17, 9, 128, 64, 3, 3, 2, True),     # stride 2: general MFMA kernel
    (2, 8, 8, 24, 40, 3, 3, 1, True),       # few channels: general MFMA kernel
    (3, 31, 29, 64, 132, 3, 3, 2, False),   # stride 2, VALID, ragged tiles
    (2, 16, 16, 6, 10, 3, 3, 2, True),      # features not x4: direct kernel
    (2, 9, 10, 64, 64, 2, 2, 1, True),      # even window: padding 0 before, 1 after
    (2, 12, 9, 64, 128, 4, 4, 1, True),     # even window: padding 1 before, 2 after
    (2, 10, 10, 64, 64, 2, 4, 1, False),    # VALID, rectangular even window
])
def test_f16_conv_input_backprop(shape):
    """Half-precision input gradient (fp32 accumulation) against the oracle in
    double precision on the same half-rounded operands."""
    batch, rows, cols, ch, feats, wr, wc, stride, same = shape
    p = ops.add_padding_to(ops.ConvParams(
        channels=ch, features=feats, batch=batch, in_rows=rows, in_cols=cols,
        window_rows=wr, window_cols=wc, stride_rows=stride,
        stride_cols=stride), same)
    rng = np.random.default_rng(780 + rows * cols + feats)
    n_dy, n_fil, _ = ops.conv_sizes(p, DIRECTION.INPUT_BACKPROP)
    dy = uniform(rng, n_dy).astype(np.float16)
    w = uniform(rng, n_fil).astype(np.float16)
    ref = oracle.conv2d_input_backprop(dy.astype(np.float32),
                                       w.astype(np.float32),
                                       oracle_params(p, feats), acc64=True)
    for algo in (ALGO.IM2COL, ALGO.DIRECT):
        got = ops.conv2d(dev(dy, torch.float16), dev(w, torch.float16), p,
                         DIRECTION.INPUT_BACKPROP, algo).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16 inbk", ALGO_NAME[algo], shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, same
    (4, 56, 56, 64, 64, 3, 1, True),      # the four ResNet 3x3 layers
    (4, 28, 28, 128, 128, 3, 1, True),
    (4, 14, 14, 256, 256, 3, 1, True),
    (4, 7, 7, 512, 512, 3, 1, True),
    (4, 28, 28, 128, 512, 1, 1, False),   # 1x1 K = 4C
    (3, 17, 9, 128, 72, 3, 2, True),      # stride 2, ragged feature tile
    (2, 9, 9, 64, 200, 5, 1, False),      # VALID, 25 taps
    (128, 28, 28, 128, 128, 3, 1, True),  # configuration 4's batch
])
def test_f16_conv_filter_backprop_on_matrix_cores(shape):
    """Half-precision filter gradient (channel counts in multiples of 64: the
    implicit-GEMM kernel reading binary16, fp32 accumulation) against the
    oracle in double precision on the same half-rounded operands; with and
    without a caller workspace for the fp32 accumulation buffer."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(782 + rows + feats)
    n_x, n_dy, n_dw = ops.conv_sizes(p, DIRECTION.FILTER_BACKPROP)
    x = uniform(rng, n_x).astype(np.float16)
    dy = uniform(rng, n_dy).astype(np.float16)
    ref = oracle.conv2d_filter_backprop(x.astype(np.float32),
                                        dy.astype(np.float32),
                                        oracle_params(p, feats), acc64=True)
    dx_, ddy = dev(x, torch.float16), dev(dy, torch.float16)
    for ws in (None, torch.empty(2 * n_dw, dtype=torch.float16,
                                 device="cuda")):
        got = ops.conv2d(dx_, ddy, p, DIRECTION.FILTER_BACKPROP, ALGO.IM2COL,
                         workspace=ws).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16 filbk mfma", shape, ws is None))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features
    (3, 17, 9, 64, 128),     # odd image, two feature tiles
    (2, 10, 30, 128, 64),    # two channel tiles
    (1, 20, 120, 64, 64),    # wide rows: bands of one row
    (5, 7, 7, 64, 64),       # several images per LDS buffer, ragged last task
    (7, 14, 14, 192, 64),    # three channel tiles
    (300, 7, 7, 64, 64),     # more tasks than work-groups
    (9, 56, 56, 64, 64),     # runs of consecutive bands across images
])
def test_f16_filter_backprop_3x3_transposing_reads(shape):
    """The 3x3 stride-1 SAME half-precision filter gradient on the binary16
    matrix cores (LDS transposing reads, partial tiles + reduction) against
    the oracle in double precision on the same half-rounded operands."""
    batch, rows, cols, ch, feats = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 3, 1, True)
    rng = np.random.default_rng(795 + rows + feats + batch)
    n_x, n_dy, n_dw = ops.conv_sizes(p, DIRECTION.FILTER_BACKPROP)
    x = uniform(rng, n_x).astype(np.float16)
    dy = uniform(rng, n_dy).astype(np.float16)
    ref = oracle.conv2d_filter_backprop(x.astype(np.float32),
                                        dy.astype(np.float32),
                                        oracle_params(p, feats), acc64=True)
    dx_, ddy = dev(x, torch.float16), dev(dy, torch.float16)
    for ws in (None, torch.empty(2 * 256 * 9 * 64 * 64, dtype=torch.float16,
                                 device="cuda")):
        got = ops.conv2d(dx_, ddy, p, DIRECTION.FILTER_BACKPROP, ALGO.IM2COL,
                         workspace=ws).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16 filbk 3x3", shape, ws is None))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features
    (3, 7, 9, 64, 64),        # one 64 x 64 tile, 189 pixels (ragged stage)
    (2, 14, 14, 64, 128),
    (32, 28, 28, 64, 256),    # 64 x 256 tiles
    (5, 8, 8, 128, 256),      # 128 x 256 tiles
    (2, 28, 28, 192, 320),    # channel and feature counts in odd multiples of 64
    (32, 7, 7, 512, 2048),    # many tiles, few splits
    (64, 28, 28, 128, 512),   # 256 splits
])
def test_f16_filter_backprop_1x1_transposing_reads(shape):
    """The 1x1 half-precision filter gradient on the binary16 matrix cores
    against the oracle in double precision on the same half-rounded
    operands."""
    batch, rows, cols, ch, feats = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 1, 1, False)
    rng = np.random.default_rng(796 + rows + feats + batch)
    n_x, n_dy, n_dw = ops.conv_sizes(p, DIRECTION.FILTER_BACKPROP)
    x = uniform(rng, n_x).astype(np.float16)
    dy = uniform(rng, n_dy).astype(np.float16)
    ref = oracle.conv2d_filter_backprop(x.astype(np.float32),
                                        dy.astype(np.float32),
                                        oracle_params(p, feats), acc64=True)
    dx_, ddy = dev(x, torch.float16), dev(dy, torch.float16)
    for ws in (None, torch.empty(2 * 256 * 4096 * 8, dtype=torch.float16,
                                 device="cuda")):
        got = ops.conv2d(dx_, ddy, p, DIRECTION.FILTER_BACKPROP, ALGO.MATMUL,
                         workspace=ws).float().cpu().numpy()
        assert_close_f16(got, ref, ("f16 filbk 1x1", shape, ws is None))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, SAME
    (8, 32, 32, 16, 16, 3, 1, True),     # ragged tiles, vector loads
    (8, 32, 32, 24, 24, 3, 1, True),
    (8, 32, 32, 40, 72, 1, 1, False),
    (4, 28, 28, 144, 144, 3, 1, True),
    (4, 28, 28, 100, 100, 5, 1, True),
    (4, 56, 56, 12, 20, 3, 2, True),
    (8, 28, 28, 128, 256, 1, 2, False),  # whole tiles, stride 2
    (8, 32, 32, 3, 64, 3, 1, True),      # channels not a multiple of 4:
    (8, 32, 32, 64, 66, 3, 1, True),     # element by element
    (8, 32, 32, 66, 10, 1, 1, False),
    (8, 32, 32, 64, 3, 3, 1, True),
    (3, 13, 11, 96, 64, 3, 1, True),     # 429 pixels: shares that end inside
    (5, 9, 7, 48, 80, 1, 1, False),      # a step of 4 (fp32) or 16 (binary16)
])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_filter_gradient_from_registers_ragged_and_half(shape, dtype):
    """Shapes that used to have no matrix-core filter gradient -- channel or
    feature counts that are not multiples of 64 (binary16: any but the 3x3 and
    1x1 stride-1 layers with whole tiles) or of 4 -- run on the kernel that
    loads both operands straight into the matrix instruction's registers
    (binary16 with counts in multiples of 4: the binary16 instruction, four
    pixels per lane regrouped in registers; other binary16 counts converted on
    the way into the fp32 instruction), against the oracle in double precision on
    the same operands; with and without a workspace for the partial filters;
    twice gives the same bits."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(790 + rows + ch + feats)
    direction = DIRECTION.FILTER_BACKPROP
    n_x, n_dy, n_dw = ops.conv_sizes(p, direction)
    half = dtype == "f16"
    x, dy = uniform(rng, n_x), uniform(rng, n_dy)
    if half:
        x, dy = x.astype(np.float16), dy.astype(np.float16)
    ref = oracle.conv2d_filter_backprop(x.astype(np.float32),
                                        dy.astype(np.float32),
                                        oracle_params(p, feats), acc64=True)
    tdt = torch.float16 if half else torch.float32
    dx_, ddy = dev(x, tdt), dev(dy, tdt)
    _, rec = ops.workspace_size(p, direction, ALGO.IM2COL, dtype=(
        capi.DTYPE.F16 if half else capi.DTYPE.F32))
    first = None
    for ws in (None, torch.empty(rec + 8, dtype=tdt, device="cuda")):
        got = ops.conv2d(dx_, ddy, p, direction, ALGO.IM2COL, workspace=ws)
        if half:
            assert_close_f16(got.float().cpu().numpy(), ref,
                             ("f16 filter gradient", shape, ws is None))
        else:
            assert_close(got.cpu().numpy(), ref,
                         ("filter gradient", shape, ws is None))
        if first is None:
            first = got
        # (fp32 layers with few (tap, channel) pairs keep the one-work-group
        # kernel, whose partial sums meet through float atomics)
        # (binary16 layers with at most 8 channels go the same way, through
        # fp32 copies)
        if ((not half or ch <= 8) and ch < 32 and feats % 4 == 0 and
                window * window * ch <= 192):
            continue
        assert torch.equal(got.view(torch.int16 if half else torch.int32),
                           first.view(torch.int16 if half else torch.int32))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, SAME
    (8, 32, 32, 64, 66, 3, 1, True),
    (8, 64, 64, 64, 3, 3, 1, True),      # an RGB output layer
    (8, 32, 32, 128, 21, 1, 1, False),   # 21 classes
    (4, 33, 31, 48, 1, 3, 2, True),      # one feature, stride 2
])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_feature_counts_that_are_not_multiples_of_four_run_padded(shape, dtype):
    """Forward convolutions (fp32) and input gradients (fp32, binary16) whose
    feature count is not a multiple of 4 run on the matrix-core kernels over
    copies of the filter and of the tensor that carries the features, widened
    with zeros, instead of one lane per output: against the oracle in double
    precision, nothing written past the result."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(805 + rows + ch + feats)
    half = dtype == "f16"
    tdt = torch.float16 if half else torch.float32
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
        n_a, n_b, n_o = ops.conv_sizes(p, direction)
        a, b = uniform(rng, n_a), uniform(rng, n_b)
        if half:
            a, b = a.astype(np.float16), b.astype(np.float16)
        ref = ORACLE_FN[direction](a.astype(np.float32), b.astype(np.float32),
                                   oracle_params(p, feats), acc64=True)
        out = torch.full((n_o + 16,), 7.0, dtype=tdt, device="cuda")
        got = ops.conv2d(dev(a, tdt), dev(b, tdt), p, direction, ALGO.IM2COL,
                         out=out[:n_o])
        if half:
            assert_close_f16(got.float().cpu().numpy(), ref,
                             ("f16 padded features", direction, shape))
        else:
            assert_close(got.cpu().numpy(), ref,
                         ("padded features", direction, shape))
        assert torch.all(out[n_o:] == 7.0)
    if not half:
        # bias and ReLU are indexed by the feature: that launch is not padded
        n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
        x, w, bias = uniform(rng, n_in), uniform(rng, n_fil), uniform(rng, feats)
        ref = oracle.conv2d_forward(x, w, oracle_params(p, feats), acc64=True)
        want = np.maximum(ref.reshape(-1, feats) + bias.astype(np.float64), 0)
        got = ops.conv2d_bias_act(dev(x), dev(w), dev(bias), p, ALGO.IM2COL,
                                  relu=True)
        assert_close(got.cpu().numpy(), want.reshape(-1),
                     ("bias + relu, ragged features", shape))


@pytest.mark.parametrize("shape", [
    (3, 67, 67, 3, 96, 11, 4, False),   # 363 (tap, channel) pairs: two parts
    (4, 40, 40, 4, 32, 11, 2, True),    # 484: three parts
    (1, 30, 30, 8, 64, 9, 1, True),     # 648: four parts
])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_few_channel_layers_with_large_windows(shape, dtype):
    """Layers of at most eight channels whose (tap, channel) range is longer
    than the one-work-group filter gradient kernel holds (an 11x11x3 stem) run
    that kernel in parts of 192 rows of dW; their binary16 input gradient and
    filter gradient run through the fp32 kernels.  All three directions
    against the oracle in double precision."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, window, stride, same)
    rng = np.random.default_rng(911 + rows + ch + feats)
    half = dtype == "f16"
    tdt = torch.float16 if half else torch.float32
    for direction in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP,
                      DIRECTION.FILTER_BACKPROP):
        n_a, n_b, n_o = ops.conv_sizes(p, direction)
        a, b = uniform(rng, n_a), uniform(rng, n_b)
        if half:
            a, b = a.astype(np.float16), b.astype(np.float16)
        ref = ORACLE_FN[direction](a.astype(np.float32), b.astype(np.float32),
                                   oracle_params(p, feats), acc64=True)
        out = torch.full((n_o + 16,), 7.0, dtype=tdt, device="cuda")
        got = ops.conv2d(dev(a, tdt), dev(b, tdt), p, direction, ALGO.IM2COL,
                         out=out[:n_o])
        if half:
            assert_close_f16(got.float().cpu().numpy(), ref,
                             ("f16 few channels", direction, shape))
        else:
            assert_close(got.cpu().numpy(), ref,
                         ("few channels", direction, shape))
        assert torch.all(out[n_o:] == 7.0)


def test_f16_conv_filter_backprop():
    p = ops.conv_params(3, 10, 9, 16, 24, 3, 1, True)
    rng = np.random.default_rng(781)
    n_x, n_dy, _ = ops.conv_sizes(p, DIRECTION.FILTER_BACKPROP)
    x = uniform(rng, n_x).astype(np.float16)
    dy = uniform(rng, n_dy).astype(np.float16)
    ref = oracle.conv2d_filter_backprop(x.astype(np.float32),
                                        dy.astype(np.float32),
                                        oracle_params(p, 24), acc64=True)
    got = ops.conv2d(dev(x, torch.float16), dev(dy, torch.float16), p,
                     DIRECTION.FILTER_BACKPROP,
                     ALGO.IM2COL).float().cpu().numpy()
    assert_close_f16(got, ref, "f16 filbk")


@pytest.mark.parametrize("shape", [(2, 28, 28, 64, 1), (2, 28, 28, 64, 2),
                                   (3, 13, 11, 8, 2), (1, 9, 9, 6, 1)])
def test_f16_depthwise_backprops(shape):
    n, h, w_, c, stride = shape
    p = ops.depthwise_params(n, h, w_, c, 1, 3, stride, True)
    op = oracle_params(p, 1)
    rng = np.random.default_rng(790 + h + c)
    x = rng.standard_normal(n * h * w_ * c).astype(np.float16)
    w = rng.standard_normal(9 * c).astype(np.float16)
    dy = rng.standard_normal(n * p.out_rows * p.out_cols * c).astype(
        np.float16)
    got = ops.depthwise_conv2d(dev(dy, torch.float16), dev(w, torch.float16),
                               p, DIRECTION.INPUT_BACKPROP)
    assert_close_f16(got.float().cpu().numpy(),
                     oracle.depthwise_input_backprop(
                         dy.astype(np.float32), w.astype(np.float32), op),
                     ("f16 dw inbk", shape))
    got = ops.depthwise_conv2d(dev(x, torch.float16), dev(dy, torch.float16),
                               p, DIRECTION.FILTER_BACKPROP)
    assert_close_f16(got.float().cpu().numpy(),
                     oracle.depthwise_filter_backprop(
                         x.astype(np.float32), dy.astype(np.float32), op),
                     ("f16 dw filbk", shape))


@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, multiplier, window, stride
    (8, 28, 28, 66, 1, 3, 1),    # channels not a multiple of 4
    (8, 28, 28, 30, 1, 3, 2),
    (4, 28, 28, 64, 2, 3, 1),    # channel multiplier 2
    (4, 28, 28, 96, 1, 5, 1),    # 5x5
    (4, 14, 14, 480, 1, 7, 1),   # 7x7
    (4, 56, 56, 3, 8, 3, 2),     # three channels, multiplier 8
    (8, 28, 28, 128, 1, 1, 1),   # 1x1 window
    (4, 56, 56, 64, 1, 3, 1),    # (binary16: the MobileNet shape itself)
    (16, 56, 56, 64, 1, 3, 1),   # (binary16, large: through the fp32 kernel)
    (16, 112, 112, 32, 1, 3, 2),
])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_depthwise_filter_gradient_general_shapes_split_over_work_groups(
        shape, dtype):
    """Depthwise filter gradients outside the fp32 3x3 kernels (other windows,
    channel multipliers, channel counts that are not multiples of 4, every
    binary16 shape) split the output pixels over work-groups whose sums meet
    through float atomics in an fp32 buffer: against the oracle in double
    precision on the same operands."""
    n, h, w_, c, mult, window, stride = shape
    p = ops.depthwise_params(n, h, w_, c, mult, window, stride, True)
    op = oracle_params(p, mult)
    rng = np.random.default_rng(795 + h + c + window)
    half = dtype == "f16"
    x = uniform(rng, n * h * w_ * c)
    dy = uniform(rng, n * p.out_rows * p.out_cols * c * mult)
    if half:
        x, dy = x.astype(np.float16), dy.astype(np.float16)
    ref = oracle.depthwise_filter_backprop(x.astype(np.float32),
                                           dy.astype(np.float32), op)
    tdt = torch.float16 if half else torch.float32
    out = torch.full((window * window * c * mult + 16,), 7.0, dtype=tdt,
                     device="cuda")
    got = ops.depthwise_conv2d(dev(x, tdt), dev(dy, tdt), p,
                               DIRECTION.FILTER_BACKPROP,
                               out=out[:window * window * c * mult])
    if half:
        assert_close_f16(got.float().cpu().numpy(), ref, ("f16 dw filbk", shape))
    else:
        assert_close(got.cpu().numpy(), ref, ("dw filbk", shape))
    assert torch.all(out[window * window * c * mult:] == 7.0)


@pytest.mark.parametrize("size,ch,stride", MOBILENET)
def test_f16_depthwise_forward(size, ch, stride):
    p = ops.depthwise_params(2, size, size, ch, 1, 3, stride, True)
    rng = np.random.default_rng(800 + size)
    x = uniform(rng, 2 * size * size * ch).astype(np.float16)
    w = uniform(rng, 9 * ch).astype(np.float16)
    ref = oracle.depthwise_forward(x.astype(np.float32), w.astype(np.float32),
                                   oracle_params(p, 1))
    got = ops.depthwise_conv2d(dev(x, torch.float16), dev(w, torch.float16),
                               p).float().cpu().numpy()
    assert_close_f16(got, ref, ("f16 dw", size, ch))


def test_f16_pooling_forward():
    p = ops.pool_params(2, 112, 112, 64, 3, 2, True)
    rng = np.random.default_rng(900)
    x = rng.standard_normal(2 * 112 * 112 * 64).astype(np.float16)
    ref = oracle.pool_max_forward(x.astype(np.float32), oracle_params(p, 0))
    got = ops.pooling_forward(dev(x, torch.float16), p, POOL_OP.MAX)
    assert np.array_equal(got.float().cpu().numpy(), ref)
    q = ops.pool_params(2, 7, 7, 2048, 7, 1, False)
    x = rng.standard_normal(2 * 49 * 2048).astype(np.float16)
    ref = oracle.pool_avg_forward(x.astype(np.float32), oracle_params(q, 0))
    got = ops.pooling_forward(dev(x, torch.float16), q, POOL_OP.AVERAGE)
    assert_close_f16(got.float().cpu().numpy(), ref, "f16 avg")


def _winograd_sweep_shapes():
    """Seeded shapes for the persistent Winograd kernel: even numbers of
    16-channel chunks, odd image sizes, both paddings, tile counts that leave
    ragged last tile blocks, enough units for a work-group to walk several."""
    rng = np.random.default_rng(20261125)
    shapes = []
    while len(shapes) < 14:
        ch = int(rng.choice([32, 64, 96, 128]))
        feats = int(rng.choice([32, 64, 96, 160]))
        rows, cols = int(rng.integers(5, 40)), int(rng.integers(5, 40))
        same = bool(rng.integers(0, 2))
        if not same and min(rows, cols) < 4:
            continue
        # keep the oracle to about a second per case
        batch = int(max(1, min(48, 1.2e9 // (rows * cols * 18 * ch * feats))))
        shapes.append((batch, rows, cols, ch, feats, same))
    return shapes


@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP])
@pytest.mark.parametrize("shape", _winograd_sweep_shapes())
def test_winograd_persistent_kernel_sweep(shape, direction):
    batch, rows, cols, ch, feats, same = shape
    p = ops.conv_params(batch, rows, cols, ch, feats, 3, 1, same)
    conv_case(p, direction, [ALGO.WINOGRAD],
              seed=4000 + 7 * rows + 3 * cols + ch + feats)


def test_winograd_stream_bias_relu_matches_separate_launches():
    """Bias and ReLU applied by the persistent Winograd kernel's stores give
    the bits of convolution, bias add and ReLU run as three launches."""
    p = ops.conv_params(40, 33, 31, 32, 64, 3, 1, True)
    rng = np.random.default_rng(1717)
    n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = dev(uniform(rng, n_in)), dev(uniform(rng, n_fil))
    bias = dev(uniform(rng, 64))
    plain = ops.conv2d(x, w, p, DIRECTION.FORWARD, ALGO.WINOGRAD)
    want = torch.relu(plain.view(-1, 64) + bias).view(-1)
    got = ops.conv2d_bias_act(x, w, bias, p, ALGO.WINOGRAD, relu=True)
    assert torch.equal(got, want)
    got = ops.conv2d_bias_act(x, w, bias, p, ALGO.WINOGRAD, relu=False)
    assert torch.equal(got, (plain.view(-1, 64) + bias).view(-1))


def test_kernel_timing_brackets_the_main_kernel():
    p = ops.conv_params(8, 28, 28, 128, 128, 3, 1, True)
    rng = np.random.default_rng(1500)
    n_in, n_fil, _ = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = dev(uniform(rng, n_in)), dev(uniform(rng, n_fil))
    for algo in (ALGO.WINOGRAD, ALGO.IM2COL):
        ops.conv2d(x, w, p, DIRECTION.FORWARD, algo)
        with ops.kernel_timing() as kt:
            for _ in range(3):
                ops.conv2d(x, w, p, DIRECTION.FORWARD, algo)
        assert kt.kernels == 3
        assert 0.001 < kt.total_ms / 3 < 5.0
    # disabled again: nothing is recorded
    ops.conv2d(x, w, p, DIRECTION.FORWARD, ALGO.IM2COL)
    with ops.kernel_timing() as kt:
        pass
    assert kt.kernels == 0


# ---- pointwise / binaryop ---------------------------------------------------

POINTWISE = ["relu", "tanh", "exp", "log", "floor", "sqrt"]


def pointwise_data(rng, op, n):
    x = rng.standard_normal(n).astype(np.float32) * 2
    if op in ("log", "sqrt"):
        x = np.abs(x) + 0.1
    return x


def assert_ulp(got, ref, ulps, what):
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    tol = ulps * np.spacing(np.maximum(np.abs(ref), np.abs(got)))
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert np.all(err <= tol), (what, float(err.max()))


@pytest.mark.parametrize("op", POINTWISE)
@pytest.mark.parametrize("n", [1, 7, 1024, 4099, 1 << 20])
def test_pointwise_forward_and_grad(op, n):
    """Against the oracle; device libm may differ from the host's by a few
    ULP on tanh / exp / log (the reference's own tests allow 10)."""
    rng = np.random.default_rng(900 + n)
    x = pointwise_data(rng, op, n)
    code = getattr(POINTWISE_OP, op.upper())
    ref = oracle.pointwise_forward(op, x)
    got = ops.pointwise_forward(dev(x), code).cpu().numpy()
    assert_ulp(got, ref, 10, (op, n, "forward"))
    if op == "floor":
        return
    err = rng.standard_normal(n).astype(np.float32)
    val = x if op == "log" else ref
    got = ops.pointwise_grad(dev(val), dev(err), code).cpu().numpy()
    # (1 - val * val) cancels near |val| = 1, where a fused multiply-add on
    # the device and the oracle's separate rounding differ by more than ULPs
    # of the result: absolute bar, tighter than the 1e-5 the reference's
    # gradient tests use (test/pointwise/pointwise_fixture.h:66-70).
    assert np.allclose(got, oracle.pointwise_grad(op, val, err), rtol=1e-5,
                       atol=1e-6), (op, n, "grad")


def test_pointwise_in_place_unaligned_and_f16():
    rng = np.random.default_rng(950)
    x = rng.standard_normal(5000).astype(np.float32)
    # in place
    d = dev(x)
    ops.pointwise_forward(d, POINTWISE_OP.RELU, out=d)
    assert np.array_equal(d.cpu().numpy(), np.maximum(x, 0))
    # operands 4 bytes off a 16-byte boundary: the one-element-per-lane kernel
    d = dev(np.concatenate([[0.0], x]).astype(np.float32))
    out = torch.zeros(5001, device="cuda")
    ops.pointwise_forward(d[1:], POINTWISE_OP.RELU, out=out[1:])
    assert np.array_equal(out.cpu().numpy()[1:], np.maximum(x, 0))
    assert out[0].item() == 0.0
    # binary16: fp32 arithmetic, one rounding
    h = x.astype(np.float16)
    got = ops.pointwise_forward(dev(h, torch.float16), POINTWISE_OP.TANH)
    ref = np.tanh(h.astype(np.float32)).astype(np.float16)
    assert_close_f16(got.float().cpu().numpy(), ref.astype(np.float32),
                     "tanh f16")
    g = ops.pointwise_grad(dev(h, torch.float16), dev(h, torch.float16),
                           POINTWISE_OP.RELU)
    assert np.array_equal(g.cpu().numpy(), np.where(h > 0, h, 0).astype(np.float16))


BINARY = {"add": np.add, "sub": np.subtract, "mul": np.multiply,
          "div": np.divide}


@pytest.mark.parametrize("op", list(BINARY))
@pytest.mark.parametrize("dims", [
    ([32, 56, 56, 64], [64]),           # bias add over NHWC: periodic operand
    ([64], [32, 56, 56, 64]),           # ... on the left
    ([3, 5, 7, 9], [3, 5, 7, 9]),       # same shape, odd size (tail)
    ([1000003], []),                    # scalar right operand
    ([], [257]),                        # scalar left operand
    ([4, 1, 6, 1], [1, 5, 1, 7]),       # general broadcasting both ways
    ([2, 3, 4, 6], [4, 6]),             # period 24, not a multiple of 4 x 8? (f32: 24 % 4 == 0)
    ([2, 3, 4, 5], [5]),                # period 5: general kernel
    ([6, 1, 5], [2, 1, 7, 1]),          # different ranks
])
def test_binaryop_shapes(op, dims):
    lhs_dims, rhs_dims = dims
    rng = np.random.default_rng(960 + len(lhs_dims) * 7 + len(rhs_dims))
    lhs = uniform(rng, int(np.prod(lhs_dims)))
    rhs = uniform(rng, int(np.prod(rhs_dims))) + 2.0  # keep div well away from 0
    ref = BINARY[op](lhs.reshape(lhs_dims), rhs.reshape(rhs_dims)).reshape(-1)
    assert np.array_equal(oracle.binaryop(op, lhs, rhs, lhs_dims, rhs_dims),
                          ref)
    got = ops.binaryop(dev(lhs), dev(rhs), lhs_dims, rhs_dims,
                       getattr(BINARY_OP, op.upper())).cpu().numpy()
    # add, sub, mul are exactly rounded on both sides; div within 1 ULP
    if op == "div":
        assert_ulp(got, ref, 1, (op, dims))
    else:
        assert np.array_equal(got, ref), (op, dims)


def test_binaryop_f16_in_place_and_errors():
    rng = np.random.default_rng(970)
    x = uniform(rng, 32 * 14 * 14 * 256).astype(np.float16)
    b = uniform(rng, 256).astype(np.float16)
    d = dev(x, torch.float16)
    ops.binaryop(d, dev(b, torch.float16), [32, 14, 14, 256], [256],
                 BINARY_OP.ADD, out=d)
    ref = (x.astype(np.float32).reshape(-1, 256) +
           b.astype(np.float32)).astype(np.float16).reshape(-1)
    assert np.array_equal(d.cpu().numpy(), ref)
    a = dev(uniform(rng, 6))
    out = torch.empty(12, device="cuda")
    # include/portdnn/internal/binaryop/launch.h:52-56: not broadcastable
    assert ops.binaryop_raw(a, a, out, [2, 3], [3, 2], BINARY_OP.ADD) == \
        STATUS.INVALID_PARAMETER
    assert ops.binaryop_raw(a, a, out, [1, 1, 1, 2, 3], [3], BINARY_OP.ADD) == \
        STATUS.INVALID_PARAMETER
    assert ops.binaryop_raw(a, a, out, [2, 3], [3], 9) == \
        STATUS.INVALID_PARAMETER


# ---- convolution with bias and activation ------------------------------------

@pytest.mark.parametrize("shape", [
    # batch, size, channels, features, window, stride
    (4, 28, 64, 64, 3, 1),      # fused Winograd epilogue
    (2, 14, 256, 256, 3, 1),    # Winograd with a channel split: separate pass
    (4, 28, 64, 256, 1, 1),     # implicit GEMM, epilogue in the kernel
    (1, 7, 512, 2048, 1, 1),    # implicit GEMM with a reduction split
    (2, 15, 24, 40, 3, 2),      # strided, ragged
    (1, 9, 3, 6, 5, 1),         # direct kernel, features % 4 != 0
])
@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("with_bias", [True, False])
def test_conv2d_bias_activation(shape, relu, with_bias):
    """snn_hip_conv2d_forward_bias_act_f32 against the composition it stands
    for: oracle convolution, oracle binaryop add of the [features] bias,
    oracle relu."""
    batch, size, ch, feats, window, stride = shape
    p = ops.conv_params(batch, size, size, ch, feats, window, stride, True)
    rng = np.random.default_rng(1000 + size + feats)
    n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
    x, w = uniform(rng, n_in), uniform(rng, n_fil)
    bias = uniform(rng, feats) * 4 if with_bias else None
    ref = oracle.conv2d_forward(x, w, oracle_params(p, feats), acc64=True)
    if with_bias:
        ref = oracle.binaryop("add", ref, bias,
                              [batch, p.out_rows, p.out_cols, feats], [feats])
    if relu:
        ref = oracle.pointwise_forward("relu", ref)
    d_bias = dev(bias) if with_bias else None
    n_run = 0
    for algo in FWD_ALGOS:
        if not supported(p, DIRECTION.FORWARD, algo):
            continue
        got = ops.conv2d_bias_act(dev(x), dev(w), d_bias, p, algo,
                                  relu=relu).cpu().numpy()
        # an output within rounding of zero may land on either side of the
        # ReLU: the absolute part of the tolerance covers it
        assert_close(got, ref, ("bias_act", ALGO_NAME[algo], shape, relu,
                                with_bias))
        n_run += 1
    assert n_run >= 2


def test_conv2d_bias_activation_rejects_unknown_activation():
    p = ops.conv_params(1, 8, 8, 4, 4, 3, 1, True)
    x = torch.zeros(ops.conv_sizes(p, 0)[0], device="cuda")
    w = torch.zeros(ops.conv_sizes(p, 0)[1], device="cuda")
    y = torch.zeros(ops.conv_sizes(p, 0)[2], device="cuda")
    rc = capi.lib().snn_hip_conv2d_forward_bias_act_f32(
        x.data_ptr(), w.data_ptr(), None, y.data_ptr(), ctypes.byref(p),
        ALGO.DIRECT, 7, None, 0, None)
    assert rc == STATUS.INVALID_PARAMETER


# ---- NCHW / FCHW operands ------------------------------------------------------

@pytest.mark.parametrize("shape", [
    # batch, rows, cols, channels, features, window, stride, same
    (2, 9, 11, 5, 7, 3, 1, True),
    (3, 12, 8, 16, 24, 3, 2, True),
    (1, 37, 41, 3, 8, 7, 2, True),      # tiles of the transposes are ragged
    (2, 6, 6, 40, 33, 1, 1, False),
])
@pytest.mark.parametrize("direction", [DIRECTION.FORWARD,
                                       DIRECTION.INPUT_BACKPROP,
                                       DIRECTION.FILTER_BACKPROP])
def test_conv2d_nchw_fchw(shape, direction):
    """DataFormat::NCHW with FilterFormat::FCHW through the Direct algorithm
    (include/portdnn/internal/conv2d/launch.h:86-88, :191-194) against the
    NHWC / HWCF oracle on permuted operands."""
    batch, rows, cols, ch, feats, window, stride, same = shape
    p = ops.add_padding_to(ops.ConvParams(
        channels=ch, features=feats, batch=batch, in_rows=rows, in_cols=cols,
        window_rows=window, window_cols=window, stride_rows=stride,
        stride_cols=stride), same)
    rng = np.random.default_rng(1100 + rows)
    x = uniform(rng, batch * rows * cols * ch).reshape(batch, rows, cols, ch)
    w = uniform(rng, window * window * ch * feats).reshape(window, window, ch,
                                                           feats)
    dy = uniform(rng, batch * p.out_rows * p.out_cols * feats).reshape(
        batch, p.out_rows, p.out_cols, feats)
    op = oracle_params(p, feats)
    nchw = lambda t: np.ascontiguousarray(t.transpose(0, 3, 1, 2)).reshape(-1)
    fchw = lambda t: np.ascontiguousarray(t.transpose(3, 2, 0, 1)).reshape(-1)
    if direction == DIRECTION.FORWARD:
        a, b = nchw(x), fchw(w)
        ref = nchw(oracle.conv2d_forward(x, w, op).reshape(dy.shape))
    elif direction == DIRECTION.INPUT_BACKPROP:
        a, b = nchw(dy), fchw(w)
        ref = nchw(oracle.conv2d_input_backprop(dy, w, op).reshape(x.shape))
    else:
        a, b = nchw(x), nchw(dy)
        ref = fchw(oracle.conv2d_filter_backprop(x, dy, op).reshape(w.shape))
    q = ops.ConvParams(**{f: getattr(p, f) for f, _ in p._fields_})
    q.input_format, q.filter_format = 1, 1
    got = ops.conv2d(dev(a), dev(b), q, direction, ALGO.DIRECT).cpu().numpy()
    assert_close(got, ref, ("nchw", shape, direction))
    # any other algorithm is refused for NCHW
    out = torch.empty(ref.size, device="cuda")
    assert ops.conv2d_raw(dev(a), dev(b), out, q, direction, ALGO.IM2COL) == \
        STATUS.INVALID_ALGORITHM
    # NCHW with an HWCF filter is an invalid combination
    q.filter_format = 0
    assert ops.conv2d_raw(dev(a), dev(b), out, q, direction, ALGO.DIRECT) == \
        STATUS.INVALID_PARAMETER


def test_scale_blend():
    """snn_hip_scale_blend_f32: y = alpha * y + beta * prior, the scaling step
    of the cuDNN-style layer (include/portdnn/compat/scaling.hpp:150-262)."""
    rng = np.random.default_rng(1200)
    y, prior = uniform(rng, 4099), uniform(rng, 4099)
    L = capi.lib()
    for alpha, beta in ((2.0, 0.0), (1.0, 1.0), (-0.5, 3.0), (0.0, 2.0)):
        d = dev(y)
        rc = L.snn_hip_scale_blend_f32(d.data_ptr(), dev(prior).data_ptr(),
                                       alpha, beta, y.size, None)
        assert rc == STATUS.OK
        torch.cuda.synchronize()
        ref = (np.float32(alpha) * y if alpha else 0 * y) + \
            np.float32(beta) * prior
        assert np.allclose(d.cpu().numpy(), ref, rtol=1e-6, atol=1e-7)
    # a zero alpha drops the data term even when it holds NaN
    d = dev(np.full(16, np.nan, dtype=np.float32))
    assert L.snn_hip_scale_blend_f32(d.data_ptr(), None, 0.0, 0.0, 16,
                                     None) == STATUS.OK
    assert np.array_equal(d.cpu().numpy(), np.zeros(16, dtype=np.float32))
    assert L.snn_hip_scale_blend_f32(d.data_ptr(), None, 1.0, 1.0, 16,
                                     None) == STATUS.INVALID_PARAMETER


@pytest.mark.gpu
def test_forward_chain_in_a_hip_graph_replays_like_eager():
    """Callers that capture their launch-bound loops (serving) record library
    calls into a HIP graph: a chain 3x3 conv (Winograd with the caller's
    workspace) -> ReLU -> 1x1 conv -> 3x3 conv (Tiled) -> depthwise 3x3 ->
    max pool 3x3 s2 is captured once and replayed three times, with eager
    work of the program's own and synchronisations in between; every replay
    must give the eager result bit for bit (these paths allocate nothing, clear
    nothing with memset nodes and add nothing atomically)."""
    batch, size, ch = 16, 56, 64
    rng = np.random.default_rng(4100)
    p3 = ops.conv_params(batch, size, size, ch, ch, 3, 1, True)
    p1 = ops.conv_params(batch, size, size, ch, 4 * ch, 1, 1, False)
    p3b = ops.conv_params(batch, size, size, 4 * ch, ch, 3, 1, True)
    pd = ops.depthwise_params(batch, size, size, ch, 1, 3, 1, True)
    pp = ops.pool_params(batch, size, size, ch, 3, 2, True)
    x = dev(uniform(rng, ops.conv_sizes(p3, DIRECTION.FORWARD)[0]))
    w3 = dev(uniform(rng, ops.conv_sizes(p3, DIRECTION.FORWARD)[1]))
    w1 = dev(uniform(rng, ops.conv_sizes(p1, DIRECTION.FORWARD)[1]))
    w3b = dev(uniform(rng, ops.conv_sizes(p3b, DIRECTION.FORWARD)[1]))
    wd = dev(uniform(rng, ops.depthwise_sizes(pd, DIRECTION.FORWARD)[1]))
    _, ws_elems = ops.workspace_size(p3, DIRECTION.FORWARD, ALGO.WINOGRAD)
    ws = torch.empty(ws_elems, device="cuda")
    n3 = ops.conv_sizes(p3, DIRECTION.FORWARD)[2]
    n1 = ops.conv_sizes(p1, DIRECTION.FORWARD)[2]
    bufs = [torch.empty(n3, device="cuda"), torch.empty(n3, device="cuda"),
            torch.empty(n1, device="cuda"), torch.empty(n3, device="cuda"),
            torch.empty(n3, device="cuda"),
            torch.empty(batch * 28 * 28 * ch, device="cuda")]

    def chain():
        ops.conv2d(x, w3, p3, DIRECTION.FORWARD, ALGO.WINOGRAD, workspace=ws,
                   out=bufs[0])
        ops.pointwise_forward(bufs[0], POINTWISE_OP.RELU, out=bufs[1])
        ops.conv2d(bufs[1], w1, p1, DIRECTION.FORWARD, ALGO.MATMUL,
                   out=bufs[2])
        ops.conv2d(bufs[2], w3b, p3b, DIRECTION.FORWARD, ALGO.TILED,
                   out=bufs[3])
        ops.depthwise_conv2d(bufs[3], wd, pd, DIRECTION.FORWARD, out=bufs[4])
        ops.pooling_forward(bufs[4], pp, POOL_OP.MAX, out=bufs[5])

    chain()
    torch.cuda.synchronize()
    eager = [b.clone() for b in bufs]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()  # first calls (function attributes, plan caches) outside capture
        with torch.cuda.graph(graph, stream=side):
            chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    scratch = torch.empty(1 << 20, device="cuda")
    for replay in range(3):
        for b in bufs:
            b.fill_(float("nan"))
        ws.fill_(float("nan"))
        scratch.normal_()  # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, (b, e) in enumerate(zip(bufs, eager)):
            assert torch.equal(b.view(torch.int32), e.view(torch.int32)), (
                "replay", replay, "buffer", i)
