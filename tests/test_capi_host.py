"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every symbol include/snn_hip.h declares, and its host logic (validation,
selector rules, workspace sizes, status codes) follows the reference."""
import ctypes
import os
import re

import numpy as np
import pytest

from golden_cases import GOLDEN_DIR
from portdnn_amd import capi, ops
from portdnn_amd.capi import ALGO, DIRECTION, STATUS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: every call returns early


def declared_symbols():
    with open(os.path.join(ROOT, "include", "snn_hip.h")) as f:
        text = f.read()
    return sorted(set(re.findall(r"\b(snn_hip_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = declared_symbols()
    assert len(names) >= 19
    L = capi.lib()
    for name in names:
        assert hasattr(L, name), name
    assert sorted(capi.SIGNATURES) == names


def test_version_and_status_strings():
    L = capi.lib()
    assert L.snn_hip_version() >= 100
    # portDNN StatusCode order, include/portdnn/status.h:31-44
    expected = ["OK", "InvalidAlgorithm", "IndexExceeded",
                "InsufficientWorkspace", "AllocationProblem",
                "InvalidParameter", "DeviceError"]
    assert [capi.status_string(i) for i in range(7)] == expected


def test_python_padding_helper_matches_reference_known_answers():
    rows = np.load(os.path.join(GOLDEN_DIR, "padding_kat.npz"))["rows"]
    for same, window, stride, inp, pad, out in rows.tolist():
        assert ops.calculate_padding(inp, window, stride, same) == (pad, out)


def _conv(**kw):
    p = ops.conv_params(2, 8, 8, 4, 4, 3, 1, True)
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def _call_conv(p, algo=ALGO.DIRECT, direction=DIRECTION.FORWARD, ws=None,
               ws_elems=0):
    name = {0: "snn_hip_conv2d_forward_f32",
            1: "snn_hip_conv2d_input_backprop_f32",
            2: "snn_hip_conv2d_filter_backprop_f32"}[direction]
    return getattr(capi.lib(), name)(FAKE, FAKE, FAKE, ctypes.byref(p), algo,
                                     ws, ws_elems, None)


@pytest.mark.parametrize("field,value", [
    ("batch", 0), ("channels", 0), ("features", -1), ("in_rows", 0),
    ("in_cols", 0), ("out_rows", 0), ("out_cols", -3), ("window_rows", 0),
    ("window_cols", 0), ("stride_rows", 0), ("stride_cols", 0),
    ("pad_rows", -1), ("pad_cols", -1), ("dilation_rows", 2),
    ("dilation_cols", 0), ("groups", 3), ("groups", 0),
])
def test_conv2d_invalid_parameter(field, value):
    """include/portdnn/internal/conv2d/launch.h:42-97"""
    assert _call_conv(_conv(**{field: value})) == STATUS.INVALID_PARAMETER


def test_conv2d_null_arguments():
    L = capi.lib()
    p = _conv()
    assert L.snn_hip_conv2d_forward_f32(None, FAKE, FAKE, ctypes.byref(p),
                                        ALGO.DIRECT, None, 0,
                                        None) == STATUS.INVALID_PARAMETER
    assert L.snn_hip_conv2d_forward_f32(FAKE, FAKE, FAKE, None, ALGO.DIRECT,
                                        None, 0,
                                        None) == STATUS.INVALID_PARAMETER


def test_conv2d_invalid_algorithm():
    """An algorithm whose selector answers NotSupported gives InvalidAlgorithm
    (internal/conv2d/launch.h:127-129,164-165)."""
    s2 = ops.conv_params(1, 9, 9, 4, 4, 3, 2, True)
    assert _call_conv(s2, ALGO.WINOGRAD) == STATUS.INVALID_ALGORITHM
    assert _call_conv(s2, ALGO.MATMUL) == STATUS.INVALID_ALGORITHM
    assert _call_conv(s2, ALGO.NOT_SUPPORTED) == STATUS.INVALID_ALGORITHM
    assert _call_conv(s2, 99) == STATUS.INVALID_ALGORITHM
    w7 = ops.conv_params(1, 16, 16, 3, 8, 7, 2, True)
    assert _call_conv(w7, ALGO.TILED) == STATUS.INVALID_ALGORITHM
    # Tiled is forward only (tiled_selector.h:76-96)
    p = _conv()
    assert _call_conv(p, ALGO.TILED,
                      DIRECTION.INPUT_BACKPROP) == STATUS.INVALID_ALGORITHM
    assert _call_conv(p, ALGO.TILED,
                      DIRECTION.FILTER_BACKPROP) == STATUS.INVALID_ALGORITHM
    # grouped convolution is not part of this library
    g = _conv(groups=2)
    assert _call_conv(g, ALGO.IM2COL) == STATUS.INVALID_ALGORITHM


def test_winograd_needs_workspace():
    """internal/conv2d/winograd/launch.h:271-286"""
    for algo in (ALGO.WINOGRAD, ALGO.WINOGRAD_LARGE):
        for d in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
            assert _call_conv(_conv(), algo,
                              d) == STATUS.INSUFFICIENT_WORKSPACE


def test_index_exceeded():
    """Tensors beyond INT32_MAX elements (launch_tiled.cc:133-141)."""
    p = ops.conv_params(4096, 1024, 1024, 4, 4, 1, 1, False)
    assert _call_conv(p) == STATUS.INDEX_EXCEEDED


def test_algorithm_support_table():
    """The concrete selectors: tiled_selector.h:45-96,
    winograd_selector.h:44-106, matmul_selector.h:44-100."""
    L = capi.lib()

    def sup(p, d, a):
        return L.snn_hip_conv2d_algorithm_supports(ctypes.byref(p), d, a) == a

    F, I, B = (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP,
               DIRECTION.FILTER_BACKPROP)
    for w, s, ok in [(1, 1, True), (1, 2, True), (3, 1, True), (3, 2, True),
                     (5, 1, True), (5, 2, False), (7, 1, False),
                     (11, 4, False)]:
        p = ops.conv_params(1, 32, 32, 4, 4, w, s, True)
        assert sup(p, F, ALGO.TILED) == ok, (w, s)
        assert not sup(p, I, ALGO.TILED)
        assert not sup(p, B, ALGO.TILED)
        assert sup(p, F, ALGO.DIRECT) and sup(p, B, ALGO.IM2COL)
    p33 = ops.conv_params(1, 32, 32, 4, 4, 3, 1, True)
    for d in (F, I, B):
        assert sup(p33, d, ALGO.WINOGRAD)
        assert sup(p33, d, ALGO.WINOGRAD_LARGE)
    p31 = ops.conv_params(1, 32, 32, 4, 4, 3, 1, True)
    p31.window_cols = 1
    assert sup(p31, F, ALGO.WINOGRAD)
    assert not sup(p31, F, ALGO.WINOGRAD_LARGE)
    p32 = ops.conv_params(1, 32, 32, 4, 4, 3, 2, True)
    assert not sup(p32, F, ALGO.WINOGRAD)
    p11 = ops.conv_params(1, 32, 32, 4, 16, 1, 1, False)
    for d in (F, I, B):
        assert sup(p11, d, ALGO.MATMUL)
    assert not sup(p33, F, ALGO.MATMUL)
    p11s2 = ops.conv_params(1, 32, 32, 4, 16, 1, 2, False)
    assert not sup(p11s2, F, ALGO.MATMUL)


def test_default_algorithm_is_launchable():
    """test/conv2d/default_selector.cc:73-98: whatever the default selector
    returns must be supported for those parameters."""
    L = capi.lib()
    for w, s in [(1, 1), (1, 2), (3, 1), (3, 2), (5, 1), (7, 2), (11, 4)]:
        for same in (True, False):
            p = ops.conv_params(2, 32, 32, 8, 16, w, s, same)
            for d in range(3):
                a = L.snn_hip_conv2d_default_algorithm(ctypes.byref(p), d)
                assert a != ALGO.NOT_SUPPORTED
                assert L.snn_hip_conv2d_algorithm_supports(
                    ctypes.byref(p), d, a) == a


def test_default_algorithm_policy_on_benchmark_layers():
    """1x1 stride-1 layers are one GEMM; 3x3 stride-1 layers whose channel
    counts fit the fused Winograd kernels take them in all three directions;
    everything else is the implicit GEMM (Tiled / Im2col tags)."""
    L = capi.lib()

    def default(p, d):
        return L.snn_hip_conv2d_default_algorithm(ctypes.byref(p), d)

    for size, ch in [(56, 64), (28, 128), (14, 256), (7, 512)]:
        p3 = ops.conv_params(32, size, size, ch, ch, 3, 1, True)
        assert default(p3, DIRECTION.FORWARD) == ALGO.WINOGRAD
        assert default(p3, DIRECTION.INPUT_BACKPROP) == ALGO.WINOGRAD
        assert default(p3, DIRECTION.FILTER_BACKPROP) == ALGO.WINOGRAD
        p1 = ops.conv_params(32, size, size, ch, 4 * ch, 1, 1, False)
        assert default(p1, DIRECTION.FORWARD) == ALGO.MATMUL
    stem = ops.conv_params(32, 224, 224, 3, 64, 7, 2, True)
    assert default(stem, DIRECTION.FORWARD) in (ALGO.TILED, ALGO.IM2COL)
    odd = ops.conv_params(32, 28, 28, 24, 40, 3, 1, True)
    assert default(odd, DIRECTION.FORWARD) in (ALGO.TILED, ALGO.IM2COL)
    assert default(odd, DIRECTION.FILTER_BACKPROP) == ALGO.IM2COL


def test_default_algorithm_and_workspace_know_the_element_type():
    """Half precision has no Winograd kernels: the typed default selector
    never answers Winograd for it, and the typed workspace query reports what
    the half kernels use (a filter-sized block or the filter gradient's
    partial tiles), never the fp32 F(2x2,3x3) transform buffers.  The
    type-blind entries keep answering for float."""
    from portdnn_amd.capi import DTYPE
    for size, ch in [(56, 64), (28, 128), (14, 256), (7, 512)]:
        p3 = ops.conv_params(128, size, size, ch, ch, 3, 1, True)
        p1 = ops.conv_params(128, size, size, ch, 4 * ch, 1, 1, False)
        fil3, fil1 = 9 * ch * ch, 4 * ch * ch
        for d in range(3):
            a32 = ops.default_algorithm(p3, d, DTYPE.F32)
            assert a32 == ops.default_algorithm(p3, d) == ALGO.WINOGRAD
            assert ops.workspace_size(p3, d, a32, DTYPE.F32) == \
                ops.workspace_size(p3, d, a32)
            a16 = ops.default_algorithm(p3, d, DTYPE.F16)
            assert a16 in (ALGO.TILED, ALGO.IM2COL)
            assert capi.lib().snn_hip_conv2d_algorithm_supports(
                ctypes.byref(p3), d, a16) == a16
            assert ops.default_algorithm(p1, d, DTYPE.F16) == ALGO.MATMUL
            # every tag, Winograd included, reports the half kernels' need
            for algo in (a16, ALGO.IM2COL, ALGO.WINOGRAD, ALGO.WINOGRAD_LARGE):
                req, rec = ops.workspace_size(p3, d, algo, DTYPE.F16)
                assert req == 0
                if d == DIRECTION.FILTER_BACKPROP:
                    assert 0 < rec <= 2 * 256 * fil3  # <= 256 fp32 partials
                else:
                    assert rec == fil3
            req, rec = ops.workspace_size(p1, d, ALGO.MATMUL, DTYPE.F16)
            assert req == 0
            if d == DIRECTION.FILTER_BACKPROP:
                assert 0 < rec <= 2 * 256 * fil1
            else:
                assert rec == 0      # W[c][k] is read in place
        assert ops.workspace_size(p3, 0, ALGO.DIRECT, DTYPE.F16) == (0, 0)
    req, rec = ctypes.c_size_t(), ctypes.c_size_t()
    assert capi.lib().snn_hip_conv2d_workspace_size_for(
        ctypes.byref(p3), 0, ALGO.IM2COL, 7, ctypes.byref(req),
        ctypes.byref(rec)) == STATUS.INVALID_PARAMETER
    assert capi.lib().snn_hip_conv2d_default_algorithm_for(
        ctypes.byref(p3), 0, 7) == ALGO.NOT_SUPPORTED


def test_kernel_timing_argument_checks():
    L = capi.lib()
    assert L.snn_hip_kernel_timing_read(None, None) == STATUS.INVALID_PARAMETER
    assert L.snn_hip_kernel_timing_enable(0) == STATUS.OK


def test_elementwise_argument_checks():
    """No device work: null pointers, zero items
    (include/portdnn/internal/pointwise/launch_internal.h:69) and missing
    dimension lists are rejected before any launch."""
    L = capi.lib()
    for name in ("snn_hip_pointwise_forward_f32",
                 "snn_hip_pointwise_forward_f16"):
        assert getattr(L, name)(None, None, 4, 0, None) == \
            STATUS.INVALID_PARAMETER
    buf = ctypes.create_string_buffer(64)
    ptr = ctypes.cast(buf, ctypes.c_void_p)
    assert L.snn_hip_pointwise_forward_f32(ptr, ptr, 0, 0, None) == \
        STATUS.INVALID_PARAMETER
    assert L.snn_hip_pointwise_grad_f32(ptr, None, ptr, 4, 0, None) == \
        STATUS.INVALID_PARAMETER
    assert L.snn_hip_binaryop_f32(ptr, ptr, ptr, None, 2, None, 0, 0, None) == \
        STATUS.INVALID_PARAMETER
    assert L.snn_hip_binaryop_f16(None, ptr, ptr, None, 0, None, 0, 0, None) == \
        STATUS.INVALID_PARAMETER


def test_workspace_sizes_reference_bounds():
    """Lower bounds of test/conv2d/workspace_size.cc:52-160 (VGG layer 1:
    3x3 s1 SAME, 224x224, 64 -> 64, batch 32)."""
    p = ops.conv_params(32, 224, 224, 64, 64, 3, 1, True)
    for algo in (ALGO.DIRECT, ALGO.TILED, ALGO.MATMUL):
        for d in range(3):
            assert ops.workspace_size(p, d, algo) == (0, 0)
    tiles, tile = 224 * 224, 3 * 3 * 64
    fil = 3 * 3 * 64 * 64
    req, rec = ops.workspace_size(p, DIRECTION.FORWARD, ALGO.IM2COL)
    assert req >= tiles * tile and rec >= 32 * tiles * tile
    req, rec = ops.workspace_size(p, DIRECTION.INPUT_BACKPROP, ALGO.IM2COL)
    assert req >= tiles * tile + fil and rec >= 32 * tiles * tile + fil
    req, rec = ops.workspace_size(p, DIRECTION.FILTER_BACKPROP, ALGO.IM2COL)
    assert req >= tiles * tile and rec >= 32 * tiles * tile
    ab = 16
    t = 112 * 112 * 64
    f = 64 * 64
    for d in (DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP):
        for algo in (ALGO.WINOGRAD, ALGO.WINOGRAD_LARGE):
            req, rec = ops.workspace_size(p, d, algo)
            assert req >= ab * (t + f + t)
            assert rec >= ab * (32 * (t + t) + f)
    # WinogradLarge runs the F(2x2,3x3) kernels: it asks for their size
    assert ops.workspace_size(p, DIRECTION.FORWARD, ALGO.WINOGRAD_LARGE) == \
        ops.workspace_size(p, DIRECTION.FORWARD, ALGO.WINOGRAD)
    # the fused F(3x3,2x2) filter gradient stores no transformed tensors, only
    # one partial filter per slice of the tile range: far below the
    # reference's bound for its three transform buffers
    req, rec = ops.workspace_size(p, DIRECTION.FILTER_BACKPROP, ALGO.WINOGRAD)
    assert req == rec and req % (9 * 64 * 64) == 0
    assert 0 < req < ab * (t + t + f)
    # figures quoted for the benchmark layers (Winograd F(2x2,3x3), batch 32)
    p56 = ops.conv_params(32, 56, 56, 64, 64, 3, 1, True)
    req, rec = ops.workspace_size(p56, DIRECTION.FORWARD, ALGO.WINOGRAD)
    assert req == 16 * (28 * 28 * 64 * 2 + 64 * 64)
    assert rec == 16 * (32 * 28 * 28 * 64 * 2 + 64 * 64)


def test_depthwise_and_pooling_validation():
    L = capi.lib()
    d = ops.depthwise_params(2, 8, 8, 4, 1, 3, 1, True)
    d.channel_multiplier = 0
    assert L.snn_hip_depthwise_conv2d_forward_f32(
        FAKE, FAKE, FAKE, ctypes.byref(d), None) == STATUS.INVALID_PARAMETER
    d = ops.depthwise_params(2, 8, 8, 4, 1, 3, 1, True)
    d.input_format = 1  # NCHW is rejected (internal/depthwise_conv2d/launch.h:108)
    assert L.snn_hip_depthwise_conv2d_forward_f32(
        FAKE, FAKE, FAKE, ctypes.byref(d), None) == STATUS.INVALID_PARAMETER
    q = ops.pool_params(2, 8, 8, 4, 3, 2, True)
    q.stride_cols = 0
    assert L.snn_hip_pooling_forward_f32(
        FAKE, FAKE, ctypes.byref(q), 0, None) == STATUS.INVALID_PARAMETER
    q = ops.pool_params(2, 8, 8, 4, 3, 2, True)
    assert L.snn_hip_pooling_max_grad_f32(
        FAKE, FAKE, FAKE, FAKE, ctypes.byref(q), 2,
        None) == STATUS.INVALID_PARAMETER  # Average is not a max operator
    assert L.snn_hip_matmul_f32(FAKE, FAKE, FAKE, 1, 0, 4, 4, 0, 0, 0.0,
                                None) == STATUS.INVALID_PARAMETER


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No CPU fallback: a missing libsnn_hip.so is an error, not a detour."""
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "_LIB_PATH", str(tmp_path / "libsnn_hip.so"))
    with pytest.raises(capi.SnnHipError):
        capi.lib()
