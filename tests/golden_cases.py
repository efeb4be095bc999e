"""Reader for the golden fixtures under tests/golden/ (data extracted from the
reference's generated tests by tests/golden/extract_fixtures.py)."""
import os
from collections import namedtuple

import numpy as np

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

Case = namedtuple("Case", "window stride n h w c k same max_val expected")


def load(group):
    """Yields every Case of tests/golden/<group>.npz."""
    data = np.load(os.path.join(GOLDEN_DIR, group + ".npz"))
    meta, values = data["meta"], data["values"]
    off = 0
    for row in meta:
        window, stride, n, h, w, c, k, same, max_val, count = (int(v) for v in row)
        yield Case(window, stride, n, h, w, c, k, bool(same), max_val,
                   values[off:off + count])
        off += count
    assert off == values.size


def case_id(case):
    return "w%ds%d_%s%dx%dx%dx%dx%d" % (
        case.window, case.stride, "SAME" if case.same else "VALID", case.n,
        case.h, case.w, case.c, case.k)


MatmulCase = namedtuple(
    "MatmulCase", "batches m k n beta trans_lhs trans_rhs lhs_offset "
    "rhs_offset out_offset max_val expected")


def load_matmul():
    """Yields every MatmulCase of tests/golden/matmul.npz (the reference's
    test/matmul/matmul_batch*_beta*_*.cc and matmul_offset.cc).  `expected`
    covers the whole output buffer, the out_offset leading elements
    included."""
    data = np.load(os.path.join(GOLDEN_DIR, "matmul.npz"))
    off = 0
    for row in data["meta"]:
        (batches, m, k, n, beta, tl, tr, lo, ro, oo, max_val,
         count) = (int(v) for v in row)
        yield MatmulCase(batches, m, k, n, float(beta), bool(tl), bool(tr), lo,
                         ro, oo, max_val, data["values"][off:off + count])
        off += count
    assert off == data["values"].size


POINTWISE_NAMES = {0: "relu", 1: "tanh", 2: "exp", 3: "log", 4: "floor",
                   5: "sqrt"}
PointwiseCase = namedtuple("PointwiseCase",
                           "op is_grad signed size max_val expected")


def load_pointwise():
    """Yields every PointwiseCase of tests/golden/pointwise.npz (the
    reference's test/pointwise/<op>_{forward,grad}.cc)."""
    data = np.load(os.path.join(GOLDEN_DIR, "pointwise.npz"))
    off = 0
    for row in data["meta"]:
        op, grad, signed, size, max_val, count = (int(v) for v in row)
        yield PointwiseCase(POINTWISE_NAMES[op], bool(grad), bool(signed),
                            size, max_val, data["values"][off:off + count])
        off += count
    assert off == data["values"].size


BINARY_NAMES = ("add", "sub", "mul", "div")
BinaryCase = namedtuple("BinaryCase", "op lhs_dims rhs_dims max_val expected")


def load_binaryop():
    """Yields every BinaryCase of tests/golden/binaryop.npz (the reference's
    test/binaryop/binaryop_{add,sub,mul,div}.cc)."""
    data = np.load(os.path.join(GOLDEN_DIR, "binaryop.npz"))
    off = 0
    for row in data["meta"]:
        row = [int(v) for v in row]
        op, n_l, n_r = row[0], row[1], row[6]
        lhs_dims, rhs_dims = row[2:2 + n_l], row[7:7 + n_r]
        max_val, count = row[11], row[12]
        yield BinaryCase(BINARY_NAMES[op], lhs_dims, rhs_dims, max_val,
                         data["values"][off:off + count])
        off += count
    assert off == data["values"].size
