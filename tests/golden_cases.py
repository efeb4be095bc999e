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
