#!/usr/bin/env python3
"""Turn the reference's generated golden tests into compact data fixtures.

The reference keeps its expected outputs as literal arrays inside generated
gtest sources (test/conv2d/forward_window3_stride1.cc:57-67,
test/depthwise_conv2d/forward_window3_stride1.cc, test/pooling/*_forward.cc,
test/pooling/*_grad.cc, test/matmul/matmul_*.cc, test/pointwise/*.cc,
test/binaryop/binaryop_*.cc).  Those sources are parsed here AS TEXT -- nothing is
compiled or executed -- and only the data (case shape, padding mode,
max_input_val and the expected output values) is written to
tests/golden/<group>.npz.  The operands are never stored: every case
regenerates them as 1,2,...,max_val,1,2,... exactly as
test/gen/iota_initialised_data.h:74-79 does.

Run inside the build container only (needs /root/reference):
    python tests/golden/extract_fixtures.py
"""
import os
import re
import sys

import numpy as np

REF = os.environ.get("PORTDNN_REFERENCE", "/root/reference")
OUT = os.path.dirname(os.path.abspath(__file__))

CASE_RE = re.compile(r"TYPED_TEST\((\w+), (\w+)\) \{(.*?)\n\}", re.S)
EXP_RE = re.compile(r"exp_out = \{(.*?)\};", re.S)
SHAPE_RE = re.compile(r"in_shape = \{\{(.*?)\}\}", re.S)
FEAT_RE = re.compile(r"(features|multiplier) = (\d+)")
PAD_RE = re.compile(r"PaddingMode::(\w+)")
MAXV_RE = re.compile(r"max_input_val = ([\d.]+)")

# (window, stride) pairs extracted per family.
CONV_FWD = [(1, 1), (1, 2), (3, 1), (3, 2), (5, 1), (5, 2), (7, 1), (7, 4)]
CONV_BK = [(1, 1), (3, 1), (3, 2), (5, 1), (7, 4)]
DW = [(1, 1), (3, 1), (3, 2), (5, 1), (7, 4)]
POOL_FWD = [(1, 1), (3, 1), (3, 2), (5, 1), (5, 2), (7, 1), (7, 4), (11, 1),
            (11, 4)]
POOL_GRAD = [(3, 1), (3, 2), (5, 2), (7, 1)]


def parse_file(path, window, stride):
    """Returns (meta[int64 n_cases x 10], values[float64]) for one file.

    meta columns: window, stride, N, H, W, C, K_or_multiplier (0 for pooling),
    is_same, max_input_val, n_values.
    """
    with open(path) as f:
        text = f.read()
    metas, vals = [], []
    for _suite, _name, body in CASE_RE.findall(text):
        exp = EXP_RE.search(body).group(1)
        values = np.array(
            [float(tok) for tok in exp.replace("\n", " ").split(",")
             if tok.strip()], dtype=np.float64)
        shape = [int(t) for t in SHAPE_RE.search(body).group(1).split(",")]
        feat = FEAT_RE.search(body)
        k = int(feat.group(2)) if feat else 0
        same = 1 if PAD_RE.search(body).group(1) == "SAME" else 0
        maxv = int(float(MAXV_RE.search(body).group(1)))
        metas.append([window, stride] + shape + [k, same, maxv, values.size])
        vals.append(values)
    if not metas:
        raise RuntimeError("no cases parsed from " + path)
    return np.array(metas, dtype=np.int64), np.concatenate(vals)


def write_group(name, rel_dir, pattern, pairs, integral):
    metas, vals = [], []
    for w, s in pairs:
        path = os.path.join(REF, "test", rel_dir, pattern.format(w=w, s=s))
        m, v = parse_file(path, w, s)
        metas.append(m)
        vals.append(v)
    meta = np.concatenate(metas)
    values = np.concatenate(vals)
    if integral:
        assert np.all(values == np.round(values)), name
        assert np.abs(values).max() <= 2 ** 24, name
        values = values.astype(np.int32)
    out = os.path.join(OUT, name + ".npz")
    np.savez_compressed(out, meta=meta, values=values)
    print("%-28s %5d cases %9d values %8d bytes" %
          (name, len(meta), values.size, os.path.getsize(out)))


def write_padding_kat():
    """Known answers of test/helpers/padding.cc:54-..., one row per input:
    is_same, window, stride, input, expected padding, expected output."""
    with open(os.path.join(REF, "test", "helpers", "padding.cc")) as f:
        text = f.read()
    rows = []
    pat = re.compile(
        r"TYPED_TEST\(PaddingTest, (Valid|Same)Window(\d+)Stride(\d+)\) \{"
        r"(.*?)\n\}", re.S)
    for mode, window, stride, body in pat.findall(text):
        vecs = {}
        for name in ("inputs", "exp_pad", "exp_out"):
            m = re.search(name + r" = \{(.*?)\};", body, re.S)
            vecs[name] = [int(t) for t in m.group(1).split(",")]
        for i, pad, out in zip(vecs["inputs"], vecs["exp_pad"],
                               vecs["exp_out"]):
            rows.append([mode == "Same", int(window), int(stride), i, pad, out])
    rows = np.array(rows, dtype=np.int64)
    assert len(rows) >= 64
    np.savez_compressed(os.path.join(OUT, "padding_kat.npz"), rows=rows)
    print("%-28s %5d rows" % ("padding_kat", len(rows)))


def write_matmul():
    """test/matmul/matmul_batch{1,3}_beta{0,1}_{lhsT}_{rhsT}.cc (27 cases per
    file) and matmul_offset.cc.  meta columns: batches, m, k, n, beta,
    transpose_lhs, transpose_rhs, lhs_offset, rhs_offset, out_offset,
    max_input_val (0 = no wrap), n_values.  Operands and the initial output
    are 1,2,...,max_val,1,... (test/matmul/fixture.h:44-46)."""
    def grab(body, name):
        m = re.search(r"const (?:int|auto|DataType) " + name +
                      r" =\s*(?:static_cast<DataType>\()?([\d.]+)", body)
        return float(m.group(1)) if m else None

    metas, vals = [], []
    files = []
    for b in (1, 3):
        for beta in (0, 1):
            for tl in ("false", "true"):
                for tr in ("false", "true"):
                    files.append(("matmul_batch%d_beta%d_%s_%s.cc" %
                                  (b, beta, tl, tr), tl == "true",
                                  tr == "true"))
    files.append(("matmul_offset.cc", False, False))
    for fname, tl, tr in files:
        with open(os.path.join(REF, "test", "matmul", fname)) as f:
            text = f.read()
        cases = CASE_RE.findall(text)
        assert cases, fname
        for _suite, _name, body in cases:
            exp = re.search(r"exp(?:_out)? = \{(.*?)\};", body, re.S).group(1)
            values = np.array(
                [float(tok) for tok in exp.replace("\n", " ").split(",")
                 if tok.strip()], dtype=np.float64)
            row = [grab(body, n) for n in ("batches", "m", "k", "n", "beta")]
            offs = [grab(body, n) or 0 for n in ("lhs_offset", "rhs_offset",
                                                 "out_offset")]
            maxv = grab(body, "max_input_val") or 0
            metas.append([int(v) for v in row] + [int(tl), int(tr)] +
                         [int(v) for v in offs] + [int(maxv), values.size])
            vals.append(values)
    meta = np.array(metas, dtype=np.int64)
    values = np.concatenate(vals)
    assert np.all(values == np.round(values))
    out = os.path.join(OUT, "matmul.npz")
    np.savez_compressed(out, meta=meta, values=values)
    print("%-28s %5d cases %9d values %8d bytes" %
          ("matmul", len(meta), values.size, os.path.getsize(out)))


def _floats(text):
    return np.array([float(tok) for tok in text.replace("\n", " ").split(",")
                     if tok.strip()], dtype=np.float64)


POINTWISE_FILES = [  # (file, operator id, is_gradient)
    ("relu_forward.cc", 0, 0), ("relu_grad.cc", 0, 1),
    ("tanh_forward.cc", 1, 0), ("tanh_grad.cc", 1, 1),
    ("log_forward.cc", 3, 0), ("log_grad.cc", 3, 1),
    ("floor_forward.cc", 4, 0),
    ("sqrt_forward.cc", 5, 0), ("sqrt_grad.cc", 5, 1),
]


def write_pointwise():
    """test/pointwise/<op>_{forward,grad}.cc.  meta columns: operator
    (0 relu, 1 tanh, 3 log, 4 floor, 5 sqrt), is_gradient, input is signed,
    size, max_val (unsigned generator only), n_values.  Inputs regenerate
    from iota_initialised_signed_data(size) or iota_initialised_data(size,
    max_val) (test/gen/iota_initialised_data.h:74-97); a gradient case feeds
    the same data as forward input and as incoming error
    (test/pointwise/pointwise_fixture.h:80-124)."""
    gen = re.compile(r"input =\s*iota_initialised_(signed_)?data<DataType>\("
                     r"(\d+)(?:,\s*(\d+))?\)")
    metas, vals = [], []
    for fname, op, grad in POINTWISE_FILES:
        with open(os.path.join(REF, "test", "pointwise", fname)) as f:
            text = f.read()
        cases = CASE_RE.findall(text)
        assert cases, fname
        for _suite, _name, body in cases:
            values = _floats(EXP_RE.search(body).group(1))
            m = gen.search(body)
            assert m, (fname, _name)
            signed, size, maxv = m.group(1) is not None, int(m.group(2)), \
                int(m.group(3) or 0)
            assert size == values.size, (fname, _name)
            metas.append([op, grad, int(signed), size, maxv, values.size])
            vals.append(values)
    meta = np.array(metas, dtype=np.int64)
    values = np.concatenate(vals)
    out = os.path.join(OUT, "pointwise.npz")
    np.savez_compressed(out, meta=meta, values=values)
    print("%-28s %5d cases %9d values %8d bytes" %
          ("pointwise", len(meta), values.size, os.path.getsize(out)))


def write_binaryop():
    """test/binaryop/binaryop_{add,sub,mul,div}.cc.  meta columns: operator
    (0 add, 1 sub, 2 mul, 3 div), n_lhs, lhs dims x4, n_rhs, rhs dims x4,
    max_input_val, n_values (unused dims are 0).  Both operands are
    1,2,...,max_val,1,... (test/binaryop/fixture.h:41-45)."""
    metas, vals = [], []
    for op, name in enumerate(("add", "sub", "mul", "div")):
        with open(os.path.join(REF, "test", "binaryop",
                               "binaryop_%s.cc" % name)) as f:
            text = f.read()
        cases = CASE_RE.findall(text)
        assert cases, name
        for _suite, _name, body in cases:
            values = _floats(EXP_RE.search(body).group(1))
            dims = []
            for side in ("lhs_dims", "rhs_dims"):
                m = re.search(side + r" = \{(.*?)\};", body, re.S)
                d = [int(t) for t in m.group(1).split(",") if t.strip()]
                assert len(d) <= 4
                dims.append(d)
            maxv = int(float(MAXV_RE.search(body).group(1)))
            row = [op]
            for d in dims:
                row += [len(d)] + d + [0] * (4 - len(d))
            metas.append(row + [maxv, values.size])
            vals.append(values)
    meta = np.array(metas, dtype=np.int64)
    values = np.concatenate(vals)
    out = os.path.join(OUT, "binaryop.npz")
    np.savez_compressed(out, meta=meta, values=values)
    print("%-28s %5d cases %9d values %8d bytes" %
          ("binaryop", len(meta), values.size, os.path.getsize(out)))


def main():
    if not os.path.isdir(REF):
        sys.exit("reference tree not found at " + REF)
    write_padding_kat()
    write_group("conv2d_forward", "conv2d",
                "forward_window{w}_stride{s}.cc", CONV_FWD, True)
    write_group("conv2d_input_backprop", "conv2d",
                "input_backprop_window{w}_stride{s}.cc", CONV_BK, True)
    write_group("conv2d_filter_backprop", "conv2d",
                "filter_backprop_window{w}_stride{s}.cc", CONV_BK, True)
    write_group("depthwise_forward", "depthwise_conv2d",
                "forward_window{w}_stride{s}.cc", DW, True)
    write_group("depthwise_input_backprop", "depthwise_conv2d",
                "input_backprop_window{w}_stride{s}.cc", DW, True)
    write_group("depthwise_filter_backprop", "depthwise_conv2d",
                "filter_backprop_window{w}_stride{s}.cc", DW, True)
    write_group("pool_max_forward", "pooling",
                "max_window{w}_stride{s}_forward.cc", POOL_FWD, True)
    write_group("pool_avg_forward", "pooling",
                "avg_window{w}_stride{s}_forward.cc", POOL_FWD, False)
    write_group("pool_max_grad", "pooling",
                "max_window{w}_stride{s}_grad.cc", POOL_GRAD, True)
    write_group("pool_avg_grad", "pooling",
                "avg_window{w}_stride{s}_grad.cc", POOL_GRAD, False)
    write_matmul()
    write_pointwise()
    write_binaryop()


if __name__ == "__main__":
    main()
