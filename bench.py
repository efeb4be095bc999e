#!/usr/bin/env python3
"""Benchmark of the conv2d forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward pass over the eight fp32 NHWC batch-32 ResNet layers of
the benchmark configuration (3x3 s1 SAME at 56x56x64, 28x28x128, 14x14x256,
7x7x512, plus the 1x1 K=4C layer of each stage), each through the algorithm
the library's default selector picks, inputs resident in HBM.  `value` is
total algorithmic TFLOP/s (2*N*OH*OW*R*S*C*K per layer, whatever the
algorithm).  The same JSON line carries

  roofline      the main kernel of the 3x3 convolutions against the fp32 MFMA
                peak: algorithmic flops per launch over its average duration,
                timed with HIP events on the launch stream,
  cpu_baseline  the reference's tiled algorithm restated in C (oracle/), timed
                on the host cores on a bounded sample of the same layers,
  detail        per-layer / per-algorithm TFLOP/s and the depthwise / pooling
                GB/s against the HBM peak.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the fused Winograd kernel, mean over the four 3x3
# layers, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs (FETCH_SIZE scaled
# by the factor a plain copy kernel of known size shows, 2.0; WRITE_SIZE 1.0).
WINOGRAD_TRAFFIC_BYTES = 42.5e6

RESNET = [(56, 64), (28, 128), (14, 256), (7, 512)]
MOBILENET = [(112, 32, 1), (112, 64, 2), (56, 128, 1), (28, 256, 2),
             (14, 512, 1), (7, 1024, 1)]
BATCH = 32


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-detail", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path "
                 "(run with --gpus 1)")

    import numpy as np
    import torch

    from portdnn_amd import capi, ops
    from portdnn_amd.capi import ALGO, DIRECTION, POOL_OP
    import ctypes

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED)

    def uniform(n):
        return torch.rand(n, device="cuda", generator=gen) * 2 - 1

    def normal(n):
        return torch.randn(n, device="cuda", generator=gen)

    def default_algo(p):
        return capi.lib().snn_hip_conv2d_default_algorithm(
            ctypes.byref(p), DIRECTION.FORWARD)

    def supports(p, algo):
        return capi.lib().snn_hip_conv2d_algorithm_supports(
            ctypes.byref(p), DIRECTION.FORWARD, algo) == algo

    def event_time_ms(fn, reps, warm=3, repeats=5):
        """Duration of one call: `reps` back-to-back calls between two HIP
        events on the launch stream, median over `repeats` such runs."""
        for _ in range(warm):
            fn()
        times = []
        for _ in range(repeats):
            start = torch.cuda.Event(enable_timing=True)
            stop = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for _ in range(reps):
                fn()
            stop.record()
            stop.synchronize()
            times.append(start.elapsed_time(stop) / reps)
        times.sort()
        return times[len(times) // 2]

    # ---- the workload --------------------------------------------------------
    layers = []
    for size, ch in RESNET:
        layers.append(("3x3_%dx%dx%d" % (size, size, ch),
                       ops.conv_params(BATCH, size, size, ch, ch, 3, 1, True)))
    for size, ch in RESNET:
        layers.append(("1x1_%dx%dx%d_k%d" % (size, size, ch, 4 * ch),
                       ops.conv_params(BATCH, size, size, ch, 4 * ch, 1, 1,
                                       False)))
    work = []
    for name, p in layers:
        n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
        algo = default_algo(p)
        _, ws_elems = ops.workspace_size(p, DIRECTION.FORWARD, algo)
        work.append(dict(
            name=name, p=p, algo=algo, x=uniform(n_in), w=uniform(n_fil),
            y=torch.empty(n_out, device="cuda"),
            ws=(torch.empty(ws_elems, device="cuda") if ws_elems else None),
            flops=ops.conv_flops(p, DIRECTION.FORWARD)))
    total_flops = sum(w["flops"] for w in work)

    def step():
        for w in work:
            ops.conv2d(w["x"], w["w"], w["p"], DIRECTION.FORWARD, w["algo"],
                       workspace=w["ws"], out=w["y"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = total_flops / (elapsed / args.steps) / 1e12

    # ---- roofline: the dominant kernel, HIP events on the launch stream -------
    # The library brackets the main kernel of each convolution launch (not the
    # filter preparation in front of it) with events on the stream it launches
    # on; these per-kernel times are what `rocprofv3 --kernel-trace --stats`
    # reports for the same kernel.
    algo_names = {1: "direct", 2: "tiled", 3: "im2col", 4: "winograd",
                  6: "matmul"}
    per_layer = []
    k3_flops = k3_kernel_ms = 0.0
    k3_kernels = 0
    for w in work:
        def call(w=w):
            ops.conv2d(w["x"], w["w"], w["p"], DIRECTION.FORWARD, w["algo"],
                       workspace=w["ws"], out=w["y"])
        ms = event_time_ms(call, reps=20)
        with ops.kernel_timing() as kt:
            for _ in range(20):
                call()
        kernel_ms = kt.total_ms / max(1, kt.kernels)
        tf = w["flops"] / ms / 1e9
        per_layer.append({"layer": w["name"], "algorithm": algo_names[w["algo"]],
                          "ms": round(ms, 4), "kernel_ms": round(kernel_ms, 4),
                          "tflops": round(tf, 2),
                          "frac_mfma_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)})
        if w["name"].startswith("3x3"):
            k3_flops += w["flops"] * kt.kernels
            k3_kernel_ms += kt.total_ms
            k3_kernels += kt.kernels
    achieved = k3_flops / k3_kernel_ms / 1e9
    k3_algos = sorted({algo_names[w["algo"]] for w in work
                       if w["name"].startswith("3x3")})
    roofline = {
        "bound": "mfma",
        "kernel": "main kernel of the 3x3 s1 forward convolution (%s), the four "
                  "ResNet stages, one launch each per step" % "/".join(k3_algos),
        "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS,
        "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
        "avg_kernel_ms": round(k3_kernel_ms / k3_kernels, 5),
        "algorithmic_gflop_per_launch": round(k3_flops / k3_kernels / 1e9, 4),
        # Winograd F(2x2,3x3) executes 16/36 of the algorithmic flops on the
        # matrix cores; this is the MFMA pipe's own utilisation
        "mfma_executed_tflops": round(
            achieved * (4.0 / 9.0 if k3_algos == ["winograd"] else 1.0), 2),
        "mfma_executed_frac": round(
            achieved * (4.0 / 9.0 if k3_algos == ["winograd"] else 1.0) /
            PEAK_FP32_MFMA_TFLOPS, 4),
        "traffic": WINOGRAD_TRAFFIC_BYTES if k3_algos == ["winograd"] else None}

    detail = {"layers": per_layer}
    if not args.no_detail:
        # every algorithm on every 3x3 / 1x1 layer
        algo_table = []
        for w in work:
            for algo in (ALGO.TILED, ALGO.IM2COL, ALGO.WINOGRAD, ALGO.MATMUL,
                         ALGO.DIRECT):
                if not supports(w["p"], algo):
                    continue
                _, ws_elems = ops.workspace_size(w["p"], DIRECTION.FORWARD, algo)
                ws = torch.empty(ws_elems, device="cuda") if ws_elems else None
                ms = event_time_ms(lambda: ops.conv2d(
                    w["x"], w["w"], w["p"], DIRECTION.FORWARD, algo,
                    workspace=ws, out=w["y"]), reps=10, warm=2)
                algo_table.append({"layer": w["name"],
                                   "algorithm": algo_names[algo],
                                   "ms": round(ms, 4),
                                   "tflops": round(w["flops"] / ms / 1e9, 2)})
                del ws
        detail["algorithms"] = algo_table

        # backprops of the 3x3 layers and the 7x7 s2 stem in all directions
        # (flops as the reference's benchmarks count them: by input pixels
        # for the two gradients)
        bk = []
        stem = ops.conv_params(BATCH, 224, 224, 3, 64, 7, 2, True)
        cases = [("stem7x7_s2_224x224x3_k64", stem, d) for d in (
            DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP,
            DIRECTION.FILTER_BACKPROP)]
        for w in work[:4]:
            cases += [(w["name"], w["p"], DIRECTION.INPUT_BACKPROP),
                      (w["name"], w["p"], DIRECTION.FILTER_BACKPROP)]
        dir_names = {DIRECTION.FORWARD: "forward",
                     DIRECTION.INPUT_BACKPROP: "input_backprop",
                     DIRECTION.FILTER_BACKPROP: "filter_backprop"}
        for name, p, direction in cases:
            algo = capi.lib().snn_hip_conv2d_default_algorithm(
                ctypes.byref(p), direction)
            n_a, n_b, n_o = ops.conv_sizes(p, direction)
            _, ws_elems = ops.workspace_size(p, direction, algo)
            a, b = uniform(n_a), uniform(n_b)
            o = torch.empty(n_o, device="cuda")
            ws = torch.empty(ws_elems, device="cuda") if ws_elems else None
            ms = event_time_ms(lambda: ops.conv2d(
                a, b, p, direction, algo, workspace=ws, out=o), reps=10,
                warm=2, repeats=3)
            fl = ops.conv_flops(p, direction)
            bk.append({"layer": name, "direction": dir_names[direction],
                       "algorithm": algo_names[algo], "ms": round(ms, 4),
                       "tflops": round(fl / ms / 1e9, 2)})
            del a, b, o, ws
        detail["backprop_and_stem"] = bk

        # half precision (fp32 accumulation), batch 128
        h = []
        for size, ch in RESNET:
            for window, feats in ((3, ch), (1, 4 * ch)):
                p = ops.conv_params(128, size, size, ch, feats, window, 1,
                                    window == 3)
                n_a, n_b, n_o = ops.conv_sizes(p, DIRECTION.FORWARD)
                a, b = uniform(n_a).half(), uniform(n_b).half()
                o = torch.empty(n_o, device="cuda", dtype=torch.float16)
                ws = torch.empty(n_b, device="cuda", dtype=torch.float16)
                ms = event_time_ms(lambda: ops.conv2d(
                    a, b, p, DIRECTION.FORWARD, ALGO.IM2COL, workspace=ws,
                    out=o), reps=10, warm=2, repeats=3)
                fl = ops.conv_flops(p, DIRECTION.FORWARD)
                h.append({"op": "conv%dx%d_%dx%dx%d_k%d_b128_f16" % (
                    window, window, size, size, ch, feats), "ms": round(ms, 4),
                    "tflops": round(fl / ms / 1e9, 1),
                    "frac_f16_mfma_peak": round(fl / ms / 1e9 / 2500.0, 4)})
                if window == 3:
                    # input gradient: the same kernel on dY (o) with the
                    # filter's taps mirrored and its roles swapped
                    dx = torch.empty(n_a, device="cuda", dtype=torch.float16)
                    o.copy_(uniform(n_o).half())
                    ms = event_time_ms(lambda: ops.conv2d(
                        o, b, p, DIRECTION.INPUT_BACKPROP, ALGO.IM2COL,
                        workspace=ws, out=dx), reps=10, warm=2, repeats=3)
                    fl = ops.conv_flops(p, DIRECTION.INPUT_BACKPROP)
                    h.append({"op": "conv3x3_%dx%dx%d_k%d_b128_f16_input_"
                              "backprop" % (size, size, ch, feats),
                              "ms": round(ms, 4),
                              "tflops": round(fl / ms / 1e9, 1),
                              "frac_f16_mfma_peak": round(
                                  fl / ms / 1e9 / 2500.0, 4)})
                    del dx
                del a, b, o, ws
        for size, ch, stride in MOBILENET:
            p = ops.depthwise_params(128, size, size, ch, 1, 3, stride, True)
            n_a, n_b, n_o = ops.depthwise_sizes(p, DIRECTION.FORWARD)
            nbytes = 2 * (n_a + n_b + n_o)
            sets = max(3, int(600e6 // nbytes) + 1)
            xs = [normal(n_a).half() for _ in range(sets)]
            ys = [torch.empty(n_o, device="cuda", dtype=torch.float16)
                  for _ in range(sets)]
            f = normal(n_b).half()
            state = {"i": 0}

            def run_h():
                i = state["i"] % sets
                state["i"] += 1
                ops.depthwise_conv2d(xs[i], f, p, out=ys[i])
            ms = event_time_ms(run_h, reps=5 * sets, warm=sets, repeats=3)
            gbs = nbytes / ms / 1e6
            h.append({"op": "depthwise3x3_%dx%dx%d_s%d_b128_f16" % (
                size, size, ch, stride), "bytes": nbytes, "ms": round(ms, 5),
                "gbs": round(gbs, 1),
                "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)})
            del xs, ys
        detail["f16_batch128"] = h

        # memory-bound operators: rotate buffer sets so that the 256 MB
        # last-level cache cannot hold the working set between launches
        mem = []

        def rotate_sets(nbytes):
            return max(3, int(600e6 // nbytes) + 1)

        def device_ms(fn, calls):
            """Mean device time of one call: HIP events the library records
            on the launch stream around the kernels of each call (what
            rocprofv3 reports per kernel), free of the host's launch rate,
            which bounds `ms` for the smallest layers."""
            with ops.kernel_timing() as kt:
                for _ in range(calls):
                    fn()
            return kt.total_ms / max(1, kt.kernels)

        def mem_entry(name, nbytes, ms, kernel_ms):
            gbs = nbytes / ms / 1e6
            kgbs = nbytes / kernel_ms / 1e6
            return {"op": name, "bytes": nbytes, "ms": round(ms, 5),
                    "gbs": round(gbs, 1),
                    "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                    "kernel_ms": round(kernel_ms, 5),
                    "kernel_gbs": round(kgbs, 1),
                    "kernel_frac_hbm_peak": round(kgbs / PEAK_HBM_GBS, 4)}

        for size, ch, stride in MOBILENET:
            p = ops.depthwise_params(BATCH, size, size, ch, 1, 3, stride, True)
            n_in, n_fil, n_out = ops.depthwise_sizes(p, DIRECTION.FORWARD)
            nbytes = 4 * (n_in + n_fil + n_out)
            sets = rotate_sets(nbytes)
            xs = [normal(n_in) for _ in range(sets)]
            ys = [torch.empty(n_out, device="cuda") for _ in range(sets)]
            f = normal(n_fil)
            state = {"i": 0}

            def run():
                i = state["i"] % sets
                state["i"] += 1
                ops.depthwise_conv2d(xs[i], f, p, out=ys[i])
            ms = event_time_ms(run, reps=5 * sets, warm=sets, repeats=3)
            mem.append(mem_entry(
                "depthwise3x3_%dx%dx%d_s%d" % (size, size, ch, stride), nbytes,
                ms, device_ms(run, 5 * sets)))
            del xs, ys
        for name, p, op in (
                ("maxpool3x3_s2_112x112x64",
                 ops.pool_params(BATCH, 112, 112, 64, 3, 2, True), POOL_OP.MAX),
                ("avgpool7x7_7x7x2048",
                 ops.pool_params(BATCH, 7, 7, 2048, 7, 1, False),
                 POOL_OP.AVERAGE)):
            n_in = p.batch * p.in_rows * p.in_cols * p.channels
            n_out = p.batch * p.out_rows * p.out_cols * p.channels
            nbytes = 4 * (n_in + n_out)
            sets = rotate_sets(nbytes)
            xs = [normal(n_in) for _ in range(sets)]
            ys = [torch.empty(n_out, device="cuda") for _ in range(sets)]
            state = {"i": 0}

            def run():
                i = state["i"] % sets
                state["i"] += 1
                ops.pooling_forward(xs[i], p, op, out=ys[i])
            ms = event_time_ms(run, reps=5 * sets, warm=sets, repeats=3)
            mem.append(mem_entry(name, nbytes, ms, device_ms(run, 5 * sets)))
            del xs, ys
        detail["memory_bound"] = mem

        # element-wise operators on the 56x56x256 activation of the first
        # ResNet stage: ReLU (read + write) and bias add (read + write + bias)
        from portdnn_amd.capi import BINARY_OP, POINTWISE_OP
        elem = []
        dims = [BATCH, 56, 56, 256]
        n_act = BATCH * 56 * 56 * 256
        sets = rotate_sets(8 * n_act)
        xs = [normal(n_act) for _ in range(sets)]
        ys = [torch.empty(n_act, device="cuda") for _ in range(sets)]
        bias = normal(256)
        state = {"i": 0}

        def run_relu():
            i = state["i"] % sets
            state["i"] += 1
            ops.pointwise_forward(xs[i], POINTWISE_OP.RELU, out=ys[i])

        def run_bias():
            i = state["i"] % sets
            state["i"] += 1
            ops.binaryop(xs[i], bias, dims, [256], BINARY_OP.ADD, out=ys[i])
        for name, fn, nbytes in (("relu_56x56x256", run_relu, 8 * n_act),
                                 ("bias_add_56x56x256", run_bias,
                                  8 * n_act + 1024)):
            ms = event_time_ms(fn, reps=5 * sets, warm=sets, repeats=3)
            gbs = nbytes / ms / 1e6
            elem.append({"op": name, "bytes": nbytes, "ms": round(ms, 5),
                         "gbs": round(gbs, 1),
                         "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)})
        del xs, ys
        detail["elementwise"] = elem

        # convolution + bias + ReLU: three launches (the reference's
        # composition) against the entry point that folds bias and
        # activation into the convolution's output stage
        fused = []
        for name, p in layers:
            algo = default_algo(p)
            n_in, n_fil, n_out = ops.conv_sizes(p, DIRECTION.FORWARD)
            x, f, b = uniform(n_in), uniform(n_fil), uniform(p.features)
            y = torch.empty(n_out, device="cuda")
            _, rec = ops.workspace_size(p, DIRECTION.FORWARD, algo)
            ws = torch.empty(max(rec, 1), device="cuda")
            out_dims = [p.batch, p.out_rows, p.out_cols, p.features]

            def three():
                ops.conv2d(x, f, p, DIRECTION.FORWARD, algo, workspace=ws,
                           out=y)
                ops.binaryop(y, b, out_dims, [p.features], BINARY_OP.ADD,
                             out=y)
                ops.pointwise_forward(y, POINTWISE_OP.RELU, out=y)

            def one():
                ops.conv2d_bias_act(x, f, b, p, algo, relu=True, workspace=ws,
                                    out=y)
            fused.append({"layer": name,
                          "three_launches_ms": round(
                              event_time_ms(three, reps=30), 5),
                          "fused_ms": round(event_time_ms(one, reps=30), 5)})
        detail["conv_bias_relu"] = fused

        # gradients of the memory-bound operators (same byte accounting:
        # every operand read or written once)
        grads = []
        for size, ch, stride in MOBILENET[:4]:
            p = ops.depthwise_params(BATCH, size, size, ch, 1, 3, stride, True)
            for direction, tag in ((DIRECTION.INPUT_BACKPROP, "input_backprop"),
                                   (DIRECTION.FILTER_BACKPROP,
                                    "filter_backprop")):
                n_a, n_b, n_o = ops.depthwise_sizes(p, direction)
                nbytes = 4 * (n_a + n_b + n_o)
                sets = rotate_sets(nbytes)
                a_s = [normal(n_a) for _ in range(sets)]
                b_s = ([normal(n_b) for _ in range(sets)]
                       if direction == DIRECTION.FILTER_BACKPROP
                       else [normal(n_b)] * sets)
                o_s = [torch.empty(n_o, device="cuda") for _ in range(sets)]
                state = {"i": 0}

                def run():
                    i = state["i"] % sets
                    state["i"] += 1
                    ops.depthwise_conv2d(a_s[i], b_s[i], p, direction,
                                         out=o_s[i])
                ms = event_time_ms(run, reps=5 * sets, warm=sets, repeats=3)
                grads.append(mem_entry(
                    "depthwise3x3_%dx%dx%d_s%d_%s" % (size, size, ch, stride,
                                                      tag),
                    nbytes, ms, device_ms(run, 5 * sets)))
                del a_s, b_s, o_s
        p = ops.pool_params(BATCH, 112, 112, 64, 3, 2, True)
        n_in = p.batch * p.in_rows * p.in_cols * p.channels
        n_out = p.batch * p.out_rows * p.out_cols * p.channels
        sets = rotate_sets(4 * (2 * n_in + 2 * n_out))
        xs = [normal(n_in) for _ in range(sets)]
        ys = [ops.pooling_forward(x, p, POOL_OP.MAX) for x in xs]
        dys = [normal(n_out) for _ in range(sets)]
        dxs = [torch.empty(n_in, device="cuda") for _ in range(sets)]
        state = {"i": 0}

        def run_max_grad():
            i = state["i"] % sets
            state["i"] += 1
            ops.pooling_max_grad(xs[i], ys[i], dys[i], p, dx=dxs[i])
        ms = event_time_ms(run_max_grad, reps=3 * sets, warm=sets, repeats=3)
        grads.append(mem_entry("maxpool3x3_s2_112x112x64_grad",
                               4 * (2 * n_in + 2 * n_out), ms,
                               device_ms(run_max_grad, 3 * sets)))

        def run_avg_grad():
            i = state["i"] % sets
            state["i"] += 1
            ops.pooling_avg_grad(dys[i], p, dx=dxs[i])
        ms = event_time_ms(run_avg_grad, reps=3 * sets, warm=sets, repeats=3)
        grads.append(mem_entry("avgpool3x3_s2_112x112x64_grad",
                               4 * (n_in + n_out), ms,
                               device_ms(run_avg_grad, 3 * sets)))
        del xs, ys, dys, dxs
        detail["memory_bound_gradients"] = grads

        # the public matmul op (sycldnn::matmul::launch) on the same MFMA kernel
        mm = []
        for batches, m, k, n, tb in ((1, 4096, 1024, 1024, False),
                                    (1, 4096, 1024, 1024, True),
                                    (16, 1568, 256, 256, False)):
            a = uniform(batches * m * k)
            b = uniform(batches * k * n)
            c = torch.empty(batches * m * n, device="cuda")
            ms = event_time_ms(lambda: ops.matmul(a, b, batches, m, k, n, False,
                                                  tb, 0.0, out=c), reps=10,
                               warm=2, repeats=3)
            tf = 2.0 * batches * m * k * n / ms / 1e9
            mm.append({"op": "matmul b%d %dx%dx%d%s" % (
                batches, m, k, n, " rhs^T" if tb else ""), "ms": round(ms, 4),
                "tflops": round(tf, 2),
                "frac_mfma_peak": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)})
        detail["matmul"] = mm

    # ---- CPU baseline: the reference's tiled algorithm, restated --------------
    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        cores = oracle.set_threads(0)
        rng = np.random.default_rng(0x5EED)
        cpu_flops = 0.0
        cpu_s = 0.0
        cpu_batch = 8
        cases = []
        for size, ch in RESNET:
            for window, feats in ((3, ch), (1, 4 * ch)):
                p = oracle.make_params(cpu_batch, size, size, ch, feats, window,
                                       1, window == 3)
                x = rng.uniform(-1, 1, cpu_batch * size * size * ch).astype(
                    np.float32)
                w = rng.uniform(-1, 1, window * window * ch * feats).astype(
                    np.float32)
                cases.append((p, x, w, 2.0 * cpu_batch * size * size * window *
                              window * ch * feats))
        for p, x, w, _ in cases:               # warm-up pass, as the
            oracle.conv2d_tiled_forward(x, w, p)   # reference's executor does
        passes = 0
        while cpu_s < 10.0 and passes < 40:
            for p, x, w, fl in cases:
                t = time.perf_counter()
                oracle.conv2d_tiled_forward(x, w, p)
                cpu_s += time.perf_counter() - t
                cpu_flops += fl
            passes += 1
        cpu = {"value": round(cpu_flops / cpu_s / 1e12, 5), "unit": "TFLOP/s",
               "cores": cores, "kind": "port",
               "sample": "%d passes over batch %d of each of the 8 layers, "
                         "portDNN tiled algorithm (2x2x4 register tiles) "
                         "restated in C with OpenMP; %.1f s of CPU time"
                         % (passes, cpu_batch, cpu_s)}

    line = {
        "metric": "conv2d fwd TFLOP/s + %MFMA peak; depthwise/pool GB/s + "
                  "%HBM peak, 1 GPU",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "conv2d forward fp32 NHWC batch 32: 3x3 s1 "
                               "SAME at (56,64),(28,128),(14,256),(7,512) + "
                               "1x1 K=4C at each stage; default selector",
                   "batch": BATCH},
        "roofline": roofline, "cpu_baseline": cpu, "detail": detail,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
