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
                peak: `achieved` = algorithmic flops per launch over its
                average duration, timed with HIP events on the launch stream;
                `frac_algorithmic` = achieved / peak, `frac` = the part of it
                the matrix cores really execute (16/36 for Winograd) / peak;
                `traffic` is read from the committed rocprofv3 summary named
                in `traffic_source`.  The memory-bound half of the metric is
                there as plain numbers: `hbm_<layer>_gbs` / `_frac` (of the
                8 TB/s peak) / `_of_stream` (of what a ReLU stream of the same
                byte count reaches in the same run: the ceiling a launch of
                that size has on this GPU) for the depthwise and pooling
                layers, `config0_*` for the single-image 56x56x64 layer,
  cpu_baseline  the reference's algorithms restated in C (oracle/), timed on
                the host cores on bounded samples: the tiled convolution on
                the same eight layers (`value`), the depthwise and pooling
                loops (`depthwise_gbs`, `maxpool_gbs`, `avgpool_gbs`) and the
                single-image layer (`config0_tflops`),
  detail        per-layer / per-algorithm TFLOP/s, gradients, half precision.

No executed fraction of a peak may exceed 1: `frac()` raises if one does.
Fractions of the algorithmic flops (the direct convolution's count, the
metric's definition) may: a Winograd launch executes 16/36 of them.
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
# HBM bytes per launch of the dominant kernel come from this committed
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary (its header says how the
# counters were scaled): the "HBM MB / launch" column of the rows of the
# kernel, averaged over the four 3x3 layers.
TRAFFIC_PROFILE = os.path.join("profiles",
                               "conv2d_forward_resnet_batch32_hbm_traffic.md")


def profiled_traffic_bytes(kernel_prefix):
    """Mean of the 'HBM MB / launch' column over the table rows whose kernel
    name starts with `kernel_prefix`, in bytes; None if there is no such row."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    if not os.path.exists(path):
        return None
    column = None
    values = []
    with open(path) as f:
        for line in f:
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if "HBM MB / launch" in cells:
                column = cells.index("HBM MB / launch")
            elif (column is not None and cells and
                  cells[0].strip("`").startswith(kernel_prefix) and
                  len(cells) > column):
                values.append(float(cells[column]))
    return sum(values) / len(values) * 1e6 if values else None


def frac(value, peak, executed_share=1.0):
    """value / peak, rounded.  `value` counts the algorithm-independent work
    (the direct convolution's flops); `executed_share` is the part of it the
    kernel really executes (16/36 for Winograd F(2x2,3x3)).  Executed work
    above the peak means the accounting is wrong; algorithmic work above it is
    what a fast algorithm is for."""
    if value * executed_share > peak:
        raise AssertionError("executed fraction of peak above 1: %r x %r / %r"
                             % (value, executed_share, peak))
    return round(value / peak, 4)


WINOGRAD_SHARE = 4.0 / 9.0

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

    # (calls bound once: each is then one C ABI call per launch, without the
    # Python wrapper's per-call argument conversions)
    step_calls = [ops.conv2d_bound(w["x"], w["w"], w["y"], w["p"],
                                   DIRECTION.FORWARD, w["algo"], w["ws"])
                  for w in work]

    def step():
        for call in step_calls:
            call()

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

    # The same step with the filters prepared once, outside the timed region
    # (snn_hip_conv2d_prepare_filter_f32 + snn_hip_conv2d_prepared_f32: the
    # inference case, one filter for many launches).  Reported beside `value`,
    # which stays the one-call form that transforms the filter in every launch.
    for w in work:
        if w["ws"] is not None:
            ops.conv2d_prepare_filter(w["w"], w["p"], DIRECTION.FORWARD,
                                      w["algo"], w["ws"])

    prepared_calls = [
        ops.conv2d_prepared_bound(w["x"], w["w"], w["y"], w["p"],
                                  DIRECTION.FORWARD, w["algo"], w["ws"])
        if w["ws"] is not None else
        ops.conv2d_bound(w["x"], w["w"], w["y"], w["p"], DIRECTION.FORWARD,
                         w["algo"])
        for w in work]

    def step_prepared():
        for call in prepared_calls:
            call()
    for _ in range(args.warmup):
        step_prepared()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_prepared()
    torch.cuda.synchronize()
    prepared_ms = (time.perf_counter() - t0) * 1e3 / args.steps

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
    executed_flops_per_step = 0.0
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
                          "frac_mfma_peak": frac(
                              tf, PEAK_FP32_MFMA_TFLOPS,
                              WINOGRAD_SHARE
                              if algo_names[w["algo"]] == "winograd" else 1.0)})
        executed_flops_per_step += w["flops"] * (
            WINOGRAD_SHARE if algo_names[w["algo"]] == "winograd" else 1.0)
        if w["name"].startswith("3x3"):
            k3_flops += w["flops"] * kt.kernels
            k3_kernel_ms += kt.total_ms
            k3_kernels += kt.kernels
    achieved = k3_flops / k3_kernel_ms / 1e9
    k3_algos = sorted({algo_names[w["algo"]] for w in work
                       if w["name"].startswith("3x3")})
    k3_share = WINOGRAD_SHARE if k3_algos == ["winograd"] else 1.0
    roofline = {
        "bound": "mfma",
        "kernel": "main kernel of the 3x3 s1 forward convolution (%s), the four "
                  "ResNet stages, one launch each per step" % "/".join(k3_algos),
        # algorithmic flops (the direct convolution's count, as the metric is
        # defined) per launch over the kernel's duration
        "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS,
        "unit": "TFLOP/s",
        # the matrix pipe's own figure: the multiplications really executed
        # (16/36 of the algorithmic count for Winograd F(2x2,3x3)) over the peak
        "frac": frac(achieved * k3_share, PEAK_FP32_MFMA_TFLOPS),
        # algorithmic flops over the peak; above 1 when the Winograd kernel
        # outruns what the matrix cores could do on the direct algorithm
        "frac_algorithmic": frac(achieved, PEAK_FP32_MFMA_TFLOPS, k3_share),
        "achieved_executed": round(achieved * k3_share, 2),
        "avg_kernel_ms": round(k3_kernel_ms / k3_kernels, 5),
        "algorithmic_gflop_per_launch": round(k3_flops / k3_kernels / 1e9, 4),
        # the whole step (Winograd layers at 16/36 of their flops, the 1x1
        # GEMM layers at all of them) over the step time
        "step_executed_tflops": round(
            executed_flops_per_step / ms_per_step / 1e9, 2),
        "step_executed_frac": frac(
            executed_flops_per_step / ms_per_step / 1e9,
            PEAK_FP32_MFMA_TFLOPS),
        # the step with every filter transformed once beforehand (two-call
        # form); `value` is the one-call form
        "step_filter_prepared_ms": round(prepared_ms, 4),
        "step_filter_prepared_tflops": round(
            total_flops / prepared_ms / 1e9, 3),
        # not measured in this run: FETCH_SIZE / WRITE_SIZE of the same kernel
        # from the committed rocprofv3 summary
        "traffic": (profiled_traffic_bytes("wino_direct_kernel")
                    if k3_algos == ["winograd"] else None),
        "traffic_source": "committed profile, not this run: " + TRAFFIC_PROFILE}

    # ---- memory-bound half of the metric: depthwise and pooling against HBM ----
    # Buffer sets rotate so that the 256 MB last-level cache cannot hold the
    # working set between launches.
    def rotate_sets(nbytes):
        return max(3, int(600e6 // nbytes) + 1)

    def device_ms(fn, calls):
        """Mean device time of one call: HIP events the library records on the
        launch stream around the kernels of each call (what rocprofv3 reports
        per kernel), free of the host's launch rate, which bounds `ms` for
        the smallest layers."""
        with ops.kernel_timing() as kt:
            for _ in range(calls):
                fn()
        return kt.total_ms / max(1, kt.kernels)

    from portdnn_amd.capi import POINTWISE_OP
    stream_cache = {}

    def stream_ms(nbytes):
        """What a launch that moves `nbytes` can reach on this GPU: a ReLU
        stream (snn_hip_pointwise_forward_f32: every element read once and
        written once, 16 bytes per lane per access) of the same total byte
        count, timed the same way as the kernels it is compared with."""
        n = max(4, int(nbytes // 8) // 4 * 4)
        if n not in stream_cache:
            sets = rotate_sets(8 * n)
            xs = [normal(n) for _ in range(sets)]
            ys = [torch.empty(n, device="cuda") for _ in range(sets)]
            state = {"i": 0}

            calls = [ops.pointwise_forward_bound(xs[i], ys[i],
                                                 POINTWISE_OP.RELU)
                     for i in range(sets)]

            def run():
                i = state["i"] % sets
                state["i"] += 1
                calls[i]()
            stream_cache[n] = (
                event_time_ms(run, reps=5 * sets, warm=sets, repeats=3),
                device_ms(run, 5 * sets))
            del xs, ys
        return stream_cache[n]

    def mem_entry(name, nbytes, ms, kernel_ms, with_stream=True):
        gbs = nbytes / ms / 1e6
        kgbs = nbytes / kernel_ms / 1e6
        entry = {"op": name, "bytes": nbytes, "ms": round(ms, 5),
                 "gbs": round(gbs, 1),
                 "frac_hbm_peak": frac(gbs, PEAK_HBM_GBS),
                 "kernel_ms": round(kernel_ms, 5),
                 "kernel_gbs": round(kgbs, 1),
                 "kernel_frac_hbm_peak": frac(kgbs, PEAK_HBM_GBS)}
        if with_stream:
            s_ms, s_kernel_ms = stream_ms(nbytes)
            entry["stream_same_bytes_ms"] = round(s_ms, 5)
            entry["stream_same_bytes_gbs"] = round(nbytes / s_ms / 1e6, 1)
            entry["of_stream"] = round(s_ms / ms, 4)
            entry["stream_same_bytes_kernel_ms"] = round(s_kernel_ms, 5)
        return entry

    def depthwise_entry(size, ch, stride):
        p = ops.depthwise_params(BATCH, size, size, ch, 1, 3, stride, True)
        n_in, n_fil, n_out = ops.depthwise_sizes(p, DIRECTION.FORWARD)
        nbytes = 4 * (n_in + n_fil + n_out)
        sets = rotate_sets(nbytes)
        xs = [normal(n_in) for _ in range(sets)]
        ys = [torch.empty(n_out, device="cuda") for _ in range(sets)]
        f = normal(n_fil)
        state = {"i": 0}

        calls = [ops.depthwise_conv2d_bound(xs[i], f, ys[i], p)
                 for i in range(sets)]

        def run():
            i = state["i"] % sets
            state["i"] += 1
            calls[i]()
        ms = event_time_ms(run, reps=5 * sets, warm=sets, repeats=3)
        return mem_entry("depthwise3x3_%dx%dx%d_s%d" % (size, size, ch, stride),
                         nbytes, ms, device_ms(run, 5 * sets))

    def pooling_entry(name, p, op):
        n_in = p.batch * p.in_rows * p.in_cols * p.channels
        n_out = p.batch * p.out_rows * p.out_cols * p.channels
        nbytes = 4 * (n_in + n_out)
        sets = rotate_sets(nbytes)
        xs = [normal(n_in) for _ in range(sets)]
        ys = [torch.empty(n_out, device="cuda") for _ in range(sets)]
        state = {"i": 0}

        calls = [ops.pooling_forward_bound(xs[i], ys[i], p, op)
                 for i in range(sets)]

        def run():
            i = state["i"] % sets
            state["i"] += 1
            calls[i]()
        ms = event_time_ms(run, reps=5 * sets, warm=sets, repeats=3)
        return mem_entry(name, nbytes, ms, device_ms(run, 5 * sets))

    POOLS = (("maxpool3x3_s2_112x112x64",
              ops.pool_params(BATCH, 112, 112, 64, 3, 2, True), POOL_OP.MAX),
             ("avgpool7x7_7x7x2048",
              ops.pool_params(BATCH, 7, 7, 2048, 7, 1, False), POOL_OP.AVERAGE))
    mem = [depthwise_entry(*layer) for layer in MOBILENET]
    mem += [pooling_entry(*pool) for pool in POOLS]
    # The entries a reader needs beside the convolution figure: kernel = what
    # ran, bytes_per_launch = (input + filter + output) * 4, the time of one
    # launch and the fraction of the 8 TB/s peak.  ms_per_launch is the mean
    # over back-to-back launches between two stream events (an upper bound of
    # the kernel's own duration, which rocprofv3 reports; the per-launch event
    # pairs behind `kernel_ms` in detail.memory_bound add 2-3 us to kernels
    # this short).
    # (plain numbers under flat keys: a reader that keeps only the scalar
    # members of `roofline` still gets the memory-bound half of the metric)
    short = {"depthwise3x3_112x112x32_s1": "dw_112x112x32_s1",
             "depthwise3x3_112x112x64_s2": "dw_112x112x64_s2",
             "depthwise3x3_56x56x128_s1": "dw_56x56x128_s1",
             "depthwise3x3_28x28x256_s2": "dw_28x28x256_s2",
             "depthwise3x3_14x14x512_s1": "dw_14x14x512_s1",
             "depthwise3x3_7x7x1024_s1": "dw_7x7x1024_s1",
             "maxpool3x3_s2_112x112x64": "maxpool",
             "avgpool7x7_7x7x2048": "avgpool"}
    roofline["hbm_peak_gbs"] = PEAK_HBM_GBS
    for e in mem:
        key = "hbm_" + short[e["op"]]
        roofline[key + "_mb"] = round(e["bytes"] / 1e6, 2)
        roofline[key + "_us"] = round(e["ms"] * 1e3, 2)
        roofline[key + "_gbs"] = e["gbs"]
        roofline[key + "_frac"] = e["frac_hbm_peak"]
        roofline[key + "_of_stream"] = e["of_stream"]
    # the ceiling itself: the ReLU stream at round sizes (read + write bytes)
    for mb in (13, 26, 32, 103, 128, 256, 411):
        s_ms, _ = stream_ms(mb * 1e6)
        roofline["hbm_stream_%dmb_gbs" % mb] = round(mb / s_ms, 1)
        roofline["hbm_stream_%dmb_frac" % mb] = frac(mb / s_ms, PEAK_HBM_GBS)

    # ---- configuration 0: one 56x56x64 image, 3x3 s1 SAME, Tiled -------------
    p0 = ops.conv_params(1, 56, 56, 64, 64, 3, 1, True)
    x0, w0 = uniform(56 * 56 * 64), uniform(9 * 64 * 64)
    y0 = torch.empty(56 * 56 * 64, device="cuda")

    call0 = ops.conv2d_bound(x0, w0, y0, p0, DIRECTION.FORWARD, ALGO.TILED)
    ms0 = event_time_ms(call0, reps=50)
    with ops.kernel_timing() as kt:
        for _ in range(50):
            call0()
    kms0 = kt.total_ms / max(1, kt.kernels)
    fl0 = ops.conv_flops(p0, DIRECTION.FORWARD)
    roofline["config0_workload"] = ("conv2d forward fp32 [1,56,56,64] x "
                                    "[3,3,64,64], s1 SAME, Tiled")
    roofline["config0_gflop"] = round(fl0 / 1e9, 4)
    roofline["config0_ms"] = round(ms0, 5)
    roofline["config0_tflops"] = round(fl0 / ms0 / 1e9, 2)
    roofline["config0_frac"] = frac(fl0 / ms0 / 1e9, PEAK_FP32_MFMA_TFLOPS)
    roofline["config0_kernel_ms"] = round(kms0, 5)

    detail = {"layers": per_layer, "memory_bound": mem}
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
                if algo in (ALGO.TILED, ALGO.IM2COL, ALGO.WINOGRAD):
                    # scalar copy for readers that keep only flat members:
                    # algorithmic fraction of the fp32 MFMA peak, whole call
                    roofline["%s_%s_frac" % (algo_names[algo], w["name"])] = \
                        round(w["flops"] / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)
                del ws
        detail["algorithms"] = algo_table

        # backprops of the 3x3 and 1x1 layers and the 7x7 s2 stem in all
        # directions.
        # `tflops_reference_accounting` counts the two gradients by input
        # pixels, 2*N*H*W*R*S*C*K, as the reference's benchmarks do
        # (bench/conv2d/base_convolution_fixture.h:91-109), which at stride 2
        # is four times the multiplies a gradient needs; `tflops` and the
        # fraction of the peak count the multiply-adds of the convolution
        # itself, 2*N*OH*OW*R*S*C*K, in every direction.
        bk = []
        stem = ops.conv_params(BATCH, 224, 224, 3, 64, 7, 2, True)
        cases = [("stem7x7_s2_224x224x3_k64", stem, d) for d in (
            DIRECTION.FORWARD, DIRECTION.INPUT_BACKPROP,
            DIRECTION.FILTER_BACKPROP)]
        for w in work[:8]:  # the four 3x3 layers, then the four 1x1 layers
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
            fl_ref = ops.conv_flops(p, direction)
            fl = ops.conv_flops(p, DIRECTION.FORWARD)
            bk.append({"layer": name, "direction": dir_names[direction],
                       "algorithm": algo_names[algo], "ms": round(ms, 4),
                       "tflops": round(fl / ms / 1e9, 2),
                       "frac_mfma_peak": frac(
                           fl / ms / 1e9, PEAK_FP32_MFMA_TFLOPS,
                           WINOGRAD_SHARE
                           if algo_names[algo] == "winograd" else 1.0),
                       "tflops_reference_accounting": round(
                           fl_ref / ms / 1e9, 2)})
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
                    out=o), reps=30, warm=5, repeats=3)
                fl = ops.conv_flops(p, DIRECTION.FORWARD)
                entry = {"op": "conv%dx%d_%dx%dx%d_k%d_b128_f16" % (
                    window, window, size, size, ch, feats), "ms": round(ms, 4),
                    "tflops": round(fl / ms / 1e9, 1),
                    "frac_f16_mfma_peak": frac(fl / ms / 1e9, 2500.0)}
                if window == 1:
                    # the 1x1 layers move (input + filter + output) x 2 bytes
                    # for little arithmetic: the large ones are HBM bound
                    nbytes = 2 * (n_a + n_b + n_o)
                    entry["bytes"] = nbytes
                    entry["gbs"] = round(nbytes / ms / 1e6, 1)
                    entry["frac_hbm_peak"] = frac(nbytes / ms / 1e6,
                                                  PEAK_HBM_GBS)
                h.append(entry)
                if window == 1:
                    # gradients of the 1x1 layers (same byte accounting)
                    o.copy_(uniform(n_o).half())
                    dx = torch.empty(n_a, device="cuda", dtype=torch.float16)
                    dw = torch.empty(n_b, device="cuda", dtype=torch.float16)
                    ws2 = torch.empty(2 * 256 * 128 * 256, device="cuda",
                                      dtype=torch.float16)
                    for direction, tag, bufs in (
                            (DIRECTION.INPUT_BACKPROP, "input_backprop",
                             (o, b, dx)),
                            (DIRECTION.FILTER_BACKPROP, "filter_backprop",
                             (a, o, dw))):
                        ms = event_time_ms(lambda: ops.conv2d(
                            bufs[0], bufs[1], p, direction, ALGO.MATMUL,
                            workspace=ws2, out=bufs[2]), reps=20, warm=3,
                            repeats=3)
                        h.append({"op": "conv1x1_%dx%dx%d_k%d_b128_f16_%s" % (
                            size, size, ch, feats, tag), "ms": round(ms, 4),
                            "tflops": round(fl / ms / 1e9, 1),
                            "frac_f16_mfma_peak": frac(fl / ms / 1e9, 2500.0),
                            "bytes": nbytes,
                            "gbs": round(nbytes / ms / 1e6, 1),
                            "frac_hbm_peak": frac(nbytes / ms / 1e6,
                                                  PEAK_HBM_GBS)})
                    del dx, dw, ws2
                if window == 3:
                    # input gradient: the same kernel on dY (o) with the
                    # filter's taps mirrored and its roles swapped
                    dx = torch.empty(n_a, device="cuda", dtype=torch.float16)
                    o.copy_(uniform(n_o).half())
                    ms = event_time_ms(lambda: ops.conv2d(
                        o, b, p, DIRECTION.INPUT_BACKPROP, ALGO.IM2COL,
                        workspace=ws, out=dx), reps=30, warm=5, repeats=3)
                    fl = ops.conv_flops(p, DIRECTION.INPUT_BACKPROP)
                    h.append({"op": "conv3x3_%dx%dx%d_k%d_b128_f16_input_"
                              "backprop" % (size, size, ch, feats),
                              "ms": round(ms, 4),
                              "tflops": round(fl / ms / 1e9, 1),
                              "frac_f16_mfma_peak": frac(
                                  fl / ms / 1e9, 2500.0)})
                    del dx
                    # filter gradient on the binary16 matrix instructions
                    # (partial fp32 tiles of up to 256 work-groups in the
                    # workspace)
                    dw = torch.empty(n_b, device="cuda", dtype=torch.float16)
                    ws2 = torch.empty(max(2 * n_b, 2 * 256 * 9 * 64 * 64),
                                      device="cuda", dtype=torch.float16)
                    ms = event_time_ms(lambda: ops.conv2d(
                        a, o, p, DIRECTION.FILTER_BACKPROP, ALGO.IM2COL,
                        workspace=ws2, out=dw), reps=20, warm=3, repeats=3)
                    fl = ops.conv_flops(p, DIRECTION.FORWARD)
                    h.append({"op": "conv3x3_%dx%dx%d_k%d_b128_f16_filter_"
                              "backprop" % (size, size, ch, feats),
                              "ms": round(ms, 4),
                              "tflops": round(fl / ms / 1e9, 1),
                              "frac_f16_mfma_peak": frac(
                                  fl / ms / 1e9, 2500.0)})
                    del dw, ws2
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
                "frac_hbm_peak": frac(gbs, PEAK_HBM_GBS)})
            del xs, ys
        detail["f16_batch128"] = h

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
                         "frac_hbm_peak": frac(gbs, PEAK_HBM_GBS)})
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
                # (the calls that take a stream-ordered temporary pay a fixed
                # cost after every synchronisation: long runs, so that the
                # figure is the steady state)
                ms = event_time_ms(run, reps=max(5 * sets, 100), warm=sets,
                                   repeats=3)
                grads.append(mem_entry(
                    "depthwise3x3_%dx%dx%d_s%d_%s" % (size, size, ch, stride,
                                                      tag),
                    nbytes, ms, device_ms(run, 5 * sets), with_stream=False))
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
                               device_ms(run_max_grad, 3 * sets),
                               with_stream=False))

        def run_avg_grad():
            i = state["i"] % sets
            state["i"] += 1
            ops.pooling_avg_grad(dys[i], p, dx=dxs[i])
        ms = event_time_ms(run_avg_grad, reps=3 * sets, warm=sets, repeats=3)
        grads.append(mem_entry("avgpool3x3_s2_112x112x64_grad",
                               4 * (n_in + n_out), ms,
                               device_ms(run_avg_grad, 3 * sets),
                               with_stream=False))
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
                "frac_mfma_peak": frac(tf, PEAK_FP32_MFMA_TFLOPS)})
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

        def cpu_time(fn, budget_s, max_runs=10):
            """Median wall time of fn() after one warm-up run, at most
            `max_runs` runs or `budget_s` seconds."""
            fn()
            times, spent = [], 0.0
            while len(times) < max_runs and (spent < budget_s or not times):
                t = time.perf_counter()
                fn()
                times.append(time.perf_counter() - t)
                spent += times[-1]
            times.sort()
            return times[len(times) // 2], len(times)

        # configuration 0 on the CPU: the single 56x56x64 image, tiled
        p = oracle.make_params(1, 56, 56, 64, 64, 3, 1, True)
        x = rng.uniform(-1, 1, 56 * 56 * 64).astype(np.float32)
        w = rng.uniform(-1, 1, 9 * 64 * 64).astype(np.float32)
        sec, runs = cpu_time(lambda: oracle.conv2d_tiled_forward(x, w, p), 2.0)
        cpu["config0_tflops"] = round(
            2.0 * 56 * 56 * 9 * 64 * 64 / sec / 1e12, 5)
        cpu["config0_ms"] = round(sec * 1e3, 3)
        cpu["config0_sample"] = ("median of %d runs of the tiled restatement "
                                 "on [1,56,56,64] x [3,3,64,64]" % runs)

        # depthwise and pooling in the reference's loop order
        # (src/depthwise_conv2d/kernels.h:58-125, src/pooling/kernels.h:61-99:
        # one work-item per output element, window rows then columns, fp32),
        # work-items spread over the host threads; batch 8 of each layer
        mem_cpu = []
        cb = 8
        for size, ch, stride in MOBILENET:
            p = oracle.make_params(cb, size, size, ch, 1, 3, stride, True)
            x = rng.standard_normal(cb * size * size * ch).astype(np.float32)
            w = rng.standard_normal(9 * ch).astype(np.float32)
            sec, runs = cpu_time(
                lambda: oracle.depthwise_forward(x, w, p, acc64=False), 1.0, 5)
            nbytes = 4 * (x.size + w.size + cb * p.out_rows * p.out_cols * ch)
            mem_cpu.append({"op": "depthwise3x3_%dx%dx%d_s%d" % (
                size, size, ch, stride), "batch": cb, "bytes": nbytes,
                "ms": round(sec * 1e3, 3),
                "gbs": round(nbytes / sec / 1e9, 2), "runs": runs})
        for name, args_, fn in (
                ("maxpool3x3_s2_112x112x64", (cb, 112, 112, 64, 0, 3, 2, True),
                 lambda x, p: oracle.pool_max_forward(x, p)),
                ("avgpool7x7_7x7x2048", (cb, 7, 7, 2048, 0, 7, 1, False),
                 lambda x, p: oracle.pool_avg_forward(x, p, acc64=False))):
            p = oracle.make_params(*args_)
            x = rng.standard_normal(
                cb * args_[1] * args_[2] * args_[3]).astype(np.float32)
            sec, runs = cpu_time(lambda: fn(x, p), 1.0, 5)
            nbytes = 4 * (x.size + cb * p.out_rows * p.out_cols * args_[3])
            mem_cpu.append({"op": name, "batch": cb, "bytes": nbytes,
                            "ms": round(sec * 1e3, 3),
                            "gbs": round(nbytes / sec / 1e9, 2), "runs": runs})
        cpu["memory_bound"] = mem_cpu
        cpu["memory_bound_unit"] = "GB/s"
        cpu["memory_bound_sample"] = ("batch %d of each layer, reference loop "
                                      "order, %d host threads" % (cb, cores))
        for e in mem_cpu:
            if e["op"].startswith("depthwise"):
                cpu["depthwise_" + e["op"].split("_", 1)[1] + "_gbs"] = e["gbs"]
            elif e["op"].startswith("maxpool"):
                cpu["maxpool_gbs"] = e["gbs"]
            else:
                cpu["avgpool_gbs"] = e["gbs"]
        dw = [e for e in mem_cpu if e["op"].startswith("depthwise")]
        cpu["depthwise_gbs"] = round(
            sum(e["bytes"] for e in dw) / sum(e["ms"] for e in dw) / 1e6, 2)

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
