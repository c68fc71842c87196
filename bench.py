#!/usr/bin/env python3
"""Benchmark of the DIA product path on one MI355X.

A step is one pass of the hot path over one batch: the three calls a locally
connected RBM layer makes on the 16384-unit / 49-diagonal / batch-128
configuration --
    up-pass          H  = A * V                    (prod 'n', beta 0)
    down-pass        V' = 0.5*V' + A^T * H         (prod 't', beta 0.5)
    weight gradient  G  = 0.9*G + (1/128)*proj_diag(Vg * Hg^T)   (densedense_to_dia)
launched back to back on one stream with every operand already in HBM.  The
operands rotate through enough distinct buffer sets that neither a step nor
a single operation timed alone can be served from the 256 MB Infinity Cache
(default: the sets' up-pass operands alone exceed 600 MB); `--sets 1` gives the
cache-warm figure instead.

value = algorithmic bytes of the step / step time (GB/s); the algorithmic bytes
count every operand once and only the valid diagonal slots
(cuv_amd.workloads.spmm_bytes / dd2dia_bytes).  `roofline` describes the
slowest of the three kernels, timed on its own with HIP events on the launch
stream.  `cpu_baseline` is the single-threaded CPU oracle (a restatement of the
reference's host loops) on the same step, on this machine's host cores;
`cpu_baseline_all_cores` runs the same oracle on every core this process may
use (threads over batch columns for the products, over diagonals for the
gradient) -- the reference itself has no threaded host path.

Every timed leg is preceded by `settle_ms` of untimed replays of the very
launches it times (clocks and caches in their steady state), so that a run of
a few steps reads what a long one reads.  `clocks` holds the shader and memory
clocks read (rocm-smi) while the step's graph is running.

Prints one JSON line on stdout.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published

# HBM bytes per launch (fetch + write-back) come from profiles/hbm_traffic.json: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE readings, each scaled by what the same counter read for a 256 MiB device copy in the same run, together
# with the revision of the tree that was profiled (commands and readings: profiles/hbm_traffic_cfg1_cfg2_cfg3.md).
def load_traffic():
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            t = json.load(f)
        return {k: int(t["bytes_per_launch"][k]) for k in ("up_pass", "down_pass", "weight_gradient")}, t.get("git_rev")
    except (OSError, KeyError, ValueError):
        return {"up_pass": None, "down_pass": None, "weight_gradient": None}, None


FP32_VALU_PEAK_TFLOPS = 157.3  # published vector fp32; the kernels use no MFMA
# The rate of v_fmac_f32 with a DPP-broadcast or scalar operand, one wave64 instruction per SIMD per 4 clocks:
# 256 CUs x 4 SIMDs x 16 lanes x 2 FLOP x 2.4 GHz (measured on the box: 75.7 TFLOP/s).  The products keep the
# batch along the lanes and broadcast the diagonal's value that way, so this is the ceiling of their arithmetic;
# only the form with three vector-register operands runs at twice that (124-137 TFLOP/s measured).
FP32_VALU_BROADCAST_TFLOPS = 78.6


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 3000 steps are 0.1 s of GPU time: runs of a few hundred steps read about 2 % slower
    ap.add_argument("--steps", type=int, default=3000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--sets", type=int, default=0,
                    help="distinct operand sets rotated through (0: enough for > 512 MB)")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch from a Python loop instead of replaying HIP graphs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy three times (known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--workload", default="step",
                    help="'step' (default): cfg1 + cfg2 + cfg3, the configuration the metric is quoted on; "
                         "'cfg4': the large layer (262144 rows, 676 diagonals, batch 256), each product timed "
                         "on its own -- an auxiliary line, no CPU leg (the oracle needs minutes for it); "
                         "'scale': the headline layer's pattern at growing map and batch sizes, an auxiliary line; "
                         "'layer': the steps either side of the products at cfg1's shape (fused bias + sigmoid "
                         "(+ sample) against separate passes, the weight-decay step) -- an auxiliary line")
    ap.add_argument("--legs", default="all", choices=["all", "rotating"],
                    help="'rotating': only the legs that stream from HBM (no cache-warm legs, no large-layer record), "
                         "so that a profiler's per-kernel averages describe the same launches as the headline figures")
    ap.add_argument("--settle-ms", type=float, default=200.0,
                    help="untimed replays of a leg's own launches before it is timed, in ms of GPU time")
    ap.add_argument("--no-clocks", action="store_true",
                    help="do not start rocm-smi to read the clocks (for runs under a profiler)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-check", action="store_true", help="skip the parity check of the timed buffers")
    return ap.parse_args()


def measure_cfg4(steps, torch, D, W, dev, with_aux=True):
    """The large layer: 256x256 map, 4 channels, 13x13 window per channel pair (676 diagonals), batch 256,
    inputs drawn on the device.  The working set (about 1.8 GB) is far beyond every cache, so no buffer
    rotation is needed.  Parity at this size is covered by tests/test_gpu_parity.py.  Returns (config, per-product
    results, auxiliary results)."""
    p = W.pattern_large(256, 4, 13)
    n, nd, batch = p.h, len(p.offsets), 256
    g = torch.Generator(device=dev)
    g.manual_seed(0xC0FFEE + 4)
    nnz = p.nnz

    def dia():
        m = D.dev_dia_matrix_f(n, n, nd, n, 1, device=dev)
        m.set_offsets(p.offsets)
        m.vec.copy_(torch.randn(nd * n, generator=g, device=dev) * 0.01)
        return m
    A, G = dia(), dia()
    X = torch.rand(batch, n, generator=g, device=dev)
    H = torch.rand(batch, n, generator=g, device=dev)
    Y = torch.empty(batch, n, device=dev)
    bd = D.dev_block_descriptor_f(G)
    A.desc
    ops = {
        "forward": (lambda: D.prod(Y, A, X, "n", "n", 1.0, 0.0, sync=False), W.spmm_bytes(p, batch, "n", 0.0)),
        "transposed": (lambda: D.prod(Y, A, H, "t", "n", 1.0, 0.0, sync=False), W.spmm_bytes(p, batch, "t", 0.0)),
        "weight_gradient": (lambda: D.densedense_to_dia(G, bd, X, H, 1.0 / batch, 0.0, sync=False),
                            W.dd2dia_bytes(p, batch, 0.0)),
    }
    avg = torch.empty(nd, device=dev)
    aux_ops = {"avg_diagonals": (lambda: D.avg_diagonals(avg, A, sync=False), 4 * nnz + 8 * nd)} if with_aux else {}
    flops = 2 * nnz * batch
    stream = torch.cuda.current_stream()

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps
    # The first operation timed after the operands are drawn read 3 - 4 % slower than the same operation timed again
    # later (whichever operation it was), and still 2 % slower with 12 untimed launches before it: 40 launches
    # (about 50 ms) go first.
    for _ in range(40):
        ops["forward"][0]()
    torch.cuda.synchronize()
    res = {}
    from cuv_amd import _lib
    for name, (fn, nbytes) in ops.items():
        ms = timed(fn)
        tf = flops / (ms * 1e-3) / 1e12
        res[name] = dict(ms=ms, kernel=_lib.lib().cuvdia_last_kernel().decode(), bytes=nbytes, flops=flops,
                         gbs=nbytes / (ms * 1e-3) / 1e9,
                         frac_hbm=nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, tflops=tf,
                         frac_fp32_valu=tf / FP32_VALU_PEAK_TFLOPS, frac_fp32_valu_broadcast=tf / FP32_VALU_BROADCAST_TFLOPS)
    aux = {}
    for name, (fn, nbytes) in aux_ops.items():
        ms = timed(fn)
        aux[name] = dict(ms=ms, bytes=nbytes, gbs=nbytes / (ms * 1e-3) / 1e9,
                         frac_hbm=nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
    config = dict(workload="cfg4: 262144x262144 DIA, 676 diagonals (4 channels x 13x13 window on a 256x256 map), "
                           "batch 256; forward, transposed and gradient products each timed alone",
                  rows=n, diagonals=nd, batch=batch, nnz=nnz)
    del A, G, X, H, Y, bd, avg
    torch.cuda.empty_cache()
    return config, res, aux


def bench_cfg4(args, torch, D, W, dev):
    steps = min(args.steps, 50)
    config, res, aux = measure_cfg4(steps, torch, D, W, dev)
    tot_ms = sum(r["ms"] for r in res.values())
    tot_bytes = sum(r["bytes"] for r in res.values())
    print(json.dumps(dict(
        metric="achieved HBM GB/s, DIA SpMM (both transposes) + densedense_to_dia, large layer", unit="GB/s",
        value=tot_bytes / (tot_ms * 1e-3) / 1e9, n_gpus=1, steps=steps, warmup=3, ms_per_step=tot_ms,
        higher_is_better=True, scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
        config=config, ops=res, aux=aux,
        note="bound by the fp32 vector rate (57 FLOP per algorithmic byte), not by HBM")))


def bench_scale(args, torch, D, W, dev):
    """The layer of the headline configuration (7x7 window, one channel, 49 diagonals) at growing map and
    batch sizes: shows what the same kernels reach once a launch holds many rounds of workgroups and its fixed
    costs (launch, first loads, final stores) no longer weigh.  Inputs are drawn on the device; from the second case
    on the operands of a call exceed the 256 MB Infinity Cache, so every launch streams from HBM."""
    cases = [(128, 128), (128, 512), (128, 2048), (128, 4096), (256, 1024), (512, 128), (512, 512), (1024, 128)]
    out = measure_scale(cases, torch, D, W, dev)
    best = max(r[k]["gbs"] for r in out for k in ("up_pass", "down_pass", "weight_gradient"))
    print(json.dumps(dict(
        metric="achieved HBM GB/s, DIA SpMM (both transposes) + densedense_to_dia, size sweep", unit="GB/s",
        value=best, n_gpus=1, steps=None, warmup=3, higher_is_better=True, scaling="weak", vs_baseline=None,
        dtype="f32", data="synthetic",
        config=dict(workload="7x7 window on a px x px map (49 diagonals), batch b, for several (px, b); "
                             "each product timed alone; value = the best single figure of the sweep"),
        cases=out)))


def measure_scale(cases, torch, D, W, dev):
    """One row per (map width, batch): each product timed alone from a HIP graph of ten launches, with the name of
    the kernel that served it."""
    from cuv_amd import _lib
    L = _lib.lib()
    g = torch.Generator(device=dev)
    g.manual_seed(0xC0FFEE + 5)
    out = []
    for px, batch in cases:
        n = px * px
        p = W.Pattern(n, n, W.window_offsets(px, 7), n)
        nd = p.nd

        def dia():
            m = D.dev_dia_matrix_f(n, n, nd, n, 1, device=dev)
            m.set_offsets(p.offsets)
            m.vec.copy_(torch.randn(nd * n, generator=g, device=dev) * 0.01)
            return m
        A, G = dia(), dia()
        X = torch.rand(batch, n, generator=g, device=dev)
        H = torch.rand(batch, n, generator=g, device=dev)
        Y = torch.rand(batch, n, generator=g, device=dev)
        bd = D.dev_block_descriptor_f(G)
        A.desc
        bias = torch.randn(n, generator=g, device=dev)
        ops = {
            "up_pass": (lambda: D.prod(Y, A, X, "n", "n", 1.0, 0.0, sync=False), W.spmm_bytes(p, batch, "n", 0.0)),
            "down_pass": (lambda: D.prod(Y, A, H, "t", "n", 1.0, 0.5, sync=False), W.spmm_bytes(p, batch, "t", 0.5)),
            "weight_gradient": (lambda: D.densedense_to_dia(G, bd, X, H, 1.0 / batch, 0.9, sync=False),
                                W.dd2dia_bytes(p, batch, 0.9)),
            # the fused layer updates: h = sample(sigmoid(A v + b)), v' = sigmoid(A^T h + b)
            "layer_up_sampled": (lambda: D.prod_bias_act(Y, A, X, "n", 1.0, 0.0, bias, _lib.ACT_SIGMOID_SAMPLE, 7, sync=False),
                                 W.spmm_bytes(p, batch, "n", 0.0) + 4 * n),
            "layer_down_sigmoid": (lambda: D.prod_bias_act(Y, A, H, "t", 1.0, 0.0, bias, _lib.ACT_SIGMOID, sync=False),
                                   W.spmm_bytes(p, batch, "t", 0.0) + 4 * n),
        }
        flops = W.flops(p, batch)
        row = dict(map=px, rows=n, batch=batch, flops=flops)
        for name, (fn, nbytes) in ops.items():
            # ten launches per graph replay: Python cannot issue launches every few microseconds
            for _ in range(3):
                fn()
            kernel = L.cuvdia_last_kernel().decode()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(10):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            reps = max(2, min(20, int(2e4 / max(1.0, nbytes / 2e6))))
            s = torch.cuda.current_stream()
            # about 30 ms of untimed replays first: an operation timed right after its operands were drawn reads a
            # few per cent slow
            w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            w0.record(s)
            graph.replay()
            w1.record(s)
            torch.cuda.synchronize()
            for _ in range(max(1, min(200, int(30.0 / max(1e-3, w0.elapsed_time(w1)))))):
                graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(s)
            for _ in range(reps):
                graph.replay()
            e1.record(s)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / (10 * reps) * 1e3
            row[name] = dict(us=us, bytes=nbytes, gbs=nbytes / us / 1e3, frac_hbm=nbytes / us / 1e3 / HBM_PEAK_GBS,
                             tflops=flops / us / 1e6, kernel=kernel)
            del graph
        out.append(row)
        del A, G, X, H, Y, bd, bias
        torch.cuda.empty_cache()
    return out


def bench_layer(args, torch, D, W, dev):
    """What the fused layer update saves at cfg1's shape: the up-pass alone, with bias + sigmoid (+ Bernoulli
    sample) in its store, and as the reference's separate passes over the activations (here torch's
    element-wise kernels); and the weight-decay step on the value vector.  Warm timings from HIP graphs of 20
    launches; parity of these operations is covered by tests/test_gpu_parity.py."""
    from cuv_amd import _lib
    w1 = W.cfg1()
    p = w1.pattern
    n, nd, batch = p.h, len(p.offsets), w1.batch
    A = D.dev_dia_matrix_f(p.h, p.w, nd, p.stride, 1, device=dev)
    A.set_offsets(p.offsets)
    A.push(w1.vals)
    G = D.dev_dia_matrix_f(p.h, p.w, nd, p.stride, 1, device=dev)
    G.set_offsets(p.offsets)
    G.push(w1.vals)
    V = D.to_device_colmajor(w1.X)
    H = torch.empty(batch, n, device=dev)
    bias = torch.randn(n, device=dev)
    A.desc

    def timed(fn, n_rep=300):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(20):
                fn()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n_rep // 20):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (n_rep // 20 * 20) * 1e3

    def separate(sample):
        D.prod(H, A, V, "n", "n", 1.0, 0.0, sync=False)
        H.add_(bias)
        torch.sigmoid_(H)
        if sample:
            H.copy_(torch.bernoulli(H))
    step_bytes = 3 * 4 * nd * p.stride
    us = {
        "prod": timed(lambda: D.prod(H, A, V, "n", "n", 1.0, 0.0, sync=False)),
        "prod_bias_sigmoid_fused": timed(lambda: D.prod_bias_act(H, A, V, "n", 1.0, 0.0, bias, _lib.ACT_SIGMOID,
                                                                 sync=False)),
        "prod_bias_sigmoid_sample_fused": timed(lambda: D.prod_bias_act(H, A, V, "n", 1.0, 0.0, bias,
                                                                        _lib.ACT_SIGMOID_SAMPLE, seed=1, sync=False)),
        "prod_then_bias_then_sigmoid": timed(lambda: separate(False)),
        "prod_then_bias_then_sigmoid_then_sample": timed(lambda: separate(True)),
        "learn_step_weight_decay": timed(lambda: D.learn_step_weight_decay(A, G, 0.01, 0.001, sync=False)),
    }
    lw = us["learn_step_weight_decay"]
    print(json.dumps(dict(
        metric="microseconds per launch, layer-update steps around the DIA products", unit="us",
        value=us["prod_bias_sigmoid_fused"], n_gpus=1, steps=300, warmup=20, ms_per_step=us["prod_bias_sigmoid_fused"] * 1e-3,
        higher_is_better=False, scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
        config=dict(workload="cfg1 shape (16384x16384 DIA, 49 diagonals, batch 128): up-pass with its bias, "
                             "sigmoid and sampling fused or as separate passes; weight-decay step on the value vector",
                    rows=n, diagonals=nd, batch=batch),
        us=us, learn_step=dict(bytes=step_bytes, gbs=step_bytes / (lw * 1e-6) / 1e9,
                               frac_hbm=step_bytes / (lw * 1e-6) / 1e9 / HBM_PEAK_GBS,
                               note="warm: the 6.4 MB working set stays in cache between launches"))))


def read_clocks(torch, enqueue, eager):
    """Shader and memory clock while the step runs: about a second of the step's launches is enqueued, rocm-smi is
    asked (a child process) while the GPU works through them, then the queue is drained.  None where rocm-smi is
    not there or does not answer."""
    import re
    import shutil
    import subprocess
    exe = shutil.which("rocm-smi") or "/opt/rocm/bin/rocm-smi"
    if not os.path.exists(exe):
        return None
    try:
        if eager:
            enqueue()
            graph = None
        else:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                enqueue()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            for _ in range(max(1, min(20000, int(1500.0 / max(1e-3, e0.elapsed_time(e1)))))):
                graph.replay()
        txt = subprocess.run([exe, "--showclocks", "-d", "0"], capture_output=True, text=True, timeout=20).stdout
        busy = not torch.cuda.current_stream().query()
        torch.cuda.synchronize()
        found = {}
        for line in txt.splitlines():
            m = re.search(r"\b(sclk|mclk|fclk|socclk) clock level:?\s*\S*\s*\((\d+)\s*Mhz\)", line, re.I)
            if m:
                found[m.group(1).lower() + "_mhz"] = int(m.group(2))
        if not found:
            return None
        found["source"] = "rocm-smi --showclocks, read after the timed legs while a graph of the step's launches was replaying"
        found["gpu_busy_when_read"] = bool(busy)
        return found
    except Exception as e:           # the clocks are a note beside the figures, never a reason to fail the run
        return dict(error=str(e)[:200])


def cpu_all_cores(O, np, p, w1, w2, w3, step_bytes, step_flops, one_core_s):
    """The oracle's step on every core this process may use (at most 16, the share of one GPU's host): the two
    products split over the batch columns, the gradient over the diagonals (its sum runs over the batch, so
    a split over columns would need a reduction the reference does not have), one thread per share -- the
    library calls release the interpreter lock.  The reference's host path is single-threaded
    (spmv.cu:145-220, densedense_to_sparse.cu:204-252): this leg says what the same loops give when all cores
    run them, not what the reference does."""
    from concurrent.futures import ThreadPoolExecutor
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    cores = max(1, min(16, cores))
    od = O.Dia(p.h, p.w, p.offsets, p.stride, 1, w1.vals)
    batch = w1.X.shape[1]
    col_cuts = [batch * k // cores for k in range(cores + 1)]
    col_shares = [(a, b) for a, b in zip(col_cuts[:-1], col_cuts[1:]) if b > a]
    dia_cuts = [p.nd * k // cores for k in range(cores + 1)]
    dia_shares = [(a, b) for a, b in zip(dia_cuts[:-1], dia_cuts[1:]) if b > a]
    subs = []
    for a, b in dia_shares:
        subs.append(O.Dia(p.h, p.w, p.offsets[a:b], p.stride, 1, w3.vals[a * p.stride:b * p.stride].copy()))
    Xs = [np.asfortranarray(w1.X[:, a:b]) for a, b in col_shares]
    Hs = [np.asfortranarray(w2.X[:, a:b]) for a, b in col_shares]
    Ds = [np.asfortranarray(w2.dst[:, a:b]) for a, b in col_shares]

    def run(pool):
        list(pool.map(lambda x: O.prod(od, x), Xs))
        list(pool.map(lambda hd: O.prod(od, hd[0], hd[1], "t", 1.0, 0.5), zip(Hs, Ds)))
        list(pool.map(lambda d: O.dd2dia(d, w3.A, w3.B, w3.alpha, w3.beta), subs))
    reps = []
    with ThreadPoolExecutor(max_workers=cores) as pool:
        run(pool)
        for _ in range(5):
            t = time.perf_counter()
            run(pool)
            reps.append(time.perf_counter() - t)
    med = statistics.median(reps)
    return dict(value=step_bytes / med / 1e9, unit="GB/s", cores=cores, kind="port",
                sample="the full step (cfg1+cfg2+cfg3), median of 5 repetitions; products split over batch columns, "
                       "gradient over diagonals, one thread per core",
                ms_per_step=med * 1e3, gflops=step_flops / med / 1e9, speedup_over_one_core=one_core_s / med,
                note="an extrapolation of the reference's host path, which is single-threaded: what its loops reach "
                     "when every core runs a share")


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path uses no collectives and every "
              "configuration fits one MI355X; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from cuv_amd import _lib, dia as D, workloads as W

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the product path)", file=sys.stderr)
        sys.exit(2)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    L = _lib.lib()

    if args.workload == "cfg4":
        return bench_cfg4(args, torch, D, W, dev)
    if args.workload == "scale":
        return bench_scale(args, torch, D, W, dev)
    if args.workload == "layer":
        return bench_layer(args, torch, D, W, dev)

    w1, w2, w3 = W.cfg1(), W.cfg2(), W.cfg3()
    p = w1.pattern
    batch = w1.batch
    step_bytes = w1.bytes + w2.bytes + w3.bytes
    step_flops = w1.flops + w2.flops + w3.flops

    # One set = every buffer a step touches.  The sets rotate so that every launch streams from HBM: their number
    # is chosen for the operation that touches the least of a set (the up-pass: A, V, H) -- timed alone, each
    # operation still walks through more than 600 MB, well past the 256 MB Infinity Cache, before it meets a
    # buffer again.  (Sized for the whole step only, 13 sets, the single-operation legs re-used their 20 - 28 MB
    # per set within 260 - 370 MB and read about 1 us per launch faster than the same launch inside the step.)
    set_bytes = 4 * (2 * p.nd * p.stride + 5 * p.h * batch)
    least_bytes = 4 * (p.nd * p.stride + 2 * p.h * batch)
    nsets = args.sets if args.sets > 0 else max(2, -(-600_000_000 // least_bytes))

    def dia_from(vals):
        m = D.dev_dia_matrix_f(p.h, p.w, p.nd, p.stride, 1, device=dev)
        m.set_offsets(p.offsets)
        m.push(vals)
        return m

    sets = []
    for _ in range(nsets):
        sets.append(dict(
            A=dia_from(w1.vals), V=D.to_device_colmajor(w1.X, dev),
            H=torch.empty(batch, p.h, device=dev),
            Hs=D.to_device_colmajor(w2.X, dev), Vp=D.to_device_colmajor(w2.dst, dev),
            G=dia_from(w3.vals), Ga=D.to_device_colmajor(w3.A, dev), Gb=D.to_device_colmajor(w3.B, dev)))
    for s in sets:
        s["A"].desc, s["G"].desc                      # build descriptors outside the timed region
        s["bd"] = D.dev_block_descriptor_f(s["G"])

    def up(s):
        D.prod(s["H"], s["A"], s["V"], "n", "n", w1.alpha, w1.beta, sync=False)

    def down(s):
        D.prod(s["Vp"], s["A"], s["Hs"], "t", "n", w2.alpha, w2.beta, sync=False)

    def grad(s):
        D.densedense_to_dia(s["G"], s["bd"], s["Ga"], s["Gb"], w3.alpha, w3.beta, sync=False)

    def step(i):
        s = sets[i % nsets]
        up(s); down(s); grad(s)

    # ---- parity of exactly these buffers, before they are mutated by repetition
    checked = None
    if not args.no_check:
        from oracle import oracle as O
        s = sets[0]
        step(0)
        torch.cuda.synchronize()
        od = O.Dia(p.h, p.w, p.offsets, p.stride, 1, w1.vals)

        def worst(got, ref, mag):
            return float((np.abs(got.astype(np.float64) - ref) / np.maximum(mag, 1e-30)).max())

        def worst_rel(got, ref):
            """max |gpu - ref| / |ref| over the elements with |ref| >= 1e-2 * max|ref|"""
            ref = np.asarray(ref, np.float64)
            big = np.abs(ref) >= 1e-2 * np.abs(ref).max()
            return float((np.abs(got.astype(np.float64)[big] - ref[big]) / np.abs(ref[big])).max())
        h_got, h_ref = D.to_host_colmajor(s["H"]), O.prod(od, w1.X)
        e1 = worst(h_got, h_ref, O.prod_mag(od, w1.X))
        v_got, v_ref = D.to_host_colmajor(s["Vp"]), O.prod(od, w2.X, w2.dst, "t", 1.0, 0.5)
        e2 = worst(v_got, v_ref, O.prod_mag(od, w2.X, w2.dst, "t", 1.0, 0.5))
        valid = O.valid_mask(od)
        ref3 = O.dd2dia(od, w3.A, w3.B, w3.alpha, w3.beta)
        mag3 = O.dd2dia_f64(O.Dia(p.h, p.w, p.offsets, p.stride, 1, np.abs(w3.vals)), w3.A, w3.B,
                            w3.alpha, w3.beta)
        g_got = s["G"].pull()[valid]
        e3 = worst(g_got, ref3[valid], mag3[valid])
        checked = dict(tolerance=1e-5, criterion="|gpu - oracle| <= tolerance * sum|terms| per element",
                       up_pass=e1, down_pass=e2, weight_gradient=e3,
                       rel_err_where_ref_not_small=dict(
                           note="max |gpu - oracle| / |oracle| over elements with |oracle| >= 1e-2 * max|oracle|",
                           up_pass=worst_rel(h_got, h_ref), down_pass=worst_rel(v_got, v_ref),
                           weight_gradient=worst_rel(g_got, ref3[valid])),
                       ok=bool(max(e1, e2, e3) <= 1e-5))
        if not checked["ok"]:
            print("PARITY FAILURE: %r" % checked, file=sys.stderr)
            sys.exit(1)
        # restore the mutated buffers of set 0
        s["Vp"].copy_(D.to_device_colmajor(w2.dst, dev)); s["G"].push(w3.vals)

    stream = torch.cuda.current_stream()

    if args.calibrate_copy:
        src = torch.zeros(64 * 1024 * 1024, dtype=torch.float32, device=dev)     # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # The kernels run for a few microseconds; a Python launch loop cannot feed
    # them that fast.  Launches are therefore captured into HIP graphs (one
    # graph = one rotation through the buffer sets) and the graphs replayed.
    def capture(fn, count):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(count):
                fn(i)
        return g

    settled = []

    def settle(fn, plan, n):
        """Untimed: the launches about to be timed, replayed for args.settle_ms of GPU time (measured on one
        replay first), so that the timed region starts with clocks, caches and the graph itself in the state
        a long run reaches."""
        if args.settle_ms <= 0:
            return
        w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def once():
            if plan is None:
                for i in range(min(n, nsets)):
                    fn(i)
            else:
                (plan[0] or plan[2]).replay()
        torch.cuda.synchronize()
        w0.record(stream)
        once()
        w1.record(stream)
        torch.cuda.synchronize()
        one_ms = max(1e-3, w0.elapsed_time(w1))
        last_replay_ms[0] = one_ms
        reps = max(1, min(100000, int(args.settle_ms / one_ms)))
        w0.record(stream)
        for _ in range(reps):
            once()
        w1.record(stream)
        torch.cuda.synchronize()
        settled.append(w0.elapsed_time(w1))

    last_replay_ms = [1.0]

    def gate_reps(plan):
        return max(2, min(2000, int(10.0 / max(1e-3, last_replay_ms[0])) + 1))

    def timed(fn, n):
        """Exactly n calls fn(0..n-1) (fn must depend on i only through i % nsets)
        between two HIP events on the launch stream; returns ms per call."""
        if args.no_graph:
            plan = None
        else:
            full, rest = divmod(n, nsets)
            gfull = capture(fn, nsets) if full else None
            grest = capture(fn, rest) if rest else None
            for g in (gfull, grest):                      # untimed first launch of each graph
                if g is not None:
                    g.replay()
            plan = (gfull, full, grest)
        settle(fn, plan, n)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        if plan is not None:
            # About 10 ms of the same replays go first, untimed, and are still running while the host enqueues the
            # first event, the timed replays and the second event: the GPU then takes the timed region from its
            # queue in the state a long run is in, and the time the host needs to submit a graph (hundreds of
            # microseconds right after a burst of replays) is not read as kernel time -- which matters when the
            # whole region is one replay of 20 steps.
            for _ in range(gate_reps(plan)):
                (plan[0] or plan[2]).replay()
        e0.record(stream)
        if plan is None:
            for i in range(n):
                fn(i)
        else:
            gfull, full, grest = plan
            for _ in range(full):
                gfull.replay()
            if grest is not None:
                grest.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    # which kernel serves each operation: asked of the library, call by call
    kernel_names, kernel_paths = {}, {}
    for name, fn in (("up_pass", up), ("down_pass", down), ("weight_gradient", grad)):
        fn(sets[0])
        kernel_names[name] = L.cuvdia_last_kernel().decode()
        kernel_paths[name] = L.cuvdia_last_path()
    torch.cuda.synchronize()
    if not kernel_names["up_pass"].startswith("spmm_") or not kernel_names["weight_gradient"].startswith("dd2dia_"):
        print("unexpected kernels: %r" % kernel_names, file=sys.stderr)
        sys.exit(1)
    t0 = time.perf_counter()
    ms_step = timed(step, args.steps)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # graph replays must reproduce the eager result: the up-pass is idempotent,
    # so after all those replays H of set 0 must equal a fresh eager H bit for bit
    if not args.no_graph:
        h_graph = sets[0]["H"].clone()
        sets[0]["H"].fill_(float("nan"))
        up(sets[0])
        torch.cuda.synchronize()
        if not torch.equal(h_graph, sets[0]["H"]):
            print("GRAPH REPLAY MISMATCH against the eager launch", file=sys.stderr)
            sys.exit(1)

    # per-kernel figures: each operation alone, same rotation, same stream
    per = {}
    for name, fn, wl in (("up_pass", up, w1), ("down_pass", down, w2), ("weight_gradient", grad, w3)):
        ms = timed(lambda i, fn=fn: fn(sets[i % nsets]), args.steps)
        per[name] = dict(us=ms * 1e3, bytes=wl.bytes, flops=wl.flops,
                         gbs=wl.bytes / (ms * 1e-3) / 1e9, gflops=wl.flops / (ms * 1e-3) / 1e9,
                         frac_hbm=wl.bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS)
    # The dominant kernel's two launches of a step as they follow each other in the step (up-pass, then down-pass,
    # set after set), reported beside the roofline entry (which is computed from the legs above).  Timed alone,
    # each product reads about 0.4 us longer per launch than here (a run of identical launches all read, then
    # all write, at the same moments); a profiler's per-kernel average over the run lies between the two.
    def up_down(i):
        s_ = sets[i % nsets]
        up(s_); down(s_)
    pair_us = timed(up_down, args.steps) * 1e3
    # cache-warm variant (one buffer set) for reference
    warm = {}
    if args.legs == "all":
        for name, fn in (("up_pass", up), ("down_pass", down), ("weight_gradient", grad)):
            ms = timed(lambda i, fn=fn: fn(sets[0]), args.steps)
            warm[name] = ms * 1e3
    # The dominant kernel is the tiled SpMM: it runs twice per step (up-pass and
    # down-pass).  Its roofline entry is per launch, averaged over the two --
    # algorithmic bytes of the two products / their two durations -- which is
    # also what a profiler's per-kernel average duration corresponds to.
    # (the same launches once more, after every timed leg: the choice of kernel must not have changed)
    for name, fn in (("up_pass", up), ("down_pass", down), ("weight_gradient", grad)):
        fn(sets[0])
        if L.cuvdia_last_kernel().decode() != kernel_names[name] or L.cuvdia_last_path() != kernel_paths[name]:
            print("kernel choice changed during the run: %s" % name, file=sys.stderr)
            sys.exit(1)
    torch.cuda.synchronize()
    traffic, traffic_rev = load_traffic()
    for name in per:
        per[name]["kernel"] = kernel_names[name]
        per[name]["traffic"] = traffic[name]
        # what the two ceilings allow: the algorithmic bytes at the HBM peak, and the FLOPs at the rate of
        # broadcast-operand FMAs (the products' form; the projection's plain FMAs could run at twice that)
        per[name]["hbm_floor_us"] = per[name]["bytes"] / (HBM_PEAK_GBS * 1e9) * 1e6
        per[name]["valu_floor_us"] = per[name]["flops"] / (FP32_VALU_BROADCAST_TFLOPS * 1e12) * 1e6
    sp_us = (per["up_pass"]["us"] + per["down_pass"]["us"]) / 2          # the same legs as ops[]
    sp_bytes = (per["up_pass"]["bytes"] + per["down_pass"]["bytes"]) / 2
    sp_flops = (per["up_pass"]["flops"] + per["down_pass"]["flops"]) / 2
    if kernel_names["up_pass"] != kernel_names["down_pass"]:
        print("the two products ran different kernels (%r): the roofline entry assumes one" % kernel_names, file=sys.stderr)
        sys.exit(1)
    if 2 * sp_us >= per["weight_gradient"]["us"]:
        gbs = sp_bytes / (sp_us * 1e-6) / 1e9
        sp_traffic = None
        if traffic["up_pass"] is not None and traffic["down_pass"] is not None:
            sp_traffic = (traffic["up_pass"] + traffic["down_pass"]) // 2
        roofline = dict(bound="hbm", achieved=gbs, peak=HBM_PEAK_GBS, unit="GB/s", frac=gbs / HBM_PEAK_GBS,
                        traffic=sp_traffic, traffic_rev=traffic_rev,
                        kernel=kernel_names["up_pass"],
                        op="up_pass+down_pass (mean per launch of ops.up_pass.us and ops.down_pass.us, each timed alone)",
                        launches_per_step=2, us_per_launch=sp_us, us_per_launch_in_step_order=pair_us / 2,
                        algorithmic_bytes=sp_bytes,
                        hbm_floor_us=sp_bytes / (HBM_PEAK_GBS * 1e9) * 1e6,
                        valu_floor_us=sp_flops / (FP32_VALU_BROADCAST_TFLOPS * 1e12) * 1e6,
                        note="by intensity (7-10 FLOP/B) the kernel sits on the ridge of the rate its broadcast-operand "
                             "FMAs issue at (78.6 TFLOP/s / 8 TB/s = 9.8 FLOP/B): both floors are given")
    else:
        g = per["weight_gradient"]
        roofline = dict(bound="hbm", achieved=g["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=g["gbs"] / HBM_PEAK_GBS,
                        traffic=traffic["weight_gradient"], traffic_rev=traffic_rev,
                        kernel=kernel_names["weight_gradient"],
                        op="weight_gradient", launches_per_step=1, us_per_launch=g["us"],
                        algorithmic_bytes=g["bytes"], hbm_floor_us=g["hbm_floor_us"], valu_floor_us=g["valu_floor_us"])

    out = dict(
        metric="achieved HBM GB/s, DIA SpMM (both transposes) + densedense_to_dia step",
        value=step_bytes / (ms_step * 1e-3) / 1e9, unit="GB/s",
        n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=ms_step,
        higher_is_better=True, scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
        config=dict(workload="cfg1+cfg2+cfg3: 16384x16384 DIA, 49 diagonals (7x7 window on a 128x128 map), "
                             "batch 128; up-pass A*V, down-pass 0.5*V'+A^T*H, gradient 0.9*G+(1/128)*proj(Vg*Hg^T)",
                    rows=p.h, diagonals=p.nd, batch=batch, buffer_sets=nsets,
                    rotation="every operation, timed alone or inside the step, meets a buffer again only after "
                             "more than 600 MB of its own traffic",
                    step_bytes=step_bytes, step_flops=step_flops),
        frac_of_hbm_peak=step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        gflops=step_flops / (ms_step * 1e-3) / 1e9,
        wall_ms_per_step_incl_capture=wall_ms, launch="eager" if args.no_graph else "hip_graph",
        settle_ms=dict(requested_per_leg=args.settle_ms, spent_per_leg=[round(x, 1) for x in settled],
                       note="untimed replays of each leg's own launches before it is timed"),
        clocks=None, ops=per, warm_us=warm, parity=checked, roofline=roofline)

    if args.legs == "all":
        # the large layer (cfg4) beside the headline figures: an auxiliary record, no part of `value`
        keep = sets[0]
        del sets, s
        torch.cuda.empty_cache()
        cfg4_config, cfg4_res, _ = measure_cfg4(20, torch, D, W, dev, with_aux=False)
        out["aux"] = dict(cfg4=dict(config=cfg4_config, ops=cfg4_res,
                                    note="bound by the fp32 vector rate (57 FLOP per algorithmic byte): "
                                         "frac_fp32_valu is against the published 157.3 TFLOP/s, "
                                         "frac_fp32_valu_broadcast against the 78.6 TFLOP/s of FMAs with a "
                                         "DPP-broadcast or scalar operand, the form these kernels use"),
                          scale=dict(config="the headline layer's pattern (7x7 window, 49 diagonals) on a px x px map at "
                                            "batch b: each product timed alone, and the fused layer updates h = sample(sigmoid(A v + b)), v' = sigmoid(A^T h + b) (full sweep: --workload scale)",
                                     cases=measure_scale([(128, 2048), (512, 128), (512, 512)], torch, D, W, dev)))

    else:
        keep = sets[0]
    # last of the GPU work (a query of the management interface is followed by slower launches for a while)
    if not args.no_clocks:
        out["clocks"] = read_clocks(torch, lambda: [(up(keep), down(keep), grad(keep)) for _ in range(30)], args.no_graph)

    if not args.no_cpu:
        from oracle import oracle as O
        od = O.Dia(p.h, p.w, p.offsets, p.stride, 1, w1.vals)
        reps = []
        for _ in range(5):
            t = time.perf_counter()
            O.prod(od, w1.X)
            O.prod(od, w2.X, w2.dst, "t", 1.0, 0.5)
            O.dd2dia(od, w3.A, w3.B, w3.alpha, w3.beta)
            reps.append(time.perf_counter() - t)
        med = statistics.median(reps)
        out["cpu_baseline"] = dict(value=step_bytes / med / 1e9, unit="GB/s", cores=1, kind="port",
                                   sample="the full step (cfg1+cfg2+cfg3), median of 5 repetitions",
                                   ms_per_step=med * 1e3, gflops=step_flops / med / 1e9)
        out["cpu_baseline_all_cores"] = cpu_all_cores(O, np, p, w1, w2, w3, step_bytes, step_flops, med)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
