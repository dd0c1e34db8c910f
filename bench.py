#!/usr/bin/env python3
"""Benchmark of the weight-only quantized linear path on one MI355X.

One step = one pass of the four Llama-2-7B-shaped decode linears at batch M=1
(int4 codes packed 8 per uint32 along K, group 32, fp16 scales, zero point 7):
4096->12288 (fused QKV), 4096->4096 (o_proj), 4096->22016 (gate/up), 11008->4096 (down),
issued as ONE launch of the list kernel (wq_q4g32_gemv_list_run).
Inputs are synthetic and resident in HBM before the timed region.  Each step
reads a different copy of the weights (a ring of copies larger than the
256 MB last-level cache), so the reported GB/s is HBM traffic, not cache hits.

Timing protocol (after src/runtime/profiling.cc:862-933 of the reference): untimed warm-up, then
`--samples` (5) samples, each a whole number of repetitions that lasts at least `--min-sample-ms`
(100 ms), HIP events on the launch stream; the median is reported, min and max beside it.

Prints ONE JSON line.  `value` is algorithmic bytes per second over the whole
step; `roofline` describes the decode GEMV kernel, `gemm` the M=2048 prefill
GEMM of the same quantization scheme, `cpu_baseline` the CPU restatement of the
reference's path timed on this machine's host cores.  Further objects on the same
line: `stack` (32 decoder layers' linears run as one captured instruction list at
M = 1, 8, 16, 32), `fpA_intB` (int8 per-channel weights, K=8192, N=28672, M = 1, 16,
128, 512), `autogptq` (N = K = 4096; under `larger_shapes` 4096 -> 22016 and 11008 -> 4096; under `decode_step_as_list`
the four decoder linears as one launch against four; under `stack` the 32-layer stack) and `kn_gemv` (the
neighbouring checkpoint layouts at decode) and
`calibration` (measured pure-read and MFMA-only ceilings); `single_gemv_4096x4096` (one linear per launch, with
its own roofline), `list_steady_state` (the list kernel over 906 MB in one launch) and `f16acc` (the
fp16-accumulate decode entry point).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "int4 GEMV HBM GB/s (M=1, %peak); int4 GEMM TFLOPS (M=2048, %MFMA peak)"
DECODE_SHAPES = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]  # (N, K)
PREFILL_SHAPES = [(11008, 4096), (4096, 11008)]
PREFILL_M = 2048
HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch of the two headline kernels come from rocprofv3 counters collected offline
# (this script cannot read hardware counters): profiles/hbm_traffic.json holds the figures, the
# summary they were taken from and its date; it is copied into the JSON line, or null if absent.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def offline_traffic(kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)[kernel]
        return t["bytes_per_launch"], {"file": t["source"], "date": t["date"]}
    except (OSError, KeyError, ValueError):
        return None, None


def gemv_bytes(M, N, K):
    """Algorithmic bytes of one format-A linear: codes + scales + x + y."""
    return N * K // 2 + N * (K // 32) * 2 + M * K * 2 + M * N * 2


def make_device_set(torch, seed):
    """Random codes / scales for the four decode linears, generated on the device."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    out = []
    for N, K in DECODE_SHAPES:
        W = torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device="cuda", generator=g)
        S = (torch.rand((N, K // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
        out.append((W, S))
    return out


def cpu_baseline(budget_s=8.0):
    """Times the CPU oracle (the reference's llvm-target semantics: decode pass +
    naive fp32-accumulate loop nest, one thread) on the same four linears."""
    from oracle import wq_oracle as o

    o.build()
    rng = np.random.default_rng(0)
    sets = []
    for N, K in DECODE_SHAPES:
        x, W, S = o.make_q4g32_inputs(1, N, K, seed=int(rng.integers(1 << 30)))
        sets.append((W, S, x))
    nbytes = sum(gemv_bytes(1, N, K) for N, K in DECODE_SHAPES)
    reps, t0 = 0, time.perf_counter()
    while True:
        for W, S, x in sets:
            o.q4g32_linear(W, S, x, nthreads=1)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s and reps >= 2:
            break
    # the same restatement with its two loop nests split over the host cores this process may use
    # (rows are independent, the sums do not change): reported next to the single-thread figure
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    cores = max(1, min(cores, 16))
    preps, p0 = 0, time.perf_counter()
    while True:
        for W, S, x in sets:
            o.q4g32_linear(W, S, x, nthreads=cores)
        preps += 1
        pdt = time.perf_counter() - p0
        if pdt >= budget_s / 4 and preps >= 2:
            break
    return {
        "value": round(nbytes * reps / dt / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{reps} full steps (the same four M=1 linears), {dt:.1f} s, single thread, "
                  f"{dt / reps * 1e3:.1f} ms per step",
        "host_cpus": os.cpu_count(),
        "parallel": {"value": round(nbytes * preps / pdt / 1e9, 4), "unit": "GB/s", "cores": cores,
                     "sample": f"{preps} full steps, {pdt:.1f} s, OpenMP over output rows"},
    }


def _time_on_stream(torch, stream, fn, reps):
    """Average milliseconds of `fn()` over `reps` calls, with events recorded on `stream`."""
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record(stream)
    for _ in range(reps):
        fn()
    b.record(stream)
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


SAMPLES = 5
MIN_SAMPLE_MS = 100.0


def _measure(torch, stream, fn, min_ms=None, samples=None):
    """Median / min / max milliseconds per call of `fn()`: `samples` samples, each enough calls to
    last `min_ms`.  Returns (median, dict with the spread)."""
    min_ms = MIN_SAMPLE_MS if min_ms is None else min_ms
    samples = SAMPLES if samples is None else samples
    fn()
    one = max(_time_on_stream(torch, stream, fn, 2), 1e-4)
    reps = max(1, int(np.ceil(min_ms / one)))
    # the first calls are slower than the steady state: size the sample from a sample
    for _ in range(3):
        one = max(_time_on_stream(torch, stream, fn, reps), 1e-4)
        if one * reps >= min_ms:
            break
        reps = int(np.ceil(1.03 * min_ms / one))
    t = sorted(_time_on_stream(torch, stream, fn, reps) for _ in range(samples))
    med = t[len(t) // 2] if len(t) % 2 else 0.5 * (t[len(t) // 2 - 1] + t[len(t) // 2])
    return med, {"samples": samples, "calls_per_sample": reps, "sample_ms": round(med * reps, 1),
                 "min": round(t[0], 6), "max": round(t[-1], 6)}


def bench_list_steady(torch, ops, stream, K=4096, rows_total=131072 * 3, linears=24):
    """The M = 1 list kernel far from its start and end: ONE launch over `linears` equal linears that together
    hold 906 MB of codes and scales (three times the last-level cache), so start-up, drain and the hand-over
    between linears weigh little: the rate the kernel's inner loop sustains."""
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    W = torch.randint(-2**31, 2**31 - 1, (rows_total, K // 8), dtype=torch.int32, device="cuda", generator=g)
    S = (torch.rand((rows_total, K // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
    x = torch.randn((1, K), device="cuda", dtype=torch.float16)
    rows = rows_total // linears
    y = torch.empty((linears, rows), device="cuda", dtype=torch.float16)
    gl = ops.Q4G32GemvList([(W[i * rows:(i + 1) * rows], S[i * rows:(i + 1) * rows], x, y[i:i + 1]) for i in range(linears)])
    gl.run()
    gl.status()
    ms, sp = _measure(torch, stream, gl.run, min_ms=MIN_SAMPLE_MS / 4)
    nbytes = linears * gemv_bytes(1, rows, K)
    del gl
    return {"kernel": "q4g32_gemv_list_kernel", "what": f"one launch, {linears} linears of {rows} x {K}, M = 1",
            "us": round(ms * 1e3, 2), "us_min": round(sp["min"] * 1e3, 2), "us_max": round(sp["max"] * 1e3, 2),
            "bytes_per_launch": nbytes, "GB/s": round(nbytes / ms / 1e6, 1),
            "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}


def bench_f16acc(torch, ops, stream, copies, xs):
    """The fp16-accumulate decode entry point (wq_q4g32_gemv_f16acc) on the four decode linears, M = 1, one launch
    each, cycling the weight copies inside one graph like `per_linear`."""
    res = []
    for si, (N, K) in enumerate(DECODE_SHAPES):
        def one(i, si=si):
            W, S = copies[i % len(copies)][si]
            ops.q4g32_gemv_f16acc(W, S, xs[si])
        for i in range(len(copies)):
            one(i)
        stream.synchronize()
        g1 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g1, stream=stream):
            for i in range(4 * len(copies)):
                one(i)
        ms1, sp1 = _measure(torch, stream, g1.replay, min_ms=MIN_SAMPLE_MS / 4)
        us = ms1 * 1e3 / (4 * len(copies))
        nb = gemv_bytes(1, N, K)
        res.append({"N": N, "K": K, "us": round(us, 3), "GB/s": round(nb / us / 1e3, 1),
                    "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": nb,
                    "us_min": round(sp1["min"] * 1e3 / (4 * len(copies)), 3),
                    "us_max": round(sp1["max"] * 1e3 / (4 * len(copies)), 3)})
        del g1
    # four rows of x in one pass over the weights (the low-batch case), on the largest of the four linears
    N, K = DECODE_SHAPES[2]
    x4 = torch.randn((4, K), device="cuda", dtype=torch.float16)

    def four(i):
        W, S = copies[i % len(copies)][2]
        ops.q4g32_gemv_f16acc(W, S, x4)

    for i in range(len(copies)):
        four(i)
    stream.synchronize()
    g4 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g4, stream=stream):
        for i in range(4 * len(copies)):
            four(i)
    ms4, _ = _measure(torch, stream, g4.replay, min_ms=MIN_SAMPLE_MS / 4)
    us4 = ms4 * 1e3 / (4 * len(copies))
    nb4 = gemv_bytes(4, N, K)
    batch = {"M": 4, "N": N, "K": K, "us": round(us4, 3), "GB/s": round(nb4 / us4 / 1e3, 1),
             "frac_of_hbm_peak": round(nb4 / us4 / 1e3 / HBM_PEAK_GBS, 4), "bytes": nb4}
    del g4
    return {"kernel": "q4g32_gemv_f16acc_kernel (wq_q4g32_gemv_f16acc)", "bound": "hbm", "M": 1, "shapes": res,
            "four_rows_one_pass": batch}


def bench_stack(torch, layers=32, batches=(1, 8, 16, 32)):
    """The four quantized linears of `layers` Llama-2-7B decoder layers (3.6 GB of codes and scales,
    so every step is cache-cold) as one instruction list of PackedFunc calls, planned and replayed
    as one HIP graph by the library's executor."""
    from relax_amd import vm

    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    weights = []
    for _ in range(layers):
        layer = {}
        for name, N, K in vm.LLAMA7B_LINEARS:
            W = torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device="cuda", generator=g)
            S = (torch.rand((N, K // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
            layer[name] = (W, S)
        weights.append(layer)
    stream = torch.cuda.Stream()
    res = {"layers": layers, "instructions_per_step": 4 * layers,
           "launch": "hip_graph of PackedFunc calls; runs of decode linears (M <= 32) fused into one launch "
                     "(M = 1: VALU list kernel; 2 .. 32: MFMA list kernel)", "batches": []}
    for M in batches:
        hidden = torch.randn((M, 4096), device="cuda", dtype=torch.float16)
        attn = torch.randn((M, 4096), device="cuda", dtype=torch.float16)
        act = torch.randn((M, 11008), device="cuda", dtype=torch.float16)
        outp = torch.empty((M, 4096), device="cuda", dtype=torch.float16)
        prog = vm.llama_linear_stack(weights, M, hidden, attn, act, outp)
        ws = prog.plan()
        prog.capture(stream)
        prog.replay(stream)
        stream.synchronize()
        ms, spread = _measure(torch, stream, lambda: prog.replay(stream))
        prog.status(stream)
        nbytes = layers * sum(gemv_bytes(M, N, K) for _, N, K in vm.LLAMA7B_LINEARS)
        res["batches"].append({"M": M, "ms_per_step": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1),
                               "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                               "ms_spread": spread, "launches_per_step": 4 * layers - sum(
                                   len(prog.fused_order(g)) - 1 for g in range(prog.num_fused_groups)),
                               "bytes_per_step": nbytes, "workspace_bytes": ws,
                               "workspace_without_reuse": prog.unplanned_bytes})
        del prog
    return res


def bench_intb(torch, ops, K=8192, N=28672, batches=(1, 16, 128, 512), copies=3, nbit=8, group=-1):
    """fp16 x int8 per-channel weights in the preprocessed layout (or, for the neighbouring schemes,
    int4 and / or group-64 scales); `copies` weight copies (more than the last-level cache) are cycled so
    that small M reads HBM."""
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    Ws = []
    for _ in range(copies):
        q = torch.randint(-127, 128, (K, N if nbit == 8 else N // 2), dtype=torch.int8, device="cuda", generator=g)
        Ws.append(ops.ft_preprocess_weight(q, 80, nbit == 4))
        del q
    s = (torch.rand((N,) if group <= 0 else (K // group, N), device="cuda", generator=g) * 0.009 + 0.001).to(torch.float16)
    stream = torch.cuda.current_stream()
    res = {"K": K, "N": N, "weight": f"int{nbit} " + ("per-channel" if group <= 0 else f"group-{group}"), "batches": []}
    for M in batches:
        x = torch.randn((M, K), device="cuda", dtype=torch.float16)
        y = torch.empty((M, N), device="cuda", dtype=torch.float16)
        it = [0]

        def fn():
            ops.fpA_intB_gemm(x, Ws[it[0] % copies], s, weight_nbit=nbit, group_size=group, out=y)
            it[0] += 1

        for _ in range(copies):
            fn()
        def cycle():
            for _ in range(copies):
                fn()

        ms, spread = _measure(torch, stream, cycle, min_ms=MIN_SAMPLE_MS / 2)
        ms /= copies
        nbytes = K * N * nbit // 8 + s.numel() * 2 + M * K * 2 + M * N * 2
        tf = 2.0 * M * N * K / ms / 1e9
        res["batches"].append({"M": M, "us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1),
                               "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                               "TFLOP/s": round(tf, 1), "frac_of_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                               "us_spread": {k: (round(v / copies * 1e3, 2) if k in ("min", "max") else v)
                                             for k, v in spread.items()}})
    return res


def bench_autogptq(torch, ops, K=4096, N=4096, group=128, batches=(1, 8), copies=40):
    """An AutoGPTQ layer of the shape the reference's test uses (int4, zero points, group 128), with and
    without a row order (desc_act); `copies` prepared layers (more than the last-level cache) are cycled
    inside one captured graph.  Bytes = codes + (scale, zero point) pairs + x + y (+ the gather's traffic)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(12)
    G = K // group
    res = {"K": K, "N": N, "group_size": group, "weight": "int4 + zero points", "cases": []}
    for act in (False, True):
        layers = []
        for _ in range(copies):
            qw = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device="cuda", generator=g)
            qz = torch.randint(-2**31, 2**31 - 1, (G, N // 8), dtype=torch.int32, device="cuda", generator=g)
            sc = (torch.rand((G, N), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
            gi = (torch.arange(K, device="cuda") // group).to(torch.int32)
            if act:
                gi = gi[torch.randperm(K, device="cuda", generator=g)].contiguous()
            layers.append(ops.gptq_prepare(qw, qz, sc, gi))
        for M in batches:
            x = torch.randn((M, K), device="cuda", dtype=torch.float16)
            y = torch.empty((M, N), device="cuda", dtype=torch.float16)
            ws = torch.empty((max(1, ops.gptq_workspace_bytes(M, K, act)),), dtype=torch.uint8, device="cuda")

            def step():
                for w in layers:
                    ops.gptq_linear(w, x, out=y, workspace=ws)

            step()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            graph.replay()
            ms, _ = _measure(torch, torch.cuda.current_stream(), graph.replay, min_ms=MIN_SAMPLE_MS / 4, samples=3)
            ms /= copies
            nbytes = N * K // 2 + N * G * 4 + M * K * 2 + M * N * 2 + (M * K * 4 + K * 4 if act else 0)
            res["cases"].append({"M": M, "row_order": act, "us": round(ms * 1e3, 2),
                                 "GB/s": round(nbytes / ms / 1e6, 1),
                                 "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)})
        del layers
    return res


def bench_autogptq_list(torch, ops, copies=6, group=128):
    """The decode step of the four Llama-2-7B-shaped linears as prepared AutoGPTQ layers (group 128) at M = 1,
    without and with a row order (desc_act): ONE launch of the list kernel per step (`wq_gptq_gemv_list_create`;
    with a row order one small gather kernel for all four layers runs in front of it, their x coming from outside
    the list) against four calls of `wq_gptq_linear` (each preceded by a gather kernel when there is a row order); `copies` weight sets (more than the last-level
    cache) are cycled inside one captured graph.  Bytes = codes + (scale, zero point) pairs + x + y."""
    g = torch.Generator(device="cuda")
    g.manual_seed(13)
    nbytes = sum(N * K // 2 + N * (K // group) * 4 + K * 2 + N * 2 for N, K in DECODE_SHAPES)
    res = {"group_size": group, "weight": "int4 + zero points", "linears": [list(s) for s in DECODE_SHAPES],
           "bytes_per_step": nbytes, "weight_sets": copies, "cases": []}
    xs = [torch.randn((1, K), device="cuda", dtype=torch.float16) for _, K in DECODE_SHAPES]
    ys = [torch.empty((1, N), device="cuda", dtype=torch.float16) for N, _ in DECODE_SHAPES]
    wss = [torch.empty((max(1, ops.gptq_workspace_bytes(1, K, True)),), dtype=torch.uint8, device="cuda")
           for _, K in DECODE_SHAPES]
    for act in (False, True):
        sets = []
        for _ in range(copies):
            layers = []
            for N, K in DECODE_SHAPES:
                G = K // group
                qw = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device="cuda", generator=g)
                qz = torch.randint(-2**31, 2**31 - 1, (G, N // 8), dtype=torch.int32, device="cuda", generator=g)
                sc = (torch.rand((G, N), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
                gi = (torch.arange(K, device="cuda") // group).to(torch.int32)
                if act:
                    gi = gi[torch.randperm(K, device="cuda", generator=g)].contiguous()
                layers.append(ops.gptq_prepare(qw, qz, sc, gi))
                del qw, qz, sc
            sets.append(layers)
        lists = [ops.GptqGemvList([(w, x, y) for w, x, y in zip(layers, xs, ys)]) for layers in sets]

        def as_list():
            for l in lists:
                l.run()

        def call_by_call():
            for layers in sets:
                for w, x, y, ws in zip(layers, xs, ys, wss):
                    ops.gptq_linear(w, x, out=y, workspace=ws)

        case = {"row_order": act}
        for name, fn in (("one_launch", as_list), ("four_calls", call_by_call)):
            fn()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(4):
                    fn()
            graph.replay()
            ms, _ = _measure(torch, torch.cuda.current_stream(), graph.replay, min_ms=MIN_SAMPLE_MS / 4, samples=3)
            ms /= 4 * copies
            case[name] = {"us_per_step": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
                          "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
            del graph
        lists[0].status()
        res["cases"].append(case)
        del lists, sets
    return res


def bench_autogptq_stack(torch, ops, layers=32, group=128):
    """The 32-layer stack of `stack` with AutoGPTQ layers (group 128, rows in group order) at M = 1: 128
    `relax_amd.autogptq_matmul` calls per step, run by the executor as one launch, and call by call."""
    from relax_amd import vm

    g = torch.Generator(device="cuda")
    g.manual_seed(14)
    weights = []
    for _ in range(layers):
        layer = {}
        for name, N, K in vm.LLAMA7B_LINEARS:
            G = K // group
            qw = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device="cuda", generator=g)
            qz = torch.randint(-2**31, 2**31 - 1, (G, N // 8), dtype=torch.int32, device="cuda", generator=g)
            sc = (torch.rand((G, N), device="cuda", generator=g) * 0.0015 + 0.0005).to(torch.float16)
            gi = (torch.arange(K, device="cuda") // group).to(torch.int32)
            layer[name] = ops.gptq_prepare(qw, qz, sc, gi)
            del qw, qz, sc
        weights.append(layer)
    hidden = torch.randn((1, 4096), device="cuda", dtype=torch.float16)
    attn = torch.randn((1, 4096), device="cuda", dtype=torch.float16)
    act = torch.randn((1, 11008), device="cuda", dtype=torch.float16)
    outp = torch.empty((1, 4096), device="cuda", dtype=torch.float16)
    nbytes = layers * sum(N * K // 2 + N * (K // group) * 4 + K * 2 + N * 2 for _, N, K in vm.LLAMA7B_LINEARS)
    res = {"layers": layers, "group_size": group, "M": 1, "bytes_per_step": nbytes}
    stream = torch.cuda.Stream()
    for name, fuse in (("one_launch", 1), ("call_by_call", 0)):
        prog = vm.llama_autogptq_stack(weights, hidden, attn, act, outp)
        prog.set_option("fuse_decode", fuse)
        prog.plan()
        prog.capture(stream)
        prog.replay(stream)
        stream.synchronize()
        ms, _ = _measure(torch, stream, lambda: prog.replay(stream), min_ms=MIN_SAMPLE_MS / 2, samples=3)
        prog.status(stream)
        res[name] = {"ms_per_step": round(ms, 4), "GB/s": round(nbytes / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                     "launches_per_step": 4 * layers - sum(len(prog.fused_order(i)) - 1 for i in range(prog.num_fused_groups))}
        del prog
    return res


def bench_kn_gemv(torch, ops, copies=24):
    """The decode linear over K-major (KN) q4f16_1 weights used in place (`wq_q4g32_kn_gemv`), M = 1, the
    four Llama-2-7B shapes; `copies` weight copies (more than the last-level cache) are cycled inside one
    captured graph.  Bytes = codes + scales + x + y."""
    from relax_amd import _lib

    L = _lib.lib()
    g = torch.Generator(device="cuda")
    g.manual_seed(13)
    res = {"weight": "q4f16_1, K-major [K/8, N]", "M": 1, "shapes": []}
    for N, K in ((12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)):
        Ws = [torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device="cuda", generator=g)
              for _ in range(copies)]
        S = (torch.rand((K // 32, N), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
        x = torch.randn((1, K), device="cuda", dtype=torch.float16)
        y = torch.empty((1, N), device="cuda", dtype=torch.float16)
        ws = torch.empty((max(16, int(L.wq_q4g32_kn_gemv_workspace_bytes(1, N, K))),), dtype=torch.uint8, device="cuda")

        def step():
            for W in Ws:
                ops.q4g32_kn_gemv(W, S, x, out=y, workspace=ws)

        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        graph.replay()
        ms, _ = _measure(torch, torch.cuda.current_stream(), graph.replay, min_ms=MIN_SAMPLE_MS / 4, samples=3)
        ms /= copies
        nbytes = N * K // 2 + N * (K // 32) * 2 + K * 2 + N * 2
        res["shapes"].append({"N": N, "K": K, "us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1),
                              "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)})
        del Ws
        torch.cuda.empty_cache()
    return res


def bench_calibration(torch):
    """What this GPU reaches with no algorithm in the way: a streaming read of 1 GiB and MFMA issue only."""
    import ctypes

    from relax_amd import _lib

    L = _lib.calibrate_lib()
    stream = torch.cuda.current_stream()
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
    scratch = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")

    def rd():
        _lib.check(L.wq_calibrate_read(src.data_ptr(), src.numel(), scratch.data_ptr(), stream.cuda_stream), "read")

    rd()
    ms_read, _ = _measure(torch, stream, rd, min_ms=MIN_SAMPLE_MS / 4, samples=3)
    flops = ctypes.c_double(0.0)

    def mf():
        _lib.check(L.wq_calibrate_mfma_f16(scratch.data_ptr(), scratch.numel(), 4000, ctypes.byref(flops),
                                           stream.cuda_stream), "mfma")

    mf()
    ms_mfma, _ = _measure(torch, stream, mf, min_ms=MIN_SAMPLE_MS / 4, samples=3)
    # the decode GEMV on a matrix large enough that launch, ramp-up and drain no longer matter
    # (131072 x 4096, 302 MB per copy, three copies cycled): the kernel's steady-state rate
    del src
    from relax_amd import ops

    Nl, Kl = 131072, 4096
    g = torch.Generator(device="cuda")
    g.manual_seed(13)
    Wl = [torch.randint(-2**31, 2**31 - 1, (Nl, Kl // 8), dtype=torch.int32, device="cuda", generator=g) for _ in range(3)]
    Sl = [(torch.rand((Nl, Kl // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16) for _ in range(3)]
    xl = torch.randn((1, Kl), device="cuda", dtype=torch.float16)
    yl = torch.empty((1, Nl), device="cuda", dtype=torch.float16)

    def big():
        for i in range(3):
            ops.q4g32_linear(Wl[i], Sl[i], xl, out=yl)

    big()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        big()
    graph.replay()
    ms_big, _ = _measure(torch, torch.cuda.current_stream(), graph.replay, min_ms=MIN_SAMPLE_MS / 4, samples=3)
    ms_big /= 3
    big_bytes = gemv_bytes(1, Nl, Kl)
    return {"read_1GiB_GB/s": round((1 << 30) / ms_read / 1e6, 1), "hbm_vendor_peak_GB/s": HBM_PEAK_GBS,
            "gemv_steady_state": {"N": Nl, "K": Kl, "us": round(ms_big * 1e3, 1),
                                  "GB/s": round(big_bytes / ms_big / 1e6, 1),
                                  "frac_of_hbm_peak": round(big_bytes / ms_big / 1e6 / HBM_PEAK_GBS, 4)},
            "mfma_f16_only_TFLOP/s": round(flops.value / ms_mfma / 1e9, 1),
            "mfma_f16_vendor_peak_TFLOP/s": MFMA_F16_PEAK_TFLOPS}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--copies", type=int, default=16, help="distinct weight copies in the ring")
    ap.add_argument("--samples", type=int, default=5, help="timed samples per measurement (the median is reported)")
    ap.add_argument("--min-sample-ms", type=float, default=100.0, help="a sample repeats its work until it lasts this long")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prefill GEMM measurement")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of through a HIP graph")
    ap.add_argument("--no-stack", action="store_true", help="skip the 32-layer stack measurement")
    ap.add_argument("--no-intb", action="store_true", help="skip the fpA_intB measurement")
    ap.add_argument("--no-autogptq", action="store_true", help="skip the AutoGPTQ layer measurement")
    ap.add_argument("--no-calibration", action="store_true", help="skip the pure-read / MFMA-only ceilings")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device copy a few times (reference point for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of rocprofv3) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch

    from relax_amd import ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)  # reads 2^30 bytes and writes 2^30 bytes per launch
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": 1 << 30, "launches": 4}))
        return
    global SAMPLES, MIN_SAMPLE_MS
    SAMPLES, MIN_SAMPLE_MS = args.samples, args.min_sample_ms
    copies = [make_device_set(torch, 1000 + i) for i in range(args.copies)]
    xs = [torch.randn((1, K), device="cuda", dtype=torch.float16) for _, K in DECODE_SHAPES]
    ys = [torch.empty((1, N), device="cuda", dtype=torch.float16) for N, _ in DECODE_SHAPES]
    step_bytes = sum(gemv_bytes(1, N, K) for N, K in DECODE_SHAPES)
    # one list per weight copy: the four linears of a step are ONE launch
    lists = [ops.Q4G32GemvList([(W, S, x, y) for (W, S), x, y in zip(c, xs, ys)]) for c in copies]

    def step(i):
        lists[i % args.copies].run()

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            step(i)
        stream.synchronize()
        if args.no_graph:
            def run_steps():
                for i in range(args.steps):
                    step(i)
        else:
            # one graph holds all timed steps: the host only issues a single launch
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(args.steps):
                    step(i)
            run_steps = graph.replay
        # EXACTLY `steps` steps per repetition, bracketed by synchronisation; median over samples
        total_ms, spread = _measure(torch, stream, run_steps)
        lists[0].status()

    ms_per_step = total_ms / args.steps
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    # the list kernel is the only kernel in the timed region, one launch per step: its average
    # launch duration (gaps between launches included, so a slight under-estimate of the kernel) is
    avg_launch_us = ms_per_step * 1e3
    achieved = step_bytes / (avg_launch_us * 1e-6) / 1e9
    traffic, traffic_src = offline_traffic("q4g32_gemv_list_kernel")

    # every linear on its own, as a single call of wq_q4g32_linear issues it (the streaming kernel of one
    # linear per launch), cycling the weight copies inside one graph
    per_shape = []
    with torch.cuda.stream(stream):
        for si, (N, K) in enumerate(DECODE_SHAPES):
            def one(i, si=si):
                W, S = copies[i % args.copies][si]
                ops.q4g32_linear(W, S, xs[si], out=ys[si], kernel="gemv")
            for i in range(args.copies):
                one(i)
            stream.synchronize()
            g1 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g1, stream=stream):
                for i in range(4 * args.copies):
                    one(i)
            ms1, sp1 = _measure(torch, stream, g1.replay, min_ms=MIN_SAMPLE_MS / 4)
            us = ms1 * 1e3 / (4 * args.copies)
            nb = gemv_bytes(1, N, K)
            per_shape.append({"N": N, "K": K, "us": round(us, 3), "GB/s": round(nb / us / 1e3, 1),
                              "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "bytes": nb,
                              "us_min": round(sp1["min"] * 1e3 / (4 * args.copies), 3),
                              "us_max": round(sp1["max"] * 1e3 / (4 * args.copies), 3)})
            del g1

    out = {
        "metric": METRIC,
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "Llama-2-7B-shaped decode linears at M=1, int4 group-32 (q4f16_1): "
                        "4096->12288, 4096->4096, 4096->22016, 11008->4096",
            "weight_copies_in_ring": args.copies,
            "ring_bytes": step_bytes * args.copies,
            "launch": ("eager" if args.no_graph else "hip_graph") + ", one launch of the list kernel per step",
            "bytes_per_step": step_bytes,
        },
        "timing": {"protocol": "median of samples; a sample is a whole number of repetitions of the timed steps "
                               "lasting at least min_sample_ms; HIP events on the launch stream",
                   "min_sample_ms": MIN_SAMPLE_MS, **spread,
                   "ms_per_step_min": round(spread["min"] / args.steps, 6),
                   "ms_per_step_max": round(spread["max"] / args.steps, 6)},
        "roofline": {
            "kernel": "q4g32_gemv_list_kernel",
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_src,
            "avg_launch_us": round(avg_launch_us, 3),
            "bytes_per_launch": step_bytes,
        },
        # the same four linears one launch each (what a single wq_q4g32_linear call costs), and the
        # 4096 x 4096 linear of the single-GEMV configuration on its own
        "per_linear": per_shape,
    }
    # the single-GEMV configuration (one 4096 x 4096 linear, one launch of the streaming kernel): its own roofline
    c1 = dict(next(p for p in per_shape if p["N"] == 4096 and p["K"] == 4096))
    c1_traffic, c1_src = offline_traffic("q4g32_gemv_kernel")
    c1["roofline"] = {"kernel": "q4_gemv_kernel<Q4G32Row> (wq_q4g32_gemv)", "bound": "hbm", "achieved": c1["GB/s"],
                      "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": c1["frac_of_hbm_peak"],
                      "avg_launch_us": c1["us"], "bytes_per_launch": c1["bytes"],
                      "traffic": c1_traffic, "traffic_source": c1_src}
    out["single_gemv_4096x4096"] = c1
    with torch.cuda.stream(stream):
        out["list_steady_state"] = bench_list_steady(torch, ops, stream)
        out["f16acc"] = bench_f16acc(torch, ops, stream, copies, xs)

    if not args.no_gemm:
        gem, vendor = [], []
        tot_flops, tot_ms, vendor_ms = 0.0, 0.0, 0.0
        cur = torch.cuda.current_stream()
        for N, K in PREFILL_SHAPES:
            g = torch.Generator(device="cuda")
            g.manual_seed(N)
            W = torch.randint(-2**31, 2**31 - 1, (N, K // 8), dtype=torch.int32, device="cuda", generator=g)
            S = (torch.rand((N, K // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
            x = torch.randn((PREFILL_M, K), device="cuda", dtype=torch.float16)
            y = torch.empty((PREFILL_M, N), device="cuda", dtype=torch.float16)
            for _ in range(3):
                ops.q4g32_linear(W, S, x, out=y, kernel="gemm")
            ms, sp = _measure(torch, cur, lambda: ops.q4g32_linear(W, S, x, out=y, kernel="gemm"))
            fl = 2.0 * PREFILL_M * N * K
            gem.append({"M": PREFILL_M, "N": N, "K": K, "us": round(ms * 1e3, 2), "tflops": round(fl / ms / 1e9, 1),
                        "us_min": round(sp["min"] * 1e3, 2), "us_max": round(sp["max"] * 1e3, 2),
                        "samples": sp["samples"], "calls_per_sample": sp["calls_per_sample"]})
            tot_flops += fl
            tot_ms += ms
            # for scale: the vendor library's plain fp16 GEMM (no dequantization) on the same shape, weights
            # as an fp16 [N, K] tensor (torch.matmul -> hipBLASLt / rocBLAS); not part of `value`
            Wf = torch.randn((N, K), device="cuda", dtype=torch.float16)
            for _ in range(3):
                torch.matmul(x, Wf.t(), out=y)
            vms, _ = _measure(torch, cur, lambda: torch.matmul(x, Wf.t(), out=y), min_ms=MIN_SAMPLE_MS / 4, samples=3)
            vendor.append({"N": N, "K": K, "us": round(vms * 1e3, 2), "tflops": round(fl / vms / 1e9, 1)})
            vendor_ms += vms
            del W, S, x, y, Wf
        # the same GEMM over weights packed along N (the layout of the reference's prefill fixture,
        # tests/python/dlight/test_gpu_matmul.py:352-401, at its own 4096 x 4096 and at the gate/up shape)
        ngroup = []
        for N, K in ((4096, 4096), PREFILL_SHAPES[0]):
            g = torch.Generator(device="cuda")
            g.manual_seed(N + 1)
            W = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
            S = (torch.rand((K, N // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
            W_nk, ST = ops.q4n32_prepare(W, S)
            x = torch.randn((PREFILL_M, K), device="cuda", dtype=torch.float16)
            y = torch.empty((PREFILL_M, N), device="cuda", dtype=torch.float16)
            for _ in range(3):
                ops.q4n32_linear(W_nk, ST, x, out=y)
            ms, _ = _measure(torch, cur, lambda: ops.q4n32_linear(W_nk, ST, x, out=y), min_ms=MIN_SAMPLE_MS / 4, samples=3)
            fl = 2.0 * PREFILL_M * N * K
            ngroup.append({"M": PREFILL_M, "N": N, "K": K, "us": round(ms * 1e3, 2), "tflops": round(fl / ms / 1e9, 1),
                           "frac_of_mfma_peak": round(fl / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4)})
            del W, S, W_nk, ST, x, y
        # ... and its decode kernel at M = 1, weight copies (more than the last-level cache) cycled inside one graph
        ngroup_decode = []
        for (N, K), ncopy in (((4096, 4096), 40), ((11008, 4096), 16)):
            g = torch.Generator(device="cuda")
            g.manual_seed(N + 2)
            prepared = []
            for _ in range(ncopy):
                W = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device="cuda", generator=g)
                S = (torch.rand((K, N // 32), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
                prepared.append(ops.q4n32_prepare(W, S))
                del W, S
            x = torch.randn((1, K), device="cuda", dtype=torch.float16)
            y = torch.empty((1, N), device="cuda", dtype=torch.float16)

            def cycle():
                for W_nk, ST in prepared:
                    ops.q4n32_linear(W_nk, ST, x, out=y)

            cycle()
            torch.cuda.synchronize()
            g1 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g1):
                cycle()
            g1.replay()
            ms, _ = _measure(torch, cur, g1.replay, min_ms=MIN_SAMPLE_MS / 4, samples=3)
            us = ms * 1e3 / ncopy
            nb = gemv_bytes(1, N, K)  # (codes + scales + x + y: the same bytes as format A)
            ngroup_decode.append({"M": 1, "N": N, "K": K, "us": round(us, 2), "GB/s": round(nb / us / 1e3, 1),
                                  "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBS, 4)})
            del g1, prepared
        tf = tot_flops / tot_ms / 1e9
        gtraffic, gsrc = offline_traffic("gemm_lds_kernel")
        out["gemm"] = {
            "kernel": "gemm_lds_kernel<Q4G32LdsPolicy>",
            "value": round(tf, 1),
            "unit": "TFLOP/s",
            "shapes": gem,
            "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": gtraffic, "traffic_source": gsrc},
            "vendor_fp16_gemm_same_shapes": {"what": "torch.matmul(x, W_fp16.T): the library's dense fp16 GEMM, no dequantization",
                                             "value": round(tot_flops / vendor_ms / 1e9, 1), "unit": "TFLOP/s",
                                             "frac_of_mfma_peak": round(tot_flops / vendor_ms / 1e9 / MFMA_F16_PEAK_TFLOPS, 4),
                                             "shapes": vendor},
            "packed_along_n": {"kernel": "gemm_lds_kernel<Q4N32LdsPolicy> (wq_q4n32_linear)", "shapes": ngroup,
                               "decode_kernel": "q4n32_gemv_kernel (wq_q4n32_linear, M <= 4)", "decode": ngroup_decode},
        }

    del lists
    del copies
    torch.cuda.empty_cache()
    if not args.no_stack:
        out["stack"] = bench_stack(torch)
    if not args.no_intb:
        out["fpA_intB"] = bench_intb(torch, ops)
        torch.cuda.empty_cache()
        # the neighbouring schemes of the same entry point, two batch sizes each
        out["fpA_intB_variants"] = [bench_intb(torch, ops, batches=(1, 128), copies=4, nbit=4),
                                    bench_intb(torch, ops, batches=(1, 128), copies=3, nbit=8, group=64)]
        torch.cuda.empty_cache()
    if not args.no_autogptq:
        out["autogptq"] = bench_autogptq(torch, ops)
        # the same layer type at the two large decoder shapes (the 4096 x 4096 matrix is 8.9 MB: launch-bound)
        out["autogptq"]["decode_step_as_list"] = bench_autogptq_list(torch, ops)
        out["autogptq"]["stack"] = bench_autogptq_stack(torch, ops)
        torch.cuda.empty_cache()
        out["autogptq"]["larger_shapes"] = [bench_autogptq(torch, ops, K=4096, N=22016, batches=(1,), copies=12),
                                            bench_autogptq(torch, ops, K=11008, N=4096, batches=(1,), copies=24)]
        out["kn_gemv"] = bench_kn_gemv(torch, ops)
    if not args.no_calibration:
        out["calibration"] = bench_calibration(torch)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
