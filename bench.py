#!/usr/bin/env python3
"""Benchmark of the forward bound-propagation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only-headline]

Prints ONE JSON line on stdout (a table for humans goes to stderr).

Headline workload ("step"): benchmark configuration 1 -- the ReLU and the tanh relaxation of
bounds lw/uw [1,128,256,512], lb/ub [1,128,512], two perturbed words, eps = 0.01, once for each
p in {1, 2, inf}: six fused concretize+relax launches per step.  `value` is the algorithmic
HBM traffic of a step (read lw, uw; write lw', uw'; read and write the constant terms:
16*L*D*H + 16*L*H bytes per launch) divided by the step time, inputs resident in HBM.

The same JSON line carries, under "ops", one entry per benchmark configuration (0..4) with
latency, achieved TFLOP/s or GB/s, roofline fraction and the CPU baseline, because the metric
is a per-op figure.

`cpu_baseline` times the CPU oracle (a PyTorch restatement of the reference's Bounds methods,
kind "port") on the host cores of the same machine; it is the checker being timed as a
baseline, never part of the measured GPU path.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "bound-prop latency & TFLOP/s (matmul/dot/conv) or HBM GB/s (relu/tanh), % roofline"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published
INF = float("inf")
WARM_SECONDS = 0.25            # minimum warm-up per measurement; --profile shortens it (the trace stays small, yet the
                               # launches that are timed, and most of those the profiler averages, run at settled clocks)

COLD_SETS = 5                  # disjoint operand sets cycled by the cold measurement (1.35 GB between reuses)


def traffic_from_profile():
    """HBM bytes per launch of the relaxation kernels as the hardware counters saw them: the lines
    `traffic_bytes_per_launch <relu|tanh> <warm|cold> <bytes>` of profiles/hbm_traffic_relaxations.txt (rocprofv3
    --pmc FETCH_SIZE / WRITE_SIZE of this program, scaled by the same counters on faith_copy_f32 of known
    size).  Empty if the summary is missing."""
    import re
    out = {}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic_relaxations.txt")) as f:
            for m in re.finditer(r"^traffic_bytes_per_launch\s+(\w+)\s+(warm|cold)\s+(\d+)", f.read(), flags=re.M):
                out[(m.group(1), m.group(2))] = int(m.group(3))
    except OSError:
        pass
    return out


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gpu_times_ms(fn, n, warmup):
    """Per-launch durations from HIP events recorded on the launch stream (torch's current one)."""
    import torch
    # warm up by count AND by time: clocks and caches settle only after ~0.2 s of sustained work
    t0 = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - t0 < WARM_SECONDS:
        fn()
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for s, e in evs:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return [s.elapsed_time(e) for s, e in evs]


def cpu_time_s(fn, reps=1, warmup=0):
    for _ in range(warmup):
        fn()
    ts = []
    for _ in range(reps):
        t = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t)
    return statistics.median(ts)


def to_dev(d):
    return {k: v.cuda().contiguous() for k, v in d.items()}


def quad(d):
    return d["lw"], d["lb"], d["uw"], d["ub"]


# ------------------------------------------------------------------------------------------
# per-configuration measurements
# ------------------------------------------------------------------------------------------
# Products the kernels multiply out of those the reference's formulas write.  The sign-split pair
# C_l = A_l W+ + A_u W-, C_u = A_u W+ + A_l W- is computed as centre -+ radius (two products, not four); of the
# dot product's eight products per term the four y terms, which share their multiplier, become two.  The roofline
# fraction counts the products that are multiplied (what the MFMA pipe does); the rate in the reference's own
# formulation is reported beside it for comparison with numbers quoted that way.
EXECUTED = {"linear": 2 / 4, "conv": 2 / 4, "dot": 6 / 8}


def op_entry(name, kind, times_ms, work, cpu=None, extra=None, form=None):
    """kind 'hbm': work in bytes -> GB/s; kind 'mfma': work in flop of the reference's formulation -> TFLOP/s of
    the products that are executed (form: a key of EXECUTED)."""
    med = statistics.median(times_ms)
    reference_work = work
    if kind == "hbm":
        ach, peak, unit = work / med / 1e6, HBM_PEAK_GBS, "GB/s"
    else:
        work = int(work * EXECUTED[form])
        ach, peak, unit = work / med / 1e9, MFMA_FP32_PEAK_TFLOPS, "TFLOP/s"
    e = {"op": name, "latency_us": round(med * 1e3, 2), "latency_min_us": round(min(times_ms) * 1e3, 2),
         "bound": kind, "achieved": round(ach, 2), "peak": peak, "unit": unit, "frac": round(ach / peak, 4),
         "work": work}
    if kind == "mfma" and EXECUTED[form] != 1.0:
        e["reference_formulation"] = {"flop": reference_work, "tflops": round(reference_work / med / 1e9, 2),
                                      "products_executed_of_written": EXECUTED[form]}
    if cpu is not None:
        e["cpu_baseline"] = cpu
    if extra:
        e.update(extra)
    return e


def bench_config0(args, ops, O, wl):
    import torch
    c = wl.make_config(0)
    x, W, b = to_dev(c["x"]), c["W"].cuda(), c["bias"].cuda()
    out = ops.linear_concretize(*quad(x), W, b, c["p"], c["eps"], 1)       # caller-owned results, reused by every call

    def step():
        ops.linear_concretize(*quad(x), W, b, c["p"], c["eps"], 1, out=out)
    flop = 4 * 2 * (16 * 64 + 16) * 64 * 64
    t = gpu_times_ms(step, 200, 20)
    # the kernel alone: 200 launches replayed from a captured HIP graph (no host between them)
    kernel_us = None
    if not args.profile:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(200):
                    step()
        torch.cuda.current_stream().wait_stream(side)
        graph.replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        graph.replay()
        e.record()
        torch.cuda.synchronize()
        kernel_us = round(s.elapsed_time(e) * 1e3 / 200, 2)
        del graph
    # the call as a fresh caller makes it (results allocated per call)
    t_alloc = gpu_times_ms(lambda: ops.linear_concretize(*quad(x), W, b, c["p"], c["eps"], 1), 200, 20)
    # and as a caller makes it who repeats the launch on the same buffers: arguments converted once
    bound = ops.bind_linear_concretize(*quad(x), W, b, c["p"], c["eps"], 1, out=out)
    t_bound = gpu_times_ms(bound, 200, 20)
    cpu = None
    if not args.no_cpu:
        xo = O.LinearBounds(*quad(c["x"]))
        s_ = cpu_time_s(lambda: O.concretize(O.linear(xo, c["W"], c["bias"]), c["p"], c["eps"]), reps=20, warmup=3)
        cpu = {"latency_us": round(s_ * 1e6, 1), "value": round(flop / s_ / 1e12, 4), "unit": "TFLOP/s"}
    return op_entry("config0 linear+concretize(p=inf) [1,16,64,64]x[64,64]", "mfma", t_bound, flop, cpu, form="linear", extra=
                    {"note": "34 MFLOP: launch-latency bound (layer and dual norm in one launch), latency is the figure of merit; "
                             "latency_us is one call from Python into caller-owned results with the arguments bound once "
                             "(ops.bind_linear_concretize: what a caller that repeats the launch on the same buffers pays)",
                     "kernel_us_back_to_back_from_a_graph": kernel_us,
                     "call_us_through_the_checking_wrapper": round(statistics.median(t) * 1e3, 2),
                     "call_us_with_results_allocated_per_call": round(statistics.median(t_alloc) * 1e3, 2)})


def bench_notebook_shapes(args, ops, O):
    """The shapes of the reference's own timing notebooks (Benchmark/tvm_ansor_benchmark.ipynb:369-1036:
    Bounds.relu at B=1, L=2, D_in = H in {64, 128, 256, 512} and Bounds.matmul at L=128, D_in = H = 64),
    the only timings the reference holds (on an NVIDIA workstation GPU; not comparable, listed for scale).
    Launch-latency bound: the figure is microseconds per call through the Python wrapper."""
    import torch
    out = []
    g = torch.Generator().manual_seed(4242)

    def obj(L, D, H):
        lw = torch.randn(1, L, D, H, generator=g) * 0.1
        lb = torch.randn(1, L, H, generator=g)
        return {"lw": lw, "lb": lb, "uw": lw + 0.01 * torch.rand(1, L, D, H, generator=g),
                "ub": lb + 0.1 * torch.rand(1, L, H, generator=g)}
    for n in (64, 128, 256, 512):
        x = obj(2, n, n)
        xd = to_dev(x)
        t = gpu_times_ms(lambda: ops.relu(*quad(xd), 2.0, 0.01, 1), 100, 10)
        cpu = None
        if not args.no_cpu:
            xo = O.LinearBounds(*quad(x))
            s = cpu_time_s(lambda: O.relu(xo, 2.0, 0.01, 1), reps=10, warmup=2)
            cpu = {"latency_us": round(s * 1e6, 1)}
        out.append(op_entry(f"extra: reference notebook shape, relu p=2 [1,2,{n},{n}]", "hbm", t, 16 * 2 * n * n + 16 * 2 * n, cpu))
    x = obj(128, 64, 64)
    xd = to_dev(x)
    W = (torch.randn(64, 64, generator=g) / 8).cuda()
    t = gpu_times_ms(lambda: ops.linear(*quad(xd), W, None), 100, 10)
    cpu = None
    if not args.no_cpu:
        xo = O.LinearBounds(*quad(x))
        Wc = W.cpu()
        s = cpu_time_s(lambda: O.linear(xo, Wc, None), reps=10, warmup=2)
        cpu = {"latency_us": round(s * 1e6, 1)}
    out.append(op_entry("extra: reference notebook shape, matmul [1,128,64,64]x[64,64]", "mfma", t,
                        4 * 2 * (128 * 64 + 128) * 64 * 64, cpu, form="linear"))
    return out


def gpu_back_to_back_ms(fn, launches, repeats=5):
    """Average duration of one launch when `launches` of them are queued back to back between one pair of
    HIP events (the event pair's own overhead, about 2 us per launch when every launch is bracketed, is
    amortised; this is the figure a kernel trace reports)."""
    import torch
    out = []
    for _ in range(repeats):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(launches):
            fn()
        e.record()
        torch.cuda.synchronize()
        out.append(s.elapsed_time(e) / launches)
    return out


def bench_config1(args, ops, O, wl, steps, warmup):
    """Returns (headline dict, per-op entries)."""
    import torch
    c = wl.make_config(1)
    x = to_dev(c["x"])
    out = tuple(torch.empty_like(t) for t in quad(x))
    nbytes = 16 * x["lw"].numel() + 16 * x["lb"].numel()
    calls = [(kind, p) for kind in ("relu", "tanh") for p in c["ps"]]

    def one(kind, p):
        getattr(ops, kind)(*quad(x), p, c["eps"], c["words"], out=out)

    def step():
        for kind, p in calls:
            one(kind, p)

    # the timed region of the contract: W warm-up steps, then exactly K steps between syncs
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    entries, per_kernel = [], {}
    for kind, p in calls:
        t = gpu_times_ms(lambda: one(kind, p), max(steps, 50), 5)
        per_kernel[(kind, p)] = t
        entries.append(op_entry(f"config1 {kind} p={p:g} [1,128,256,512] words=2", "hbm", t, nbytes))
    # the other relaxations on the same skeleton and the product of two objects, same shape, p = 2
    # (not among the five configurations; reciprocal and sqrt get strictly positive pre-activations)
    xp = {k: v.clone() for k, v in x.items()}       # distinct memory: the product must read both objects
    xp["lb"] = x["lb"].abs() + 2.0
    xp["ub"] = xp["lb"] + (x["ub"] - x["lb"])
    for kind, src_x in (("exp", x), ("sqr", x), ("sqrt", xp), ("reciprocal", xp)):
        t = gpu_times_ms(lambda: getattr(ops, kind)(*quad(src_x), 2.0, c["eps"], c["words"], out=out), 50, 5)
        entries.append(op_entry(f"extra: {kind} p=2 [1,128,256,512] words=2", "hbm", t, nbytes))
    t = gpu_times_ms(lambda: ops.multiply(quad(x), quad(xp), 2.0, c["eps"], c["words"], out=out), 50, 5)
    entries.append(op_entry("extra: multiply(Bounds, Bounds) p=2 [1,128,256,512] words=2", "hbm", t,
                            24 * x["lw"].numel() + 24 * x["lb"].numel()))
    # softmax over 128 key positions of four heads (the attention scores of configuration 3's shape): the
    # same bytes as a relaxation of configuration 1 -- one read and one write of lw / uw
    sx = tuple(v.reshape((4, 128, 256, 128) if v.dim() == 4 else (4, 128, 128)) for v in quad(x))
    t = gpu_times_ms(lambda: ops.softmax(*sx, 2.0, c["eps"], c["words"]), 50, 5)
    entries.append(op_entry("extra: softmax p=2 [4,128,256,128] words=2 (exp, sum, reciprocal, product in one launch)", "hbm",
                            t, nbytes))
    # random contents: a buffer of zeros streams about 15 % faster on this part, which flatters a yardstick
    src = torch.randn(nbytes // 8, device="cuda")
    dst = torch.empty_like(src)
    from faith_amd import _lib
    st = torch.cuda.current_stream().cuda_stream
    tc = gpu_times_ms(lambda: _lib.call("faith_copy_f32", src.data_ptr(), dst.data_ptr(), src.numel(), st), 50, 5)
    entries.append(op_entry("plain copy of the same byte count (yardstick, not a bound op)", "hbm", tc, nbytes))

    # Two instantiations of one kernel share a step evenly (relu: eight wavefronts, two workgroups per CU; tanh: three
    # per CU).  `roofline` is the slower of the two (its slowest norm); the other is quoted under "also".
    slowest = {kind: max((k for k in per_kernel if k[0] == kind), key=lambda k: statistics.mean(per_kernel[k]))
               for kind in ("relu", "tanh")}
    dom = max(slowest.values(), key=lambda k: statistics.mean(per_kernel[k]))
    other = slowest["tanh" if dom[0] == "relu" else "relu"]
    avg_ms = statistics.mean(gpu_back_to_back_ms(lambda: one(*dom), 20))
    other_ms = statistics.mean(gpu_back_to_back_ms(lambda: one(*other), 20))
    traffic = traffic_from_profile()
    kernel_of = {"relu": "act_resident", "tanh": "act_resident"}
    kernel = kernel_of[dom[0]]
    roofline = {"bound": "hbm", "kernel": f"{kernel}<{dom[0]}, p={dom[1]:g}>",
                "achieved": round(nbytes / avg_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(nbytes / avg_ms / 1e6 / HBM_PEAK_GBS, 4),
                "avg_launch_us": round(avg_ms * 1e3, 2), "bytes_per_launch": nbytes,
                "traffic": traffic.get((dom[0], "warm")),
                "also": {"kernel": f"{kernel_of[other[0]]}<{other[0]}, p={other[1]:g}>",
                         "achieved": round(nbytes / other_ms / 1e6, 1), "frac": round(nbytes / other_ms / 1e6 / HBM_PEAK_GBS, 4),
                         "avg_launch_us": round(other_ms * 1e3, 2), "traffic": traffic.get((other[0], "warm"))},
                "note": "the configuration as specified: one operand set (269 MB) reused by every launch, against 256 MB "
                        "of Infinity Cache; roofline_cold cycles disjoint sets"}

    # Cold: the same launches over COLD_SETS disjoint operand and result sets, so that 1.35 GB pass
    # through the memory system before any byte is touched again and nothing is served from the 256 MB
    # Infinity Cache.  Same kernel, same bytes per launch.
    sets = [(x, out)] + [({k: v.clone() for k, v in x.items()}, tuple(torch.empty_like(t) for t in out))
                         for _ in range(COLD_SETS - 1)]
    turn = [0]

    def one_cold(kind, p):
        xs, os_ = sets[turn[0] % COLD_SETS]
        turn[0] += 1
        getattr(ops, kind)(*quad(xs), p, c["eps"], c["words"], out=os_)

    cold_entries = {}
    streaming = {}
    for kind in ("relu", "tanh"):
        for _ in range(2 * COLD_SETS):
            one_cold(kind, dom[1])
        cold_ms = statistics.mean(gpu_back_to_back_ms(lambda: one_cold(kind, dom[1]), 4 * COLD_SETS))
        cold_entries[kind] = cold_ms
        entries.append(op_entry(f"config1 {kind} p={dom[1]:g} COLD: {COLD_SETS} disjoint operand sets in turn "
                                f"({COLD_SETS * nbytes / 1e9:.2f} GB between reuses), average of back-to-back launches",
                                "hbm", [cold_ms], nbytes))
        # the one-tile kernel with sixteen wavefronts and non-temporal loads (what every relaxation takes by itself for
        # objects that cannot be cache resident, more than 576 MB of traffic), forced here through the tuning knob
        _lib.call("faith_tune_set", 0, 7)
        try:
            for _ in range(2 * COLD_SETS):
                one_cold(kind, dom[1])
            streaming[kind] = statistics.mean(gpu_back_to_back_ms(lambda: one_cold(kind, dom[1]), 4 * COLD_SETS))
        finally:
            _lib.call("faith_tune_set", 0, 0)
        entries.append(op_entry(f"config1 {kind} p={dom[1]:g} COLD, one-tile kernel shaped for HBM streams forced (tuning knob)",
                                "hbm", [streaming[kind]], nbytes))
    srcs = [torch.randn(nbytes // 8, device="cuda") for _ in range(COLD_SETS)]
    dsts = [torch.empty_like(t) for t in srcs]

    def copy_cold():
        i = turn[0] % COLD_SETS
        turn[0] += 1
        _lib.call("faith_copy_f32", srcs[i].data_ptr(), dsts[i].data_ptr(), srcs[i].numel(), st)
    for _ in range(2 * COLD_SETS):
        copy_cold()
    copy_cold_ms = statistics.mean(gpu_back_to_back_ms(copy_cold, 4 * COLD_SETS))
    entries.append(op_entry(f"plain copy of the same byte count COLD ({COLD_SETS} disjoint buffer pairs in turn; yardstick)",
                            "hbm", [copy_cold_ms], nbytes))
    del srcs, dsts
    cold_ms = cold_entries[dom[0]]
    roofline_cold = {"bound": "hbm", "kernel": roofline["kernel"], "achieved": round(nbytes / cold_ms / 1e6, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(nbytes / cold_ms / 1e6 / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(cold_ms * 1e3, 2), "bytes_per_launch": nbytes,
                     "traffic": traffic.get((dom[0], "cold")), "operand_sets": COLD_SETS,
                     "also": {"kernel": f"{kernel_of[other[0]]}<{other[0]}, p={dom[1]:g}>",
                              "achieved": round(nbytes / cold_entries[other[0]] / 1e6, 1),
                              "frac": round(nbytes / cold_entries[other[0]] / 1e6 / HBM_PEAK_GBS, 4),
                              "avg_launch_us": round(cold_entries[other[0]] * 1e3, 2),
                              "traffic": traffic.get((other[0], "cold"))},
                     "plain_copy_cold_frac": round(nbytes / copy_cold_ms / 1e6 / HBM_PEAK_GBS, 4),
                     "frac_with_streaming_thread_shape": round(nbytes / streaming[dom[0]] / 1e6 / HBM_PEAK_GBS, 4)}
    del sets

    cpu = None
    if not args.no_cpu:
        xo = O.LinearBounds(*quad(c["x"]))

        def cpu_step():
            for kind, p in calls:
                getattr(O, kind)(xo, p, c["eps"], c["words"])
        getattr(O, "relu")(xo, 2.0, c["eps"], c["words"])      # warm the allocator
        s = cpu_time_s(cpu_step, reps=2)
        cpu = {"value": round(len(calls) * nbytes / s / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
               "cpu_model": cpu_model(), "kind": "port", "sec_per_step": round(s, 3),
               "sample": "2 full steps (6 calls each) on the identical tensors, median"}
    head = {"value": round(len(calls) * nbytes / ms_per_step / 1e6, 1), "ms_per_step": round(ms_per_step, 4),
            "roofline": roofline, "roofline_cold": roofline_cold, "cpu_baseline": cpu,
            "bytes_per_step": len(calls) * nbytes}
    return head, entries


def run_cold_only(ops, wl):
    """For counter runs (rocprofv3 --pmc ...): nothing but cold launches of the configuration-1 relaxations
    (p = inf) and of the plain copy, each over COLD_SETS disjoint operand sets in turn, so that the per-kernel
    averages of the counters are those of launches that find nothing in the Infinity Cache."""
    import torch
    from faith_amd import _lib
    c = wl.make_config(1)
    x = to_dev(c["x"])
    sets = [({k: v.clone() for k, v in x.items()}, tuple(torch.empty_like(t) for t in quad(x))) for _ in range(COLD_SETS)]
    srcs = [torch.randn(x["lw"].numel() * 2, device="cuda") for _ in range(COLD_SETS)]
    dsts = [torch.empty_like(t) for t in srcs]
    st = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    n = 0
    for rnd in range(4):
        for i in range(COLD_SETS):
            xs, os_ = sets[i]
            ops.relu(*quad(xs), INF, c["eps"], c["words"], out=os_)
        for i in range(COLD_SETS):
            xs, os_ = sets[i]
            ops.tanh(*quad(xs), INF, c["eps"], c["words"], out=os_)
        for i in range(COLD_SETS):
            _lib.call("faith_copy_f32", srcs[i].data_ptr(), dsts[i].data_ptr(), srcs[i].numel(), st)
        n += 3 * COLD_SETS
    torch.cuda.synchronize()
    print(json.dumps({"cold_only": True, "launches": n, "operand_sets": COLD_SETS}), flush=True)


def bench_config2(args, ops, O, wl):
    import torch
    c = wl.make_config(2)
    x, W, b = to_dev(c["x"]), c["W"].cuda(), c["bias"].cuda()
    L, D, H, N = 256, 512, 1024, 1024
    out = (torch.empty(1, L, D, N, device="cuda"), torch.empty(1, L, N, device="cuda"),
           torch.empty(1, L, D, N, device="cuda"), torch.empty(1, L, N, device="cuda"))
    flop = 4 * 2 * (L * D + L) * H * N
    n = 10 if args.profile else 100
    t = gpu_times_ms(lambda: ops.linear(*quad(x), W, b, out=out), n, 2)
    tc = gpu_times_ms(lambda: ops.concretize(*out, c["p"], c["eps"], 1), n, 2)
    cpu = None
    if not args.no_cpu:
        # bounded sample: L = 32 of 256 rows (1/8 of the work), same D_in, H, N
        xs = O.LinearBounds(*(t_[:, :32] for t_ in quad(c["x"])))
        s = cpu_time_s(lambda: O.linear(xs, c["W"], c["bias"]), reps=3, warmup=1)
        cpu = {"value": round(flop / 8 / s / 1e12, 4), "unit": "TFLOP/s", "sample": "L=32 of 256 rows, median of 3",
               "sec_full_size_est": round(s * 8, 2)}
    e = op_entry("config2 linear [1,256,512,1024]x[1024,1024]", "mfma", t, flop, cpu, form="linear")
    e2 = op_entry("config2 concretize(p=2) of the result", "hbm", tc, 8 * L * D * N + 16 * L * N)
    # layer and dual norm through one entry point: the tiled kernel folds the column norms into its epilogue and
    # writes l, u itself, the result is not read again
    lu = (torch.empty(1, L, N, device="cuda"), torch.empty(1, L, N, device="cuda"))
    tf = gpu_times_ms(lambda: ops.linear_concretize(*quad(x), W, b, c["p"], c["eps"], 1, out=(*out, *lu)), n, 2)
    e3 = op_entry("config2 linear + concretize(p=2) in one call (column norms in the GEMM epilogue)", "mfma", tf, flop,
                  None, form="linear", extra={"separately_us": round((statistics.median(t) + statistics.median(tc)) * 1e3, 1)})
    return [e, e2, e3]


def bench_config3(args, ops, O, wl):
    import torch
    c = wl.make_config(3)
    x, y = to_dev(c["x"]), to_dev(c["y"])
    B, L, D, d = 4, 128, 256, 64
    out = (torch.empty(B, L, D, L, device="cuda"), torch.empty(B, L, L, device="cuda"),
           torch.empty(B, L, D, L, device="cuda"), torch.empty(B, L, L, device="cuda"))
    flop = B * (8 * 2 * L * D * d * L + 8 * 2 * L * d * L)
    t = gpu_times_ms(lambda: ops.dot_product_qk(quad(x), quad(y), c["p"], c["eps"], 1, out=out), 50, 5)
    cpu = None
    if not args.no_cpu:
        xo, yo = O.LinearBounds(*quad(c["x"])), O.LinearBounds(*quad(c["y"]))
        s = cpu_time_s(lambda: O.dot_product(xo, yo, c["p"], c["eps"]), reps=3, warmup=1)
        cpu = {"value": round(flop / s / 1e12, 4), "unit": "TFLOP/s", "sample": "full size, median of 3",
               "latency_ms": round(s * 1e3, 1)}
    e = op_entry("config3 dot_product QK 4 heads [4,128,256,64] (concretize + planes + contraction)",
                 "mfma", t, flop, cpu, form="dot")
    # the second half of attention on the same shapes (not one of the five configurations): context =
    # probabilities [4,128,256,128] . values [4,128,256,64]; the scores bounds just computed serve as
    # the probability operand
    probs = tuple(out)
    outv = (torch.empty(B, L, D, d, device="cuda"), torch.empty(B, L, d, device="cuda"),
            torch.empty(B, L, D, d, device="cuda"), torch.empty(B, L, d, device="cuda"))
    flopv = B * (8 * 2 * L * D * L * d + 8 * 2 * L * L * d)
    tv = gpu_times_ms(lambda: ops.dot_product_v(probs, quad(y), c["p"], c["eps"], 1, out=outv), 50, 5)
    ev = op_entry("extra: context (probs.value) 4 heads [4,128,256,128].[4,128,256,64]", "mfma", tv, flopv, form="dot")
    # the same scores through the reference's own calling convention: operands [B, L, dim_out, dim_in], result
    # [B, Lx, Ly, dim_in] (MFMA with the operands straight from that layout: y terms per column j, x terms per row i)
    from faith_amd import c_bound
    T = lambda t_: t_.transpose(2, 3).contiguous()
    xt, yt = (T(x["lw"]), T(x["uw"])), (T(y["lw"]), T(y["uw"]))
    scr = [torch.empty(B, L, d, device="cuda") for _ in range(4)]
    zt = (torch.empty(B, L, L, device="cuda"), torch.empty(B, L, L, device="cuda"),
          torch.empty(B, L, L, D, device="cuda"), torch.empty(B, L, L, D, device="cuda"))
    c_bound.p, c_bound.words = c["p"], 1
    tt = gpu_times_ms(lambda: c_bound.c_dot_product_verification_QK(*scr, x["lb"], x["ub"], y["lb"], y["ub"], xt[0], xt[1],
                                                                    yt[0], yt[1], *zt, B, L, d, D, c["eps"]), 50, 5)
    c_bound.p = 2.0
    et = op_entry("extra: config3 scores in the reference's transposed layout (c_bound.c_dot_product_verification_QK: "
                  "concretize + constant terms + y-term and x-term MFMA launches)", "mfma", tt, flop, form="dot")
    return [e, ev, et]


def bench_config4(args, ops, O, wl):
    import torch
    c = wl.make_config(4)
    x, W, b = to_dev(c["x"]), c["W"].cuda(), c["bias"].cuda()
    D, Ci, Co, Hh = 256, 64, 128, 32
    out = (torch.empty(1, D, Co, Hh, Hh, device="cuda"), torch.empty(1, Co, Hh, Hh, device="cuda"),
           torch.empty(1, D, Co, Hh, Hh, device="cuda"), torch.empty(1, Co, Hh, Hh, device="cuda"))
    flop = 4 * 2 * (D + 1) * Co * Hh * Hh * Ci * 9
    n = 10 if args.profile else 100
    t = gpu_times_ms(lambda: ops.conv2d(*quad(x), W, b, 1, 1, out=out), n, 2)
    tc = gpu_times_ms(lambda: ops.concretize_conv(*out, c["p"], c["eps"]), n, 2)
    cpu = None
    if not args.no_cpu:
        xs = O.LinearBounds(c["x"]["lw"][:, :32], c["x"]["lb"], c["x"]["uw"][:, :32], c["x"]["ub"])
        s = cpu_time_s(lambda: O.conv2d(xs, c["W"], c["bias"], 1, 1), reps=3, warmup=1)
        cpu = {"value": round(4 * 2 * 33 * Co * Hh * Hh * Ci * 9 / s / 1e12, 4), "unit": "TFLOP/s",
               "sample": "D_in=32 of 256, median of 3"}
    e = op_entry("config4 conv3x3 64->128 [1,256,64,32,32]", "mfma", t, flop, cpu, form="conv")
    e2 = op_entry("config4 concretize(p=inf) of the result", "hbm", tc, 8 * D * Co * Hh * Hh + 16 * Co * Hh * Hh)
    out_entries = [e, e2]
    # the other layer shapes of a CNN verifier, same D_in = 256 and 32 x 32 input (not among the five configurations):
    # each takes a straight-line instantiation of the implicit-GEMM kernel with the tile that fits its result
    del out
    g = torch.Generator().manual_seed(1404)
    for (ci, co, k, s_, p_, what) in ((64, 128, 3, 2, 1, "3x3 stride 2 64->128"), (64, 128, 1, 1, 0, "1x1 64->128"),
                                      (32, 64, 5, 1, 2, "5x5 32->64"), (3, 64, 3, 1, 1, "3x3 3->64 (first layer)")):
        lw = (torch.randn(1, D, ci, Hh, Hh, generator=g) * 0.05).cuda()
        uw = lw + 0.005
        lb = torch.randn(1, ci, Hh, Hh, generator=g).cuda()
        ub = lb + 0.1
        Wk = (torch.randn(co, ci, k, k, generator=g) * (2.0 / (ci * k * k)) ** 0.5).cuda()
        ho = (Hh + 2 * p_ - k) // s_ + 1
        o_ = ops.conv2d(lw, lb, uw, ub, Wk, None, s_, p_)
        tk = gpu_times_ms(lambda: ops.conv2d(lw, lb, uw, ub, Wk, None, s_, p_, out=o_), 10 if args.profile else 50, 2)
        fl = 4 * 2 * (D + 1) * co * ho * ho * ci * k * k
        out_entries.append(op_entry(f"extra: conv {what} [1,256,{ci},32,32]", "mfma", tk, fl, None, form="conv", extra=
                                    {"result_write_GBs": round(2 * D * co * ho * ho * 4 / statistics.median(tk) / 1e6, 1)}))
        del lw, uw, o_
    return out_entries


def bench_sub_blocks(args, rows, hidden, inter):
    """The encoder sub-blocks of the batched propagation as single operators, at its size (rows positions of dim_in =
    hidden): dense + residual + layer norm and dense + ReLU in one pass over the coefficients, beside the separate
    launches they replace.  TFLOP/s count the layer's two executed products per term."""
    import torch
    from faith_amd import ops
    g = torch.Generator().manual_seed(78)
    n = 5 if args.profile else 20
    out = []

    def obj(width):
        lw = (torch.randn(1, rows, hidden, width, generator=g) * 0.05).cuda()
        lb = torch.randn(1, rows, width, generator=g).cuda()
        return lw, lb, lw + 0.005, lb + 0.1
    for what, K, N in (("attention output", hidden, hidden), ("feed-forward output", inter, hidden)):
        x, r = obj(K), obj(N)
        W, b = (torch.randn(N, K, generator=g) / K ** 0.5).cuda(), (0.05 * torch.randn(N, generator=g)).cuda()
        w, sh = (1.0 + 0.1 * torch.randn(N, generator=g)).cuda(), (0.05 * torch.randn(N, generator=g)).cuda()
        fused = gpu_times_ms(lambda: ops.linear_layer_norm(*x, W, b, w, sh, r), n, 2)
        apart = gpu_times_ms(lambda: ops.layer_norm(*ops.linear(*x, W, b), w, sh, r), n, 2)
        out.append(op_entry(f"extra: dense {K}->{N} + residual + layer norm (no_var) in one pass, {what} of the batched "
                            f"propagation [1,{rows},{hidden},{K}]", "mfma", fused, 4 * 2 * rows * (hidden + 1) * K * N,
                            form="linear", extra={"separate_launches_us": round(statistics.median(apart) * 1e3, 1)}))
        del x, r
    x = obj(hidden)
    W, b = (torch.randn(inter, hidden, generator=g) / hidden ** 0.5).cuda(), (0.05 * torch.randn(inter, generator=g)).cuda()
    fused = gpu_times_ms(lambda: ops.linear_relu(*x, W, b, 2.0, 0.01), n, 2)
    apart = gpu_times_ms(lambda: ops.relu(*ops.linear(*x, W, b), 2.0, 0.01), n, 2)
    out.append(op_entry(f"extra: dense {hidden}->{inter} + ReLU (p=2) in one pass, feed-forward input of the batched "
                        f"propagation [1,{rows},{hidden},{hidden}]", "mfma", fused, 4 * 2 * rows * (hidden + 1) * hidden * inter,
                        form="linear", extra={"separate_launches_us": round(statistics.median(apart) * 1e3, 1)}))
    return out


def bench_layer(args, wl):
    """The path as its caller uses it: one encoder layer + pooler + margin classifier propagated by
    faith_amd/forward.py (about 30 kernel launches), at a small-BERT size.  Wall clock, host included."""
    import time
    import torch
    from types import SimpleNamespace
    from faith_amd import BoundsMaker, forward as F, ops
    hidden, heads, inter, length, eps, p = 256, 4, 512, 32, 0.01, 2.0
    g = torch.Generator().manual_seed(77)
    layer = wl.random_layer(g, hidden, heads, inter)
    norm = SimpleNamespace(weight=1.0 + 0.1 * torch.randn(hidden, generator=g), bias=0.05 * torch.randn(hidden, generator=g))
    pooler = SimpleNamespace(weight=torch.randn(hidden, hidden, generator=g) / hidden ** 0.5, bias=0.05 * torch.randn(hidden, generator=g))
    clf = SimpleNamespace(weight=torch.randn(2, hidden, generator=g) / hidden ** 0.5, bias=0.05 * torch.randn(2, generator=g))
    emb = torch.randn(1, length, hidden, generator=g)

    def run(make, parts, e):
        lay, nrm, pool, cl = parts
        x = F.bound_input(make, e, 3, eps, 1, p, nrm, "no_var")
        _, _, out = F.bound_layer(x, lay, "no_var", "relu")
        return F.bound_classifier(F.bound_pooling(out, pool, make), cl, 0)

    gparts = tuple(wl.to_device(x, "cuda") for x in (layer, norm, pooler, clf))
    # the maker that lets the input builders leave out the zero coefficient rows of the positions that are not
    # perturbed where that pays (here: the batched propagation; the single query is written out at once)
    gmake = BoundsMaker()
    ge = emb.cuda()
    net = SimpleNamespace(embedding_norm=gparts[1], layers=[gparts[0]], pooler=gparts[2], classifier=gparts[3],
                          layer_norm="no_var", hidden_act="relu")
    if args.layer_only:
        # under a profiler: ten batched propagations of the sentence's 30 positions and nothing else
        positions = list(range(1, length - 1))
        for _ in range(10):
            F.verify_safety_batch(gmake, net, ge, positions, [eps] * len(positions), 0, p)
        torch.cuda.synchronize()
        return []
    single = lambda: F.verify_safety(gmake, net, ge, 3, eps, 0, p)      # ends with the verdict on the host
    t0 = time.time()
    while time.time() - t0 < max(WARM_SECONDS, 0.05):
        single()
    torch.cuda.synchronize()
    times = []
    for _ in range(10):
        t0 = time.perf_counter()
        single()
        times.append((time.perf_counter() - t0) * 1e3)
    e = {"op": f"extra: encoder layer + pooler + classifier, hidden {hidden}, {heads} heads, FFN {inter}, L={length}, "
               f"one perturbed word, p=2 (forward.verify_safety, wall clock)",
         "latency_us": round(statistics.median(times) * 1e3, 1), "latency_min_us": round(min(times) * 1e3, 1),
         "bound": "host", "achieved": 0.0, "peak": 1.0, "unit": "-", "frac": 0.0, "work": 0}
    # the same query with the caller keeping every result buffer across calls (ops.Workspace): no allocation per call
    ws = ops.Workspace()
    kept = lambda: F.verify_safety(gmake, net, ge, 3, eps, 0, p, buffers=ws)
    for _ in range(20):
        kept()
    times = []
    for _ in range(10):
        t0 = time.perf_counter()
        kept()
        times.append((time.perf_counter() - t0) * 1e3)
    e["latency_us_with_persistent_buffers"] = round(statistics.median(times) * 1e3, 1)
    del ws
    if not args.no_cpu:
        from tests.oracle_bounds import OracleBounds            # cpu_baseline leg only
        omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
        s = cpu_time_s(lambda: run(omake, (layer, norm, pooler, clf), emb), reps=2, warmup=1)
        e["cpu_baseline"] = {"latency_ms": round(s * 1e3, 1), "cores": torch.get_num_threads(), "kind": "port",
                             "sample": "the same layer on the CPU oracle, median of 2"}

    # the caller's loop: one bisection step for every perturbable position of the sentence
    # (Verifier.verify), as one propagation with a batch element per position
    positions = list(range(1, length - 1))
    radii = [eps] * len(positions)
    step = lambda: F.verify_safety_batch(gmake, net, ge, positions, radii, 0, p)
    t0 = time.time()
    while time.time() - t0 < max(WARM_SECONDS, 0.05):
        step()
    times = []
    for _ in range(10):
        t0 = time.perf_counter()
        step()                                                   # ends with the verdicts on the host
        times.append((time.perf_counter() - t0) * 1e3)
    per = statistics.median(times) * 1e3 / len(positions)
    e2 = {"op": f"extra: the same network, one bisection step of all {len(positions)} positions as one batched "
                f"propagation (forward.verify_safety_batch, input coefficients held for the perturbed positions only, "
                f"wall clock per (position, radius))",
          "latency_us": round(per, 1), "latency_min_us": round(min(times) * 1e3 / len(positions), 1),
          "bound": "host", "achieved": 0.0, "peak": 1.0, "unit": "-", "frac": 0.0, "work": 0,
          "batch_latency_us": round(statistics.median(times) * 1e3, 1)}
    # the same step with the input object written out in full (zero coefficient rows included), as the reference builds it
    from faith_amd import Bounds
    plain = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    for _ in range(3):
        F.verify_safety_batch(plain, net, ge, positions, radii, 0, p)
    times = []
    for _ in range(10):
        t0 = time.perf_counter()
        F.verify_safety_batch(plain, net, ge, positions, radii, 0, p)
        times.append((time.perf_counter() - t0) * 1e3)
    e2["batch_latency_us_with_the_zero_rows_written_out"] = round(statistics.median(times) * 1e3, 1)

    # the same two, replayed from a HIP graph captured once (forward.CapturedVerifier)
    out = [e, e2]
    out.extend(bench_sub_blocks(args, len(positions) * length, hidden, inter))
    for batch, pos in ((1, [3]), (len(positions), positions)):
        cap = F.CapturedVerifier(gmake, net, ge, batch, 0, p)
        rr = [eps] * batch
        t0 = time.time()
        while time.time() - t0 < max(WARM_SECONDS, 0.05):
            cap(pos, rr)
        times = []
        for _ in range(10):
            t0 = time.perf_counter()
            cap(pos, rr)
            times.append((time.perf_counter() - t0) * 1e3)
        out.append({"op": f"extra: the same network from a captured HIP graph, {batch} (position, radius) per replay "
                          f"(wall clock per pair, input update and verdict readback included)",
                    "latency_us": round(statistics.median(times) * 1e3 / batch, 1),
                    "latency_min_us": round(min(times) * 1e3 / batch, 1), "bound": "host", "achieved": 0.0, "peak": 1.0,
                    "unit": "-", "frac": 0.0, "work": 0})
        del cap
    return out


def measured_mfma_clock_mhz(compute_units):
    """Median shader clock over all workgroups while every SIMD issues fp32 MFMAs (about 2 ms)."""
    import torch
    from faith_amd import _lib
    n = 2 * compute_units
    out = torch.zeros(n, device="cuda")
    stream = torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())
    for _ in range(3):                       # the first launches after idle run at lower clocks
        _lib.call("faith_mfma_clock", out.data_ptr(), n, 2000, stream)
    torch.cuda.synchronize()
    return float(out.median())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only-headline", action="store_true", help="skip configurations 0, 2, 3, 4")
    ap.add_argument("--configs", default="0,2,3,4", help="extra configurations to report under 'ops'")
    ap.add_argument("--cold-only", action="store_true",
                    help="for counter runs: only cold launches of the configuration-1 relaxations and of the plain copy")
    ap.add_argument("--layer-only", action="store_true",
                    help="for runs under rocprofv3: ten batched propagations of the encoder layer (30 positions each), no timing")
    ap.add_argument("--profile", action="store_true",
                    help="for runs under rocprofv3: warm up by count only, so the trace stays small")
    args = ap.parse_args()
    if args.profile:
        global WARM_SECONDS
        WARM_SECONDS = 0.05
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; every op is independent across the length axis and "
              "nothing here uses a second GPU, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    torch.set_num_threads(min(16, os.cpu_count() or 1))
    from faith_amd import ops, workloads as wl
    O = None
    if not args.no_cpu:
        from oracle import bounds_oracle as O     # cpu_baseline leg only

    if args.cold_only:
        run_cold_only(ops, wl)
        return
    if args.layer_only:
        print(json.dumps({"ops": bench_layer(args, wl)}))
        return

    prop = torch.cuda.get_device_properties(0)
    clock_mhz = measured_mfma_clock_mhz(prop.multi_processor_count)
    peak_here = prop.multi_processor_count * 256 * clock_mhz * 1e-6        # 256 fp32 MFMA flop / clock / CU
    log(f"device: {prop.name}, {prop.multi_processor_count} CUs, host: {cpu_model()}, {torch.get_num_threads()} threads; shader clock "
        f"under MFMA load {clock_mhz:.0f} MHz -> fp32 MFMA peak at that clock {peak_here:.1f} TFLOP/s "
        f"(roofline fractions below use the published {MFMA_FP32_PEAK_TFLOPS} TFLOP/s)")

    head, entries = bench_config1(args, ops, O, wl, args.steps, args.warmup)
    extra = set() if args.only_headline else {int(c) for c in args.configs.split(",") if c.strip()}
    if 0 in extra:
        entries = [bench_config0(args, ops, O, wl)] + entries
        if not args.profile:
            entries += bench_notebook_shapes(args, ops, O)
    if 2 in extra:
        entries += bench_config2(args, ops, O, wl)
    if 3 in extra:
        entries += bench_config3(args, ops, O, wl)
    if 4 in extra:
        entries += bench_config4(args, ops, O, wl)
    if extra and not args.profile:
        entries.extend(bench_layer(args, wl))

    for e in entries:
        cb = e.get("cpu_baseline")
        rf = e.get("reference_formulation")
        log(f"{e['op']:<90s} {e['latency_us']:>10.1f} us  {e['achieved']:>9.1f} {e['unit']:<8s} "
            f"{100 * e['frac']:5.1f}% of {e['peak']:g}"
            + (f"   ({rf['tflops']:.1f} TFLOP/s in the reference's formulation)" if rf else "")
            + (f"   cpu: {cb}" if cb else ""))

    # the five configurations' dominant kernels inside `roofline` (the record that is kept whole): latency of the
    # operator, the roofline that bounds it, the fraction reached (contractions: products executed, see EXECUTED)
    def cfg_entry(prefix, kernel):
        for e in entries:
            if e["op"].startswith(prefix):
                return {"kernel": kernel, "avg_us": e["latency_us"], "bound": e["bound"], "achieved": e["achieved"],
                        "unit": e["unit"], "frac": e["frac"]}
        return None
    per_config = {
        "0": cfg_entry("config0", "signsplit_gemm_concretize_short<inf, 4> (layer + dual norm, one launch; latency bound)"),
        "1": {"kernel": head["roofline"]["kernel"], "avg_us": head["roofline"]["avg_launch_us"], "bound": "hbm",
              "achieved": head["roofline"]["achieved"], "unit": "GB/s", "frac": head["roofline"]["frac"],
              "cold_frac": head["roofline_cold"]["frac"]},
        "2": cfg_entry("config2 linear [", "signsplit_gemm<true>"),
        "3": cfg_entry("config3 dot_product", "dot_tiled<false, 8> + concretize + constant terms (whole operator)"),
        "4": cfg_entry("config4 conv3x3", "conv_signsplit_k3s1 + constant terms (whole operator)"),
    }
    head["roofline"]["per_config"] = {k: v for k, v in per_config.items() if v is not None}

    line = {
        "metric": METRIC, "value": head["value"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config1: relu+tanh relaxation, lw/uw [1,128,256,512], words=2, eps=0.01, "
                               "p in {1,2,inf} (6 launches per step)",
                   "bytes_per_step": head["bytes_per_step"], "device": prop.name,
                   "compute_units": prop.multi_processor_count, "shader_clock_mhz_under_mfma_load": round(clock_mhz, 1),
                   "fp32_mfma_peak_at_measured_clock_tflops": round(peak_here, 1)},
        "roofline": head["roofline"], "roofline_cold": head["roofline_cold"], "cpu_baseline": head["cpu_baseline"],
        "ops": entries,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
