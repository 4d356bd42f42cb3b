#!/usr/bin/env python3
"""Benchmark of the log-space contraction path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one ``lt2exp`` call on the large configuration (R=64, S=I=J=64, K=4096,
fp32, seeded synthetic inputs already resident in HBM).  An untimed pre-conditioning
phase of the same call (250 ms, reported as ``prewarm_ms``), W untimed steps, then
exactly K steps bracketed by ``torch.cuda.synchronize()``; rank 0 prints ONE
JSON line on stdout (progress goes to stderr).  The same line carries

  roofline      fp32-MFMA roofline of the dominant kernel: algorithmic flops per
                launch / average launch duration from HIP events recorded on the
                launch stream around the timed region;
  cpu_baseline  the reference's torch recipe (restated in oracle/torch_baseline.py)
                timed on this host's cores on a bounded sample of the same workload;
  lm2exp, c2, c4, max
                the other kernels and configurations of the path, each measured the
                same way (lm2exp R=64, I=J=256, K=4096; lm2exp R=16, I=J=K=512;
                lt2exp R=16, S=64, I=J=32, K=2048; matmax / vmax on the 64x64x4096
                operand), with their own roofline objects.

``--back-to-back`` runs the four contraction regions only (prewarm, warm-up, timed steps:
every launch of a contraction kernel back to back on one stream) -- the run a kernel trace
is taken over, so that the trace's average launch duration is that of the timed launches.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

PEAK_FP32_MFMA_TFLOPS = 157.3  # 256 CU x 4 SIMD x 64 flop/clk x 2.4 GHz
PEAK_HBM_GBPS = 8000.0
PEAK_BF16_MFMA_TFLOPS = 2516.6  # 16x the fp32 matrix rate

# HBM bytes per launch come from the committed counter summary (rocprofv3 --pmc FETCH_SIZE, then
# WRITE_SIZE, one run each over `bench.py --profile-pass`, scaled by what the same counters read for
# trt_copy_bytes of 256 MiB): the row of the kernel that this run times, looked up by the name
# the library reports for the call.  No row for that kernel: the bench stops and says so.
COUNTER_SUMMARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                               "lt2exp_lm2exp_max_counters.md")
PREWARM_MS = 250.0  # untimed launches of the same call before the warm-up steps (clock / power settle)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def measured_traffic_bytes(kernel: str) -> float:
    """HBM bytes per launch of `kernel` from the 'total MB' column of the counter summary."""
    with open(COUNTER_SUMMARY) as f:
        rows = [ln for ln in f if ln.startswith("| `")]
    for ln in rows:
        cells = [c.strip() for c in ln.strip().strip("|").split("|")]
        if cells[0].strip("`") == kernel and len(cells) >= 7:
            return float(cells[5]) * 1e6
    raise SystemExit(
        f"bench.py: {COUNTER_SUMMARY} has no HBM-traffic row for the kernel this run times, `{kernel}`: "
        "regenerate the counter summary (the commands are in that file) before quoting a roofline")


_burn = {}


def clock_burn(ms: float = 200.0):
    """Keeps the GPU busy with an unrelated kernel (torch.mm) for `ms`: after a host-bound phase
    (input generation) the engine clock has dropped, and the first launches of whatever runs
    next are 15-25 % slow.  Used by --back-to-back only, so that every launch of a contraction
    kernel that a trace of the run records -- not only the timed ones -- runs at speed."""
    if not _burn:
        _burn["x"] = torch.randn(4096, 4096, device="cuda")
        _burn["y"] = torch.empty(4096, 4096, device="cuda")
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(10):
            torch.mm(_burn["x"], _burn["x"], out=_burn["y"])
        torch.cuda.synchronize()


def timed_region(fn, steps: int, warmup: int, per_launch: bool = True, prewarm_fn=None):
    """Times exactly `steps` calls: {wall_s, event_s} over the whole region (HIP events recorded on
    the launch stream) and the median / q10 / q90 of per-call HIP-event times from a second pass of
    the same length.  Before the warm-up steps the call is repeated, untimed, for PREWARM_MS so
    that a short region does not measure the clock and power transient left by what ran before."""
    pre = prewarm_fn or fn
    if not per_launch:
        clock_burn()
    pre()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_pre = 0
    while (time.perf_counter() - t0) * 1e3 < PREWARM_MS:
        for _ in range(8):
            pre()
        torch.cuda.synchronize()
        n_pre += 8
    prewarm_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()  # on the current stream: the stream the kernels are launched on
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev = start.elapsed_time(stop) * 1e-3
    if not per_launch:
        return {"wall_s": wall, "event_s": ev, "median_ms": None, "q10_ms": None, "q90_ms": None,
                "prewarm_ms": round(prewarm_ms, 1), "prewarm_calls": n_pre}
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    marks[0].record()
    for i in range(steps):
        fn()
        marks[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    q = lambda f: per[min(len(per) - 1, int(f * len(per)))]
    return {"wall_s": wall, "event_s": ev, "median_ms": q(0.5), "q10_ms": q(0.1), "q90_ms": q(0.9),
            "prewarm_ms": round(prewarm_ms, 1), "prewarm_calls": n_pre}


def do_bench(fn, *, warmup_ms=150.0, rep_ms=1000.0, flush_bytes=512 << 20):
    """Median / q10 / q90 milliseconds of single calls, each preceded by a cache flush
    (the protocol of the reference's benchmarks: benchmarks/lm2exp.py:94)."""
    flush = torch.empty(flush_bytes, dtype=torch.uint8, device="cuda")
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(5):
        fn()
    e.record()
    torch.cuda.synchronize()
    est = max(s.elapsed_time(e) / 5, 1e-3)
    n_warm = max(1, int(warmup_ms / est))
    n_rep = max(5, min(2000, int(rep_ms / est)))
    for _ in range(n_warm):
        fn()
    ss = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    ee = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for i in range(n_rep):
        flush.zero_()
        ss[i].record()
        fn()
        ee[i].record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in zip(ss, ee))
    q = lambda f: ts[min(len(ts) - 1, int(f * len(ts)))]
    return {"median_ms": q(0.5), "q10_ms": q(0.1), "q90_ms": q(0.9), "reps": n_rep}


def graph_time(fn, calls: int = 20, reps: int = 20, prewarm_ms: float = 0.0, both: bool = False, operands=None):
    """Average seconds per call of a short kernel: `calls` launches captured in one HIP
    graph (no host launch gaps), replayed `reps` times between HIP events.  With `prewarm_ms`
    the graph is first replayed, untimed, for that long (as `timed_region` does): after an
    idle or host-bound phase the engine clock takes some hundred milliseconds of load to come
    up, and the streaming kernels follow it.  `both`: returns (seconds after the prewarm,
    seconds of the same measurement taken before it).  With `operands` the calls of the graph
    are fn(operands[0]), fn(operands[1]), ... in turn: enough copies of an operand that none of
    them is still in a cache when its turn comes again."""
    if operands is not None:
        n_ops = len(operands)
        calls = max(calls, n_ops) // n_ops * n_ops
        turn = iter(range(1 << 60))
        call = lambda: fn(operands[next(turn) % n_ops])
    else:
        call = fn
    # (warm-up on the launch stream itself: a kernel on a second stream displaces what the
    # read-once sweeps find in the dies' L2s from one call to the next, and vmax then runs 2 us
    # slower for the rest of the process -- not what a caller with one stream sees)
    for _ in range(3):
        fn(operands[0]) if operands is not None else fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(calls):
            call()
    g.replay()
    torch.cuda.synchronize()

    def measure() -> float:
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            g.replay()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) * 1e-3 / (calls * reps)

    before = measure() if (both or not prewarm_ms) else None
    if not prewarm_ms:
        return (before, before) if both else before
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < prewarm_ms:
        for _ in range(reps):
            g.replay()
        torch.cuda.synchronize()
    after = measure()
    return (after, before) if both else after


def profile_pass(dev) -> int:
    """Few launches of each kernel for counter collection.  The copy kernel moves a known
    number of bytes (256 MiB read + 256 MiB written), which calibrates the byte counters."""
    from ctypes import c_void_p

    from triturus_amd import _lib
    from triturus_amd import workloads as W
    from triturus_amd.lm2exp import lm2exp
    from triturus_amd.lt2exp import lt2exp
    from triturus_amd.max import matmax, vmax

    lib = _lib.load()
    nbytes = 256 << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    stream = _lib.current_stream(dev)
    for _ in range(3):
        _lib.check(lib.trt_copy_bytes(c_void_p(src.data_ptr()), c_void_p(dst.data_ptr()), nbytes, stream),
                   "trt_copy_bytes")
    torch.cuda.synchronize()
    cfg = W.c5()
    w, a, b = (cfg[k].to(dev) for k in "wab")
    for _ in range(3):
        lt2exp(w, a, b, _precision="fp32")
    for prec in ("bf16x3", "bf16x6"):
        for _ in range(3):
            lt2exp(w, a, b, _precision=prec)
    torch.cuda.synchronize()
    a1, b1 = a[:, :, :1].contiguous(), b[:, :, :1].contiguous()  # one column: the sweep over w
    for _ in range(3):
        lt2exp(w, a1, b1, _precision="fp32")
    torch.cuda.synchronize()
    # one s per batch: the rows (s, i) of w on the rows of the MFMA (101 MB of w, a, b and c)
    gen = torch.Generator().manual_seed(7)
    wf = torch.rand(2048, 1, 64, 64, generator=gen).to(dev)
    af = (torch.randn(2048, 64, 64, generator=gen) * 10 - 30).to(dev)
    bf = (torch.randn(2048, 64, 64, generator=gen) * 10 - 30).to(dev)
    for _ in range(3):
        lt2exp(wf, af, bf, _precision="fp32")
    torch.cuda.synchronize()
    del wf, af, bf
    # few units over many batches: a lane per output column (405 MB of w, a, b and c)
    wf = torch.rand(8192, 4, 4, 4, generator=gen).to(dev)
    af = (torch.randn(8192, 4, 1024, generator=gen) * 10 - 30).to(dev)
    bf = (torch.randn(8192, 4, 1024, generator=gen) * 10 - 30).to(dev)
    for _ in range(3):
        lt2exp(wf, af, bf, _precision="fp32")
    torch.cuda.synchronize()
    del wf, af, bf
    flat = b.view(-1)
    for _ in range(3):
        vmax(flat)
        matmax(b.view(4096, 4096), 0)
        matmax(b.view(4096, 4096), 1)
    torch.cuda.synchronize()
    del w, a, b
    cfg3 = W.c3()
    a3, b3 = cfg3["a"].to(dev), cfg3["b"].to(dev)
    for _ in range(3):
        lm2exp(a3, b3, _precision="fp32")
    for prec in ("bf16x3", "bf16x6"):
        for _ in range(3):
            lm2exp(a3, b3, _precision=prec)
    torch.cuda.synchronize()
    del a3, b3
    c2 = W.c2()
    a2, b2 = c2["a"].to(dev), c2["b"].to(dev)
    c4 = W.c4()
    w4, a4, b4 = (c4[k].to(dev) for k in "wab")
    for _ in range(3):
        lm2exp(a2, b2, _precision="fp32")
        lt2exp(w4, a4, b4, _precision="fp32")
    torch.cuda.synchronize()
    log("profile pass done: 3 x (copy 256 MiB, lt2exp large [fp32, bf16x3, bf16x6, one column], vmax, matmax x2, "
        "lm2exp rectangular [fp32, bf16x3, bf16x6], lm2exp R=16 512^3, lt2exp R=16 S=64 I=J=32 K=2048)")
    return 0


def lookup_traffic(kernel: str, required: bool):
    """HBM bytes per launch of `kernel` from the counter summary; without a row: stop (required)
    or None."""
    try:
        return measured_traffic_bytes(kernel)
    except SystemExit:
        if required:
            raise
        return None


def contraction_line(workload: str, fn, flops: int, nbytes: int, kernel: str, args, *, required_traffic: bool,
                     sibling=None):
    """One contraction configuration: prewarm, warm-up, `steps` timed calls; GFLOP/s from the wall
    clock, roofline from HIP events on the launch stream around the same region.  `sibling`: the
    same call on another tile of the same kernel family.  Under --back-to-back it does the
    pre-conditioning (power and clock take some 25 launches to settle under a matrix load), so that
    in a kernel trace of the run the launches of the timed kernel are the warm-up and timed steps
    and nothing else, and the trace's average duration can be held against the timed figure."""
    tr = timed_region(fn, args.steps, args.warmup, per_launch=not args.back_to_back,
                      prewarm_fn=sibling if args.back_to_back else None)
    wall, ev = tr["wall_s"], tr["event_s"]
    ach = flops / (ev / args.steps) / 1e12
    roof = {"bound": "mfma", "achieved": round(ach, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": lookup_traffic(kernel, required_traffic),
            "kernel": kernel,
            "launch_ms": {"mean": round(ev / args.steps * 1e3, 5)}}
    if tr["median_ms"] is not None:
        roof["launch_ms"].update(median=round(tr["median_ms"], 5), q10=round(tr["q10_ms"], 5),
                                 q90=round(tr["q90_ms"], 5))
        roof["frac_at_median"] = round(flops / (tr["median_ms"] * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)
    line = {"workload": workload, "value": round(flops * args.steps / wall / 1e9, 1), "unit": "GFLOP/s",
            "ms_per_step": round(wall / args.steps * 1e3, 5), "algorithmic_bytes": nbytes,
            "algorithmic_flops": flops, "roofline": roof, "prewarm_ms": tr["prewarm_ms"]}
    log(f"{workload}: {line['ms_per_step']:.4f} ms/step wall, {ev / args.steps * 1e3:.4f} ms/launch (HIP events), "
        f"{ach:.1f} TFLOP/s = {ach / PEAK_FP32_MFMA_TFLOPS * 100:.1f}% of fp32 MFMA peak  [{kernel}]")
    return line


def cpu_passes(fn, passes: int = 3):
    """Median seconds of fn() on the host cores: one warm-up, then `passes` timed passes."""
    fn()
    ts = []
    for _ in range(passes):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts), passes


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip lm2exp / c2 / c4 / max / do_bench sections")
    ap.add_argument("--back-to-back", action="store_true",
                    help="the contraction regions only, every launch back to back (for a kernel trace): no "
                         "cache-flushed repetitions, no per-launch events, no bf16 / max / host-cost sections")
    ap.add_argument("--profile-pass", action="store_true",
                    help="for rocprofv3 --pmc: launch a 256 MiB trt_copy_bytes and every kernel the bench "
                         "times three times each, print nothing to stdout")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this path is built and measured on ONE GPU; R and K shard without any "
            "exchange step, so a multi-GPU figure would be N independent copies of this run. "
            "Run with --gpus 1.")
        return 2
    if not torch.cuda.is_available():
        log("bench.py: no HIP device visible")
        return 3
    if args.back_to_back:
        args.no_cpu_baseline = True

    from triturus_amd import _lib
    from triturus_amd import workloads as W
    from triturus_amd.lm2exp import lm2exp
    from triturus_amd.lt2exp import lt2exp
    from triturus_amd.max import bmatmax, matmax, vmax

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    log(f"device: {torch.cuda.get_device_name(0)}; torch {torch.__version__}")

    if args.profile_pass:
        return profile_pass(dev)

    # ------------------------------------------------------------ lt2exp, large
    R, S, I, J, K = 64, 64, 64, 64, 4096
    cfg = W.c5(R, S, I, J, K)
    w, a, b = (cfg[k].to(dev) for k in "wab")
    flops = W.lt2exp_flops(R, S, I, J, K)
    step = lambda: lt2exp(w, a, b, _precision="fp32")
    kernel = _lib.kernel_name("lt2exp", R, S, I, J, K, _lib.MODE_AUTO, 0, 1)
    head = contraction_line("lt2exp R=64 S=64 I=64 J=64 K=4096 (unsplit)", step, flops,
                            W.lt2exp_bytes(R, S, I, J, K), kernel, args, required_traffic=True,
                            sibling=lambda: lt2exp(w, a, b, _precision="fp32", _variant=2))  # j-chunks of 32
    value = head["value"]
    launch_ms = head["roofline"]["launch_ms"]["mean"]
    result = {
        "metric": "lt2exp GFLOP/s (fp32, 2*R*S*I*J*K flops per call)",
        "value": value,
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded: w ~ Dirichlet(1) over i*j, a,b ~ N(-30,10)), resident in HBM",
        "config": {"workload": head["workload"], "R": R, "S": S, "I": I, "J": J,
                   "K": K, "algorithmic_bytes": head["algorithmic_bytes"], "algorithmic_flops": flops},
        "roofline": head["roofline"],
        "prewarm_ms": head["prewarm_ms"],
    }

    from oracle import torch_baseline  # CPU competitor lines only; never on the GPU path

    if not args.no_cpu_baseline:
        torch.set_num_threads(max(1, min(16, os.cpu_count() or 1)))
        # the whole workload, one batch at a time (the recipe materialises I*J*K floats per batch)
        sec, reps = cpu_passes(lambda: torch_baseline.lt2exp_fp32_chunked(cfg["w"], cfg["a"], cfg["b"], 1))
        cpu_gflops = flops / sec / 1e9
        result["cpu_baseline"] = {
            "value": round(cpu_gflops, 2),
            "unit": "GFLOP/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"the whole workload (all {R} batches of the same inputs), torch fp32 recipe "
                      f"(amax/clamp/exp/outer/bmm/log) one batch at a time, {sec:.2f} s per pass, median of {reps} "
                      f"passes after 1 warm-up pass; host has {os.cpu_count()} logical CPUs",
            "speedup_gpu_over_cpu": round(value / cpu_gflops, 1),
        }
        log(f"cpu baseline lt2exp: {cpu_gflops:.1f} GFLOP/s on {torch.get_num_threads()} threads ({sec:.2f} s per pass)")

    def split_bf16_line(fn_of_precision, flops_alg):
        """The same call on the bf16 matrix pipe (fp32 in/out, operands cut into bf16 pieces):
        not the headline figure -- the arithmetic is not the fp32 matrix instruction."""
        out = {}
        for prec, mfmas in (("bf16x3", 3), ("bf16x6", 6)):
            fn = lambda: fn_of_precision(prec)
            t = timed_region(fn, args.steps, args.warmup)["event_s"] / args.steps
            out[prec] = {
                "ms": round(t * 1e3, 5),
                "equivalent_TFLOPs": round(flops_alg / t / 1e12, 2),
                "speedup_over_fp32_pipe": None,
                "roofline": {"bound": "mfma", "achieved": round(mfmas * flops_alg / t / 1e12, 1),
                             "peak": PEAK_BF16_MFMA_TFLOPS, "unit": "TFLOP/s (bf16 MFMA issued)",
                             "frac": round(mfmas * flops_alg / t / 1e12 / PEAK_BF16_MFMA_TFLOPS, 4)},
            }
            log(f"  {prec}: {t * 1e3:.4f} ms, {flops_alg / t / 1e12:.1f} TFLOP/s fp32-equivalent")
        return out

    extras = not args.no_extras
    full = extras and not args.back_to_back
    if full:
        result["do_bench_lt2exp"] = do_bench(step)
        sb = split_bf16_line(lambda prec: lt2exp(w, a, b, _precision=prec), flops)
        for v in sb.values():
            v["speedup_over_fp32_pipe"] = round(launch_ms / v["ms"], 2)
        result["lt2exp_split_bf16"] = sb
    if extras:
        del w, a, b
        # ------------------------------------------------------- lm2exp, rectangular
        R2, I2, J2, K2 = 64, 256, 256, 4096
        cfg3 = W.c3(R2, I2, J2, K2)
        a3, b3 = cfg3["a"].to(dev), cfg3["b"].to(dev)
        fl3 = W.lm2exp_flops(R2, I2, J2, K2)
        step3 = lambda: lm2exp(a3, b3, _precision="fp32")
        kernel3 = _lib.kernel_name("lm2exp", R2, I2, J2, K2, 0, 0, 1)
        lm = contraction_line("lm2exp R=64 I=256 J=256 K=4096 (b ~ N(-50,20), 5% -inf)", step3, fl3,
                              W.lm2exp_bytes(R2, I2, J2, K2), kernel3, args, required_traffic=True,
                              sibling=lambda: lm2exp(a3, b3, _precision="fp32", _variant=17))  # 128-row paired tile
        if full:
            lm["do_bench"] = do_bench(step3)
        if not args.no_cpu_baseline:
            sec, reps = cpu_passes(lambda: [torch_baseline.lm2exp_fp32(cfg3["a"][r:r + 1], cfg3["b"][r:r + 1])
                                            for r in range(R2)])
            g = fl3 / sec / 1e9
            lm["cpu_baseline"] = {"value": round(g, 2), "unit": "GFLOP/s", "cores": torch.get_num_threads(),
                                  "kind": "port",
                                  "sample": f"the whole workload (all {R2} batches, one at a time), {sec:.2f} s per "
                                            f"pass, median of {reps} passes after 1 warm-up pass",
                                  "speedup_gpu_over_cpu": round(lm["value"] / g, 1)}
            log(f"cpu baseline lm2exp: {g:.1f} GFLOP/s ({sec:.2f} s per pass)")
        if full:
            sb3 = split_bf16_line(lambda prec: lm2exp(a3, b3, _precision=prec), fl3)
            for v in sb3.values():
                v["speedup_over_fp32_pipe"] = round(lm["roofline"]["launch_ms"]["mean"] / v["ms"], 2)
                v["algorithmic_GBps"] = round(lm["algorithmic_bytes"] / (v["ms"] * 1e-3) / 1e9, 1)
            lm["split_bf16"] = sb3
        result["lm2exp"] = lm
        del a3, b3

        # ------------------------------- the two mid-size configurations (grids of 1-2 tiles per CU)
        c2 = W.c2()
        a2, b2 = c2["a"].to(dev), c2["b"].to(dev)
        result["c2"] = contraction_line(
            "lm2exp R=16 I=J=K=512 (b ~ N(-20,5), 1% -inf, one -inf column per batch)",
            lambda: lm2exp(a2, b2, _precision="fp32"), W.lm2exp_flops(16, 512, 512, 512),
            W.lm2exp_bytes(16, 512, 512, 512), _lib.kernel_name("lm2exp", 16, 512, 512, 512, 0, 0, 1), args,
            required_traffic=False, sibling=lambda: lm2exp(a2, b2, _precision="fp32", _variant=1))
        del a2, b2
        c4 = W.c4()
        w4, a4, b4 = (c4[k].to(dev) for k in "wab")
        result["c4"] = contraction_line(
            "lt2exp R=16 S=64 I=J=32 K=2048 (a,b ~ N(-20,5), 2% -inf)",
            lambda: lt2exp(w4, a4, b4, _precision="fp32"), W.lt2exp_flops(16, 64, 32, 32, 2048),
            W.lt2exp_bytes(16, 64, 32, 32, 2048),
            _lib.kernel_name("lt2exp", 16, 64, 32, 32, 2048, _lib.MODE_AUTO, 0, 1), args, required_traffic=False,
            sibling=lambda: lt2exp(w4, a4, b4, _precision="fp32", _variant=4, mode="unsplit"))  # 32-row tile
        del w4, a4, b4

    if full:
        # ------------------------------------ lm2exp, smallest configuration: bound by the host
        c1 = W.c1()
        a1, b1 = c1["a"].to(dev), c1["b"].to(dev)
        for _ in range(200):
            lm2exp(a1, b1)
        torch.cuda.synchronize()
        n1 = 2000
        t0 = time.perf_counter()
        for _ in range(n1):
            lm2exp(a1, b1)
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t0) / n1 * 1e6
        result["c1"] = {"workload": "lm2exp R=4 I=J=K=64", "eager_us_per_call": round(eager_us, 2),
                        "hip_graph_us_per_call": round(graph_time(lambda: lm2exp(a1, b1)) * 1e6, 2)}
        log(f"lm2exp smallest configuration: {eager_us:.2f} us per eager call through the Python wrapper, "
            f"{result['c1']['hip_graph_us_per_call']:.2f} us inside a HIP graph")

        # ------------------------------------------------ lt2exp with few columns (HBM bound)
        # The large configuration's weights under 1, 4 and 8 columns -- one sample per batch, or a
        # handful: a serving call.  The contraction is then a sweep over w (67.1 MB), timed like
        # the reductions below: 8 copies of w in turn (from HBM) and the same w again and again.
        from benchmarks.torch_recipes import torch_lt2exp  # the eager torch recipe, on the GPU

        wl = cfg["w"].to(dev)
        wcopies = [wl] + [wl.clone() for _ in range(7)]
        wbytes = wl.numel() * 4
        sv = {"workload": "lt2exp R=64 S=I=J=64, K = 1, 4, 8 (a,b ~ N(-30,10))", "bytes": wbytes, "unit": "GB/s",
              "peak": PEAK_HBM_GBPS, "protocol": "us / achieved / frac: 8 copies of w in turn (every call streams "
                                                 "from HBM); same_operand: one w again and again"}
        for kk in (1, 4, 8):
            ak, bk = cfg["a"][:, :, :kk].contiguous().to(dev), cfg["b"][:, :, :kk].contiguous().to(dev)
            fnk = lambda z: lt2exp(z, ak, bk, _precision="fp32")
            hot = graph_time(lambda: fnk(wl), prewarm_ms=PREWARM_MS)
            cold = graph_time(fnk, calls=24, prewarm_ms=PREWARM_MS / 2, operands=wcopies)
            tor = graph_time(lambda: torch_lt2exp(wl, ak, bk))
            sv[f"k{kk}"] = {"kernel": _lib.kernel_name("lt2exp", 64, 64, 64, 64, kk, _lib.MODE_AUTO, 0, 1),
                            "us": round(cold * 1e6, 2), "achieved": round(wbytes / cold / 1e9, 1),
                            "frac": round(wbytes / cold / 1e9 / PEAK_HBM_GBPS, 4),
                            "same_operand": {"us": round(hot * 1e6, 2), "achieved": round(wbytes / hot / 1e9, 1)},
                            "torch_recipe_same_operand_us": round(tor * 1e6, 2)}
            log(f"lt2exp K={kk}: {cold * 1e6:.2f} us from HBM ({wbytes / cold / 1e9:.0f} GB/s = "
                f"{wbytes / cold / 1e9 / PEAK_HBM_GBPS * 100:.1f}% of 8 TB/s), {hot * 1e6:.2f} us on the same w, "
                f"torch recipe {tor * 1e6:.2f} us")
        result["few_columns"] = sv
        del wl, wcopies

        # ------------------------------------------------ lt2exp with few s per batch
        # Many batches of one to eight s: the library puts the rows (s, i) of w on the rows of the
        # MFMA and contracts j first.  Bytes: w, a, b and c once (a and b outweigh w here).
        fr = {"protocol": "the same operands again and again, inside a HIP graph", "unit": "GB/s", "peak": PEAK_HBM_GBPS}
        gen = torch.Generator().manual_seed(7)
        for (rr, ss, ii, jj, kk) in ((2048, 1, 64, 64, 64), (2048, 4, 64, 64, 64), (512, 2, 128, 128, 32), (128, 8, 200, 100, 64)):
            wf = torch.rand(rr, ss, ii, jj, generator=gen).to(dev)
            af = (torch.randn(rr, ii, kk, generator=gen) * 10 - 30).to(dev)
            bf = (torch.randn(rr, jj, kk, generator=gen) * 10 - 30).to(dev)
            nbytes_f = 4 * (wf.numel() + af.numel() + bf.numel() + rr * ss * kk)
            sec = graph_time(lambda: lt2exp(wf, af, bf, _precision="fp32"), prewarm_ms=PREWARM_MS / 2)
            tor = graph_time(lambda: torch_lt2exp(wf, af, bf), calls=5, reps=5)
            fr[f"R{rr}_S{ss}_I{ii}_J{jj}_K{kk}"] = {
                "kernel": _lib.kernel_name("lt2exp", rr, ss, ii, jj, kk, _lib.MODE_AUTO, 0, 1), "bytes": nbytes_f,
                "us": round(sec * 1e6, 2), "achieved": round(nbytes_f / sec / 1e9, 1),
                "frac": round(nbytes_f / sec / 1e9 / PEAK_HBM_GBPS, 4),
                "tflops": round(2.0 * rr * ss * ii * jj * kk / sec / 1e12, 2), "torch_recipe_us": round(tor * 1e6, 2)}
            log(f"lt2exp R={rr} S={ss} I={ii} J={jj} K={kk}: {sec * 1e6:.2f} us ({nbytes_f / sec / 1e9:.0f} GB/s), "
                f"torch recipe {tor * 1e6:.2f} us")
            del wf, af, bf
        result["few_rows"] = fr

        # ------------------------------------------------ lt2exp on layers of few units over many batches
        # S = I = J = 4, 8 over 8192 batches: a lane per output column, the batch's weights as scalar
        # operands.  Bytes: w, a, b and c once.
        fu = {"protocol": "the same operands again and again, inside a HIP graph", "unit": "GB/s", "peak": PEAK_HBM_GBPS}
        for (rr, uu, kk) in ((8192, 4, 1024), (8192, 8, 256), (8192, 8, 1024), (2048, 16, 512)):
            ss = 1 if uu == 16 else uu
            wf = torch.rand(rr, ss, uu, uu, generator=gen).to(dev)
            af = (torch.randn(rr, uu, kk, generator=gen) * 10 - 30).to(dev)
            bf = (torch.randn(rr, uu, kk, generator=gen) * 10 - 30).to(dev)
            nbytes_f = 4 * (wf.numel() + af.numel() + bf.numel() + rr * ss * kk)
            sec = graph_time(lambda: lt2exp(wf, af, bf, _precision="fp32"), prewarm_ms=PREWARM_MS / 2)
            tor = graph_time(lambda: torch_lt2exp(wf, af, bf), calls=5, reps=5)
            fu[f"R{rr}_S{ss}_I{uu}_J{uu}_K{kk}"] = {
                "kernel": _lib.kernel_name("lt2exp", rr, ss, uu, uu, kk, _lib.MODE_AUTO, 0, 1), "bytes": nbytes_f,
                "us": round(sec * 1e6, 2), "achieved": round(nbytes_f / sec / 1e9, 1),
                "frac": round(nbytes_f / sec / 1e9 / PEAK_HBM_GBPS, 4), "torch_recipe_us": round(tor * 1e6, 2)}
            log(f"lt2exp R={rr} S={ss} I=J={uu} K={kk}: {sec * 1e6:.2f} us ({nbytes_f / sec / 1e9:.0f} GB/s = "
                f"{nbytes_f / sec / 1e9 / PEAK_HBM_GBPS * 100:.1f}% of 8 TB/s), torch recipe {tor * 1e6:.2f} us")
            del wf, af, bf
        from benchmarks.torch_recipes import torch_lm2exp

        for (rr, uu, kk) in ((8192, 4, 1024), (8192, 8, 1024)):   # lm2exp: the same kernel, the rows of a as the weights
            am = torch.rand(rr, uu, uu, generator=gen).to(dev)
            bm = (torch.randn(rr, uu, kk, generator=gen) * 10 - 30).to(dev)
            nbytes_f = 4 * (am.numel() + bm.numel() + rr * uu * kk)
            sec = graph_time(lambda: lm2exp(am, bm, _precision="fp32"), prewarm_ms=PREWARM_MS / 2)
            tor = graph_time(lambda: torch_lm2exp(am, bm), calls=5, reps=5)
            fu[f"lm2exp_R{rr}_I{uu}_J{uu}_K{kk}"] = {
                "kernel": _lib.kernel_name("lm2exp", rr, uu, uu, kk, 0, 0, 1), "bytes": nbytes_f,
                "us": round(sec * 1e6, 2), "achieved": round(nbytes_f / sec / 1e9, 1),
                "frac": round(nbytes_f / sec / 1e9 / PEAK_HBM_GBPS, 4), "torch_recipe_us": round(tor * 1e6, 2)}
            log(f"lm2exp R={rr} I=J={uu} K={kk}: {sec * 1e6:.2f} us ({nbytes_f / sec / 1e9:.0f} GB/s = "
                f"{nbytes_f / sec / 1e9 / PEAK_HBM_GBPS * 100:.1f}% of 8 TB/s), torch recipe {tor * 1e6:.2f} us")
            del am, bm
        result["few_units"] = fu

        # ------------------------------------------------ lm2exp on narrow outputs of few rows per batch
        # At most 64 columns and 32 rows: one tile per batch, its contraction cut over the four
        # wavefronts.  Bytes: a, b and c once (b outweighs the rest).
        nw = {"protocol": "the same operands again and again, inside a HIP graph", "unit": "GB/s", "peak": PEAK_HBM_GBPS}
        for (rr, ii, jj, kk) in ((8192, 1, 256, 16), (4096, 16, 256, 16), (8192, 32, 64, 16), (4096, 1, 256, 32)):
            am = torch.rand(rr, ii, jj, generator=gen).to(dev)
            bm = (torch.randn(rr, jj, kk, generator=gen) * 10 - 30).to(dev)
            nbytes_f = 4 * (am.numel() + bm.numel() + rr * ii * kk)
            sec = graph_time(lambda: lm2exp(am, bm, _precision="fp32"), prewarm_ms=PREWARM_MS / 2)
            tor = graph_time(lambda: torch_lm2exp(am, bm), calls=5, reps=5)
            nw[f"lm2exp_R{rr}_I{ii}_J{jj}_K{kk}"] = {
                "kernel": _lib.kernel_name("lm2exp", rr, ii, jj, kk, 0, 0, 1), "bytes": nbytes_f,
                "us": round(sec * 1e6, 2), "achieved": round(nbytes_f / sec / 1e9, 1),
                "frac": round(nbytes_f / sec / 1e9 / PEAK_HBM_GBPS, 4), "torch_recipe_us": round(tor * 1e6, 2)}
            log(f"lm2exp R={rr} I={ii} J={jj} K={kk}: {sec * 1e6:.2f} us ({nbytes_f / sec / 1e9:.0f} GB/s = "
                f"{nbytes_f / sec / 1e9 / PEAK_HBM_GBPS * 100:.1f}% of 8 TB/s), torch recipe {tor * 1e6:.2f} us")
            del am, bm
        result["narrow"] = nw

        # ------------------------------------------------ max reductions (HBM bound)
        # Two figures per reduction.  `us`, `achieved`, `frac`: 8 copies of the 64 MiB operand
        # (512 MiB) taken in turn, so that every call streams from HBM -- the figure to hold
        # against the HBM roofline.  `same_operand`: one operand call after call, as a caller
        # that reduces one tensor repeatedly sees it -- the operand then fits the 256 MB
        # memory-side cache, and the library's read-once loads leave in place whatever part of
        # it an earlier pass left in the dies' L2s; not an HBM figure.
        x = cfg["b"].to(dev)  # 64 x 64 x 4096
        nbytes = x.numel() * 4
        copies = [x] + [x.clone() for _ in range(7)]
        mx = {"bytes": nbytes, "unit": "GB/s", "peak": PEAK_HBM_GBPS,
              "protocol": "us / achieved / frac: 8 operands in turn (every call streams from HBM); "
                          "same_operand: one operand again and again (served in part by the caches)"}
        fns = (("vmax", lambda z: vmax(z.view(-1))), ("matmax_axis0", lambda z: matmax(z.view(4096, 4096), 0)),
               ("matmax_axis1", lambda z: matmax(z.view(4096, 4096), 1)),
               ("bmatmax_shift", lambda z: bmatmax(z, clamp=True)),  # 64 x 64 x 4096 -> 64 x 4096: the shift m
               ("torch_amax_batched", lambda z: torch.amax(z, 1)),
               ("torch_max", lambda z: torch.max(z.view(-1), 0)),
               ("torch_amax_axis0", lambda z: torch.amax(z.view(4096, 4096), 0)),
               ("torch_amax_axis1", lambda z: torch.amax(z.view(4096, 4096), 1)))
        # (all the one-operand figures first: what a sweep over 512 MiB leaves in the caches is
        # not what a caller that keeps reducing one tensor finds there)
        same = {}
        for name, fn in fns:
            sec, before = graph_time(lambda: fn(x), prewarm_ms=PREWARM_MS, both=True)
            same[name] = {"us": round(sec * 1e6, 2), "achieved": round(nbytes / sec / 1e9, 1),
                          "frac": round(nbytes / sec / 1e9 / PEAK_HBM_GBPS, 4),
                          "us_before_prewarm": round(before * 1e6, 2)}
            log(f"{name}, same operand: {sec * 1e6:.2f} us, {nbytes / sec / 1e9:.0f} GB/s "
                f"({before * 1e6:.2f} us before the prewarm)")
        for name, fn in fns:
            cold = graph_time(fn, calls=24, prewarm_ms=PREWARM_MS / 2, operands=copies)
            mx[name] = {"us": round(cold * 1e6, 2), "achieved": round(nbytes / cold / 1e9, 1),
                        "frac": round(nbytes / cold / 1e9 / PEAK_HBM_GBPS, 4), "same_operand": same[name]}
            log(f"{name}, 8 operands in turn (from HBM): {cold * 1e6:.2f} us, {nbytes / cold / 1e9:.0f} GB/s = "
                f"{nbytes / cold / 1e9 / PEAK_HBM_GBPS * 100:.1f}% of 8 TB/s")
        mx["prewarm_ms"] = PREWARM_MS
        result["max"] = mx

    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
