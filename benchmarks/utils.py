"""Shared pieces of the benchmark sweeps: the reference's metric definitions
(benchmarks/utils.py:1-9 there) and a small runner in place of triton.testing."""

from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

QUANTILES = [0.5, 0.1, 0.9]


def eval_tflops(nflops: int, ms: float) -> float:
    return (nflops * 1e-12) / (ms * 1e-3)


def eval_gbps(size: int, ms: float, *, bpe: int = 4) -> float:
    return ((size * bpe) * 1e-9) / (ms * 1e-3)


_flush = None


def do_bench(fn, *, warmup: float = 25.0, rep: float = 100.0, quantiles=QUANTILES):
    """Milliseconds at the given quantiles.  `warmup` / `rep` are time budgets in ms, every
    timed call is preceded by zeroing a 512 MiB buffer (MI355X has 256 MiB of Infinity
    Cache), timing with HIP events on the current stream -- the protocol the reference
    gets from triton.testing.do_bench (benchmarks/lm2exp.py:94 there)."""
    global _flush
    if _flush is None:
        _flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(5):
        _flush.zero_()
        fn()
    e.record()
    torch.cuda.synchronize()
    est = max(s.elapsed_time(e) / 5, 1e-3)
    n_warm = max(1, int(warmup / est))
    n_rep = max(10, min(1000, int(rep / est)))
    for _ in range(n_warm):
        fn()
    ss = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    ee = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for i in range(n_rep):
        _flush.zero_()
        ss[i].record()
        fn()
        ee[i].record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in zip(ss, ee))
    return [ts[min(len(ts) - 1, int(q * len(ts)))] for q in quantiles]


def run_sweep(name: str, x_name: str, x_vals, providers, measure, *, unit: str, out_dir: str | None):
    """measure(x, provider) -> (value, lo, hi).  Prints one table and optionally writes JSON."""
    rows = []
    print(f"\n{name}  [{unit}]", flush=True)
    print(f"{x_name:>10s} " + " ".join(f"{p:>22s}" for p in providers), flush=True)
    for x in x_vals:
        vals = []
        for p in providers:
            try:
                v = measure(x, p)
            except torch.OutOfMemoryError:
                v = (float("nan"),) * 3
            vals.append(v)
        rows.append({"x": x, **{p: v for p, v in zip(providers, vals)}})
        print(f"{x:>10d} " + " ".join(f"{v[0]:>22.2f}" for v in vals), flush=True)
    if out_dir:
        Path(out_dir).mkdir(parents=True, exist_ok=True)
        fname = "".join(c if c.isalnum() else "_" for c in name) + ".json"
        (Path(out_dir) / fname).write_text(json.dumps({"name": name, "x": x_name, "unit": unit, "rows": rows}))
    return rows


def out_dir_from_argv() -> str | None:
    return sys.argv[1] if len(sys.argv) > 1 else None
