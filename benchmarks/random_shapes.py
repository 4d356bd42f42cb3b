"""Random shapes off the reference's grid: lm2exp and lt2exp against the torch recipe on the same
GPU, for shapes drawn log-uniformly (dimensions 1..4096, K up to 8192, bounded in bytes and flops).
Not one of the reference's sweeps: a scan for shapes the tile rules handle badly (warm timing,
event-timed back-to-back calls).  Writes <output_dir>/random_shapes.md, which benchmarks.report appends.

    python -m benchmarks.random_shapes [output_dir] [seed] [count]
"""

import math
import random
import statistics
import sys
from pathlib import Path

import torch

from benchmarks.torch_recipes import torch_lm2exp, torch_lt2exp
from triturus.lm2exp import lm2exp
from triturus.lt2exp import lt2exp
from triturus.utils import set_matrix_precision

PRECISIONS = ["fp32", "bf16x3", "bf16x6"]


def timed(fn, reps=6):
    """Microseconds per call: the better of two event-timed batches after three warm-up calls (a
    single batch now and then catches an allocator stall left by the previous, larger call)."""
    for _ in range(3):
        fn()
    best = float("inf")
    for _ in range(2):
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) / reps * 1e3)
    return best


def main():
    out_dir = Path(sys.argv[1]) if len(sys.argv) > 1 else None
    rng = random.Random(int(sys.argv[2]) if len(sys.argv) > 2 else 3)
    count = int(sys.argv[3]) if len(sys.argv) > 3 else 400
    dev = torch.device("cuda:0")

    def draw(lo, hi):
        return int(round(math.exp(rng.uniform(math.log(lo), math.log(hi)))))

    rows = []
    for it in range(count):
        if it % 2 == 0:
            while True:
                R, I, J, K = draw(1, 512), draw(1, 4096), draw(1, 4096), draw(1, 8192)
                if R * (I * J + J * K + I * K) < 2.5e8 and R * I * J * K < 4e11:
                    break
            a, b = torch.rand(R, I, J, device=dev), torch.randn(R, J, K, device=dev)
            shape, reference, call = (R, I, J, K), (lambda: torch_lm2exp(a, b)), (lambda: lm2exp(a, b))
            op = "lm2exp"
        else:
            while True:
                R, S, I, J, K = draw(1, 256), draw(1, 1024), draw(1, 256), draw(1, 256), draw(1, 8192)
                if max(R * I * J * K, R * S * I * J, R * S * K) < 2.5e8 and R * S * I * J * K < 4e11:
                    break
            w = torch.rand(R, S, I, J, device=dev)
            a, b = torch.randn(R, I, K, device=dev), torch.randn(R, J, K, device=dev)
            shape, reference, call = (R, S, I, J, K), (lambda: torch_lt2exp(w, a, b)), (lambda: lt2exp(w, a, b))
            op = "lt2exp"
        row = {"op": op, "shape": shape, "torch": timed(reference)}
        for precision in PRECISIONS:
            set_matrix_precision(precision)
            row[precision] = timed(call)
        set_matrix_precision(None)
        rows.append(row)
        print(row, flush=True)

    lines = [f"## Random shapes ({count} drawn log-uniformly, seed fixed): speed-up over the torch recipe on the same GPU",
             "", "| op | precision | geometric mean | minimum | shapes slower than torch |", "|---|---|---:|---:|---:|"]
    for op in ("lm2exp", "lt2exp"):
        sel = [r for r in rows if r["op"] == op]
        for precision in PRECISIONS:
            ratio = [r["torch"] / r[precision] for r in sel]
            lines.append(f"| {op} | {precision} | {statistics.geometric_mean(ratio):.2f} | {min(ratio):.2f} | "
                         f"{sum(x < 1 for x in ratio)} of {len(ratio)} |")
    worst = sorted(rows, key=lambda r: r["torch"] / r["fp32"])[:8]
    lines += ["", "Slowest against torch (fp32 pipe), times in µs:", "", "| op | shape | torch | fp32 | bf16x3 | bf16x6 |",
              "|---|---|---:|---:|---:|---:|"]
    for r in worst:
        lines.append(f"| {r['op']} | {'×'.join(map(str, r['shape']))} | {r['torch']:.1f} | {r['fp32']:.1f} | "
                     f"{r['bf16x3']:.1f} | {r['bf16x6']:.1f} |")
    text = "\n".join(lines) + "\n"
    print(text)
    if out_dir is not None:
        out_dir.mkdir(parents=True, exist_ok=True)
        (out_dir / "random_shapes.md").write_text(text)


if __name__ == "__main__":
    main()
