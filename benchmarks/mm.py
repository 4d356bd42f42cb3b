"""mm and vadd sweeps over the reference's grids (benchmarks/mm.py:16-29 and
benchmarks/add.py:16-27 there).  Metrics, as there: TFLOPS with m*n*(2k-1) flops for mm and n
additions for vadd (the reference's grid stops at n = 49152, where a launch dominates; two
large sizes are appended).  Neither is on the log-space path.

    python -m benchmarks.mm [output_dir]
"""

import torch

from benchmarks.utils import do_bench, eval_tflops, out_dir_from_argv, run_sweep
from triturus.add import vadd
from triturus.mm import mm
from triturus.utils import ensure_reproducibility, set_tf32_enabled

PROVIDERS = ["torch", "triturus", "triturus (allow_tf32)"]


def measure_mm(n, provider):
    ensure_reproducibility()
    set_tf32_enabled(provider == "triturus (allow_tf32)")
    a = torch.rand(n, n)
    b = torch.rand(n, n)
    fn = (lambda: torch.mm(a, b)) if provider == "torch" else (lambda: mm(a, b))
    ms, lo, hi = do_bench(fn)
    set_tf32_enabled(False)
    nflops = n * n * (2 * n - 1)
    return eval_tflops(nflops, ms), eval_tflops(nflops, hi), eval_tflops(nflops, lo)


def measure_vadd(n, provider):
    ensure_reproducibility()
    x = torch.rand(n)
    y = torch.rand(n)
    fn = (lambda: x + y) if provider == "torch" else (lambda: vadd(x, y))
    ms, lo, hi = do_bench(fn)
    return eval_tflops(n, ms), eval_tflops(n, hi), eval_tflops(n, lo)


def main():
    out = out_dir_from_argv()
    run_sweep("mm", "m=k=n", [48, 128, 192, 512, 768, 2048, 3072, 8192], PROVIDERS, measure_mm,
              unit="TFLOPS", out_dir=out)
    run_sweep("vadd", "n", [32, 48, 128, 192, 512, 768, 2048, 3072, 8192, 12288, 32768, 49152, 1 << 24, 1 << 28],
              PROVIDERS[:2], measure_vadd, unit="TFLOPS (additions)", out_dir=out)


if __name__ == "__main__":
    main()
