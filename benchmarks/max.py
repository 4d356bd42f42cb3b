"""vmax / vamax / matmax sweeps over the reference's grid (benchmarks/max.py:16-66
there).  Metric, as there: comparisons per second in "TFLOPS" -- n-1 for a vector,
n*(m-1) (axis 0) or m*(n-1) (axis 1) for a matrix.

    python -m benchmarks.max [output_dir]
"""

import torch

from benchmarks.utils import do_bench, eval_tflops, out_dir_from_argv, run_sweep
from triturus.max import matmax, vamax, vmax
from triturus.utils import ensure_reproducibility

PROVIDERS = ["torch", "triturus"]


def measure_vmax(n, provider, return_idx):
    ensure_reproducibility()
    x = torch.rand(n)
    if provider == "torch":
        fn = (lambda: torch.max(x, dim=0)) if return_idx else (lambda: torch.amax(x, dim=0))
    else:
        fn = (lambda: vmax(x)) if return_idx else (lambda: vamax(x))
    ms, lo, hi = do_bench(fn)
    return eval_tflops(n - 1, ms), eval_tflops(n - 1, hi), eval_tflops(n - 1, lo)


def measure_matmax(m, n, provider, axis):
    ensure_reproducibility()
    x = torch.rand(m, n)
    fn = (lambda: torch.amax(x, dim=axis)) if provider == "torch" else (lambda: matmax(x, axis=axis))
    ms, lo, hi = do_bench(fn)
    nflops = n * (m - 1) if axis == 0 else m * (n - 1)
    return eval_tflops(nflops, ms), eval_tflops(nflops, hi), eval_tflops(nflops, lo)


def main():
    out = out_dir_from_argv()
    for return_idx in (False, True):
        run_sweep(f"vmax (return_idx={return_idx})", "n",
                  [32, 96, 256, 768, 2048, 6144, 16384, 49152, 131072, 393216, 1048576, 16777216], PROVIDERS,
                  lambda x, p: measure_vmax(x, p, return_idx), unit="TFLOPS (comparisons)", out_dir=out)
    for axis in (0, 1):
        run_sweep(f"matmax (axis={axis})", "m=n", [32, 48, 128, 192, 512, 768, 2048, 3072, 8192], PROVIDERS,
                  lambda x, p: measure_matmax(x, x, p, axis), unit="TFLOPS (comparisons)", out_dir=out)


if __name__ == "__main__":
    main()
