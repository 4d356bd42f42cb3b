"""lt2exp sweep over the reference's grid (benchmarks/lt2exp.py:32-63 there):
square m=j=k=n, batch 1; rectangular m=j=k, n=256, batch 32 and 128.  Metric: GB/s of
input bytes, batch*(m*j*k + j*n + k*n)*4 / t (benchmarks/lt2exp.py:90-95 there).

    python -m benchmarks.lt2exp [output_dir]
"""

import torch

from benchmarks.torch_recipes import torch_lt2exp
from benchmarks.utils import do_bench, eval_gbps, out_dir_from_argv, run_sweep
from triturus.lt2exp import lt2exp
from triturus.utils import ensure_reproducibility, set_tf32_enabled

PROVIDERS = ["torch", "triturus", "triturus (unsplit)", "triturus (allow_tf32)"]


def measure(batch, m, j, k, n, provider):
    ensure_reproducibility()
    set_tf32_enabled(provider == "triturus (allow_tf32)")
    w = torch.rand(batch, m, j, k)
    a = torch.randn(batch, j, n)
    b = torch.randn(batch, k, n)
    if provider == "torch":
        fn = lambda: torch_lt2exp(w, a, b)
    elif provider in ("triturus", "triturus (allow_tf32)"):
        fn = lambda: lt2exp(w, a, b)
    else:
        fn = lambda: lt2exp(w, a, b, mode="unsplit")
    ms, lo, hi = do_bench(fn)
    set_tf32_enabled(False)
    size = batch * (m * j * k + j * n + k * n)
    return eval_gbps(size, ms), eval_gbps(size, hi), eval_gbps(size, lo)


def main():
    out = out_dir_from_argv()
    run_sweep("lt2exp (square, batch=1)", "m=j=k=n", [16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512],
              PROVIDERS, lambda x, p: measure(1, x, x, x, x, p), unit="GB/s", out_dir=out)
    for batch in (32, 128):
        run_sweep(f"lt2exp (rectangular, n=256 batch={batch})", "m=j=k", [16, 24, 32, 48, 64, 96, 128, 192, 256],
                  PROVIDERS, lambda x, p: measure(batch, x, x, x, 256, p), unit="GB/s", out_dir=out)


if __name__ == "__main__":
    main()
