"""lm2exp sweep over the reference's grid (benchmarks/lm2exp.py:26-56 there):
square m=k=n, batch 1; rectangular m=k, n=256, batch 64 and 384.  Metric: GB/s of
input bytes, batch*(m*k + k*n)*4 / t (benchmarks/lm2exp.py:95-100 there).  The reference
draws one plot per allow_tf32 value (benchmarks/lm2exp.py:36-39 there); here the flag is a
provider: "triturus (allow_tf32)" runs the same call with set_tf32_enabled(True).

    python -m benchmarks.lm2exp [output_dir]
"""

import torch

from benchmarks.torch_recipes import torch_lm2exp
from benchmarks.utils import do_bench, eval_gbps, out_dir_from_argv, run_sweep
from triturus.lm2exp import lm2exp
from triturus.utils import ensure_reproducibility, set_tf32_enabled

PROVIDERS = ["torch", "triturus", "triturus (allow_tf32)"]


def measure(batch, m, k, n, provider):
    ensure_reproducibility()
    set_tf32_enabled(provider == "triturus (allow_tf32)")
    a = torch.rand(batch, m, k)
    b = torch.randn(batch, k, n)
    fn = (lambda: torch_lm2exp(a, b)) if provider == "torch" else (lambda: lm2exp(a, b))
    ms, lo, hi = do_bench(fn)
    set_tf32_enabled(False)
    size = batch * (m * k + k * n)
    return eval_gbps(size, ms), eval_gbps(size, hi), eval_gbps(size, lo)


def main():
    out = out_dir_from_argv()
    run_sweep("lm2exp (square matrices, batch=1)", "m=k=n", [128, 192, 256, 384, 512, 768, 1024, 1536, 2048],
              PROVIDERS, lambda x, p: measure(1, x, x, x, p), unit="GB/s", out_dir=out)
    for batch in (64, 384):
        run_sweep(f"lm2exp (rectangular matrices, n=256 batch={batch})", "m=k",
                  [64, 96, 128, 192, 256, 384, 512, 768, 1024], PROVIDERS,
                  lambda x, p: measure(batch, x, x, 256, p), unit="GB/s", out_dir=out)


if __name__ == "__main__":
    main()
