"""The reference's torch recipes in fp32, op for op.  Test infrastructure.

These are the CPU competitor lines: the benchmark times them on the host cores
next to the GPU kernels, and the parity tests use them as the fp32 ground truth
the reference's own tests use (tests/lm2exp.py:16, tests/lt2exp.py:23).
Restated from baselines/lm2exp.py:4-14 and baselines/lt2exp.py:4-25; they run
on whatever device the inputs live on.
"""

from __future__ import annotations

import torch


def lm2exp_fp32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    m = torch.amax(b, dim=1, keepdim=True)
    m = torch.clamp(m, -1e38, 1e38)
    r = torch.bmm(a, torch.exp(b - m))
    return m + torch.log(r)


def lt2exp_fp32(w: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    batch, m, n = w.shape[0], w.shape[1], a.shape[2]
    ma = torch.amax(a, dim=1, keepdim=True)
    ma = torch.clamp(ma, -1e38, 1e38)
    exp_a = torch.exp(a - ma)
    mb = torch.amax(b, dim=1, keepdim=True)
    mb = torch.clamp(mb, -1e38, 1e38)
    exp_b = torch.exp(b - mb)
    s = exp_a.unsqueeze(dim=2) * exp_b.unsqueeze(dim=1)
    s = s.view(batch, -1, n)
    w = w.view(batch, m, -1)
    r = torch.bmm(w, s)
    return ma + mb + torch.log(r)


def lt2exp_fp32_chunked(w: torch.Tensor, a: torch.Tensor, b: torch.Tensor, batch_chunk: int) -> torch.Tensor:
    """Same recipe, ``batch_chunk`` batches at a time: the R x (I*J) x K intermediate
    of the one-shot recipe is 4.3 GB at R=64, I=J=64, K=4096."""
    out = []
    for r0 in range(0, w.shape[0], batch_chunk):
        sl = slice(r0, r0 + batch_chunk)
        out.append(lt2exp_fp32(w[sl], a[sl], b[sl]))
    return torch.cat(out, dim=0)
