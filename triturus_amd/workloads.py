"""Seeded synthetic inputs of the five benchmark configurations.

All tensors are drawn on the CPU with a private ``torch.Generator`` (seed =
42 + configuration index) so that the GPU kernels and any CPU checker see the
same values; callers move them to the device.
"""

from __future__ import annotations

import torch

NEG_INF = float("-inf")


def _gen(index: int) -> torch.Generator:
    return torch.Generator(device="cpu").manual_seed(42 + index)


def _knock_out(t: torch.Tensor, p: float, g: torch.Generator) -> torch.Tensor:
    """Set a Bernoulli(p) subset of t to -inf (in place)."""
    mask = torch.rand(t.shape, generator=g) < p
    t[mask] = NEG_INF
    return t


def c1():
    """lm2exp R=4, I=J=K=64: a ~ U(0,1) row-normalised over j; b ~ N(-10, 3)."""
    g = _gen(1)
    a = torch.rand(4, 64, 64, generator=g)
    a = a / a.sum(dim=2, keepdim=True)
    b = -10.0 + 3.0 * torch.randn(4, 64, 64, generator=g)
    return {"op": "lm2exp", "a": a, "b": b}


def c2(R: int = 16, n: int = 512):
    """lm2exp square batch: b ~ N(-20, 5), 1% -inf, one all -inf column per batch."""
    g = _gen(2)
    a = torch.rand(R, n, n, generator=g)
    a = a / a.sum(dim=2, keepdim=True)
    b = -20.0 + 5.0 * torch.randn(R, n, n, generator=g)
    _knock_out(b, 0.01, g)
    cols = torch.randint(0, n, (R,), generator=g)
    for r in range(R):
        b[r, :, cols[r]] = NEG_INF
    return {"op": "lm2exp", "a": a, "b": b, "neg_inf_cols": cols}


def c3(R: int = 64, I: int = 256, J: int = 256, K: int = 4096):
    """lm2exp rectangular: a ~ Dirichlet(1) rows; b ~ N(-50, 20), 5% -inf."""
    g = _gen(3)
    a = torch.empty(R, I, J).exponential_(1.0, generator=g)
    a = a / a.sum(dim=2, keepdim=True)
    b = -50.0 + 20.0 * torch.randn(R, J, K, generator=g)
    _knock_out(b, 0.05, g)
    return {"op": "lm2exp", "a": a, "b": b}


def c4(R: int = 16, S: int = 64, I: int = 32, J: int = 32, K: int = 2048):
    """lt2exp: w ~ U(0,1) normalised over (i,j); a, b ~ N(-20, 5), 2% -inf each."""
    g = _gen(4)
    w = torch.rand(R, S, I, J, generator=g)
    w = w / w.sum(dim=(2, 3), keepdim=True)
    a = -20.0 + 5.0 * torch.randn(R, I, K, generator=g)
    b = -20.0 + 5.0 * torch.randn(R, J, K, generator=g)
    _knock_out(a, 0.02, g)
    _knock_out(b, 0.02, g)
    return {"op": "lt2exp", "w": w, "a": a, "b": b}


def c5(R: int = 64, S: int = 64, I: int = 64, J: int = 64, K: int = 4096):
    """lt2exp large: w ~ Dirichlet(1) over the flattened (i,j); a, b ~ N(-30, 10)."""
    g = _gen(5)
    w = torch.empty(R, S, I, J).exponential_(1.0, generator=g)
    w = w / w.sum(dim=(2, 3), keepdim=True)
    a = -30.0 + 10.0 * torch.randn(R, I, K, generator=g)
    b = -30.0 + 10.0 * torch.randn(R, J, K, generator=g)
    return {"op": "lt2exp", "w": w, "a": a, "b": b}


CONFIGS = {"c1": c1, "c2": c2, "c3": c3, "c4": c4, "c5": c5}


def lm2exp_flops(R: int, I: int, J: int, K: int) -> int:
    return 2 * R * I * J * K


def lm2exp_bytes(R: int, I: int, J: int, K: int) -> int:
    return 4 * (R * I * J + R * J * K + R * I * K)


def lt2exp_flops(R: int, S: int, I: int, J: int, K: int) -> int:
    return 2 * R * S * I * J * K


def lt2exp_bytes(R: int, S: int, I: int, J: int, K: int) -> int:
    return 4 * (R * S * I * J + R * I * K + R * J * K + R * S * K)
