"""float64 oracles for lm2exp / lt2exp (CPU, torch + NumPy).  Test infrastructure.

``lm2exp64`` / ``lt2exp64`` restate the reference's ground-truth recipes
(baselines/lm2exp.py:11-14 and baselines/lt2exp.py:15-25: amax -> clamp to
+-1e38 -> exp(shifted) -> bmm -> add the shift back to log) in float64.
``lm2exp_lse`` / ``lt2exp_lse`` are independent closed forms,
log-sum-exp over the contracted axes of ``log(weight) + log-operands``,
usable on small shapes; the tests compare the two families.
"""

from __future__ import annotations

import numpy as np
import torch
from scipy.special import logsumexp

CLAMP = 1e38  # baselines/lm2exp.py:12


def _f64(t, device="cpu") -> torch.Tensor:
    return torch.as_tensor(t).detach().to(device, torch.float64)


def lm2exp64(a, b, *, device="cpu") -> torch.Tensor:
    """c[r,i,k] = log sum_j a[r,i,j] exp b[r,j,k]; recipe of baselines/lm2exp.py:11-14.
    ``device``: where torch evaluates it (the CPU; or the GPU, whose float64 ATen / BLAS
    routines share nothing with the kernels under test, for full-size inputs)."""
    a, b = _f64(a, device), _f64(b, device)
    m = torch.amax(b, dim=1, keepdim=True)
    m = torch.clamp(m, -CLAMP, CLAMP)
    r = torch.bmm(a, torch.exp(b - m))
    return m + torch.log(r)


def lt2exp64(w, a, b, *, batch_chunk: int = 1, device="cpu") -> torch.Tensor:
    """c[r,s,k] = log sum_ij w[r,s,i,j] exp a[r,i,k] exp b[r,j,k]; recipe of
    baselines/lt2exp.py:15-25, evaluated ``batch_chunk`` batches at a time so the
    R x (I*J) x K intermediate stays small.  ``device`` as for lm2exp64."""
    w, a, b = _f64(w, device), _f64(a, device), _f64(b, device)
    R, S, I, J = w.shape
    K = a.shape[2]
    out = torch.empty((R, S, K), dtype=torch.float64, device=device)
    for r0 in range(0, R, batch_chunk):
        sl = slice(r0, min(R, r0 + batch_chunk))
        ma = torch.clamp(torch.amax(a[sl], dim=1, keepdim=True), -CLAMP, CLAMP)
        mb = torch.clamp(torch.amax(b[sl], dim=1, keepdim=True), -CLAMP, CLAMP)
        ea = torch.exp(a[sl] - ma)
        eb = torch.exp(b[sl] - mb)
        s = (ea.unsqueeze(2) * eb.unsqueeze(1)).reshape(ea.shape[0], I * J, K)
        r = torch.bmm(w[sl].reshape(-1, S, I * J), s)
        out[sl] = ma + mb + torch.log(r)
    return out


def lm2exp_lse(a, b) -> np.ndarray:
    """Closed form: logsumexp_j(log a[r,i,j] + b[r,j,k]) with scipy (small shapes)."""
    a = np.asarray(_f64(a))
    b = np.asarray(_f64(b))
    with np.errstate(divide="ignore"):
        la = np.log(a)
    t = la[:, :, :, None] + b[:, None, :, :]  # R I J K
    with np.errstate(invalid="ignore"):
        return logsumexp(t, axis=2)


def lt2exp_lse(w, a, b) -> np.ndarray:
    """Closed form: logsumexp_{i,j}(log w[r,s,i,j] + a[r,i,k] + b[r,j,k]) with scipy."""
    w = np.asarray(_f64(w))
    a = np.asarray(_f64(a))
    b = np.asarray(_f64(b))
    with np.errstate(divide="ignore"):
        lw = np.log(w)
    t = lw[:, :, :, :, None] + a[:, None, :, None, :] + b[:, None, None, :, :]  # R S I J K
    with np.errstate(invalid="ignore"):
        return logsumexp(t, axis=(2, 3))


def compare(result, oracle, *, rtol: float = 1e-4, atol: float = 1e-5) -> dict:
    """The accuracy gate: fp32 result against a float64 oracle.

    -inf positions must coincide exactly, no NaN may appear where the oracle has
    none, and finite entries must satisfy |x - y| <= atol + rtol * |y|.
    """
    x = np.asarray(torch.as_tensor(result).detach().to("cpu", torch.float64))
    y = np.asarray(torch.as_tensor(oracle).detach().to("cpu", torch.float64))
    assert x.shape == y.shape, (x.shape, y.shape)
    nan_extra = int(np.sum(np.isnan(x) & ~np.isnan(y)))
    ninf_x, ninf_y = np.isneginf(x), np.isneginf(y)
    inf_mismatch = int(np.sum(ninf_x != ninf_y))
    fin = np.isfinite(y) & np.isfinite(x)
    err = np.abs(x[fin] - y[fin])
    tol = atol + rtol * np.abs(y[fin])
    worst = float(np.max(err / tol)) if err.size else 0.0
    nonfinite_mismatch = int(np.sum(np.isfinite(x) != np.isfinite(y)))
    return {
        "ok": nan_extra == 0 and inf_mismatch == 0 and nonfinite_mismatch == 0 and worst <= 1.0,
        "nan_extra": nan_extra,
        "neg_inf_mismatch": inf_mismatch,
        "nonfinite_mismatch": nonfinite_mismatch,
        "worst_err_over_tol": worst,
        "max_abs_err": float(np.max(err)) if err.size else 0.0,
        "n_neg_inf": int(np.sum(ninf_y)),
    }
