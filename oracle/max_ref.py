"""Brute-force max / first-occurrence arg-max with torch's NaN rule (NumPy).

Test infrastructure.  The reference tests compare against torch.amax and
torch.max (tests/max.py:13,22,32); these loops are an independent statement of
the same rule: a NaN wins over every number, and among equal winners the
lowest index is reported.
"""

from __future__ import annotations

import numpy as np


def vmax_ref(x) -> tuple[float, int]:
    x = np.asarray(x)
    nan = np.isnan(x)
    if nan.any():
        i = int(np.flatnonzero(nan)[0])
        return float("nan"), i
    best, bi = x[0], 0
    for i in range(1, x.shape[0]):
        if x[i] > best:
            best, bi = x[i], i
    return float(best), bi


def vmax_ref_fast(x) -> tuple[float, int]:
    """Vectorised equivalent of ``vmax_ref`` for large inputs."""
    x = np.asarray(x)
    nan = np.isnan(x)
    if nan.any():
        return float("nan"), int(np.argmax(nan))
    i = int(np.argmax(x))  # numpy returns the first maximum
    return float(x[i]), i


def matmax_ref(x, axis: int) -> np.ndarray:
    x = np.asarray(x)
    out = np.max(x, axis=axis)  # np.max propagates NaN
    return out
