"""Optional measured tile selection, the counterpart of the reference's ``@triton.autotune``
(triturus/lm2exp.py:61, triturus/lt2exp.py:225,360): the first call for a shape key times
every candidate tile variant with HIP events and later calls reuse the fastest.

Off by default -- the shape rules compiled into the library are within a few per cent of
the best variant on the reference's benchmark grid, and a measured choice may differ from
run to run (the results then differ in the last bits: another summation order).  Enable
with ``set_autotune(True)`` or ``TRITURUS_AUTOTUNE=1``.  Never measures while the current
stream is being captured into a graph: the rules are used there.
"""

from __future__ import annotations

import os
from typing import Callable, Hashable, Sequence

import torch

_enabled: bool = os.environ.get("TRITURUS_AUTOTUNE", "0") == "1"
_best: dict = {}
REPS = 3


def set_autotune(enabled: bool) -> None:
    global _enabled
    _enabled = bool(enabled)


def is_autotune_enabled() -> bool:
    return _enabled


def clear() -> None:
    _best.clear()


def chosen() -> dict:
    """Shape key -> variant picked so far (for inspection)."""
    return dict(_best)


def pick(key: Hashable, candidates: Sequence[int], launch: Callable[[int], object]) -> int:
    """Variant to use for `key`: 0 (the library's rule) unless tuning is on."""
    if not _enabled:
        return 0
    hit = _best.get(key)
    if hit is not None:
        return hit
    if torch.cuda.is_current_stream_capturing():
        return 0
    times = {}
    for v in candidates:
        launch(v)  # warm-up (also first-use costs of the kernel)
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(REPS):
            launch(v)
        stop.record()
        stop.synchronize()
        times[v] = start.elapsed_time(stop)
    best = min(times, key=times.get)
    _best[key] = best
    return best
