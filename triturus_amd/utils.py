"""Global flags and seeding, same names as the reference's triturus/utils.py.

``set_tf32_enabled`` / ``is_triturus_tf32_enabled`` (triturus/utils.py:33-53):
the flag is recorded, but gfx950 has no TF32/xf32 matrix instruction, so the
kernels always contract in IEEE fp32 -- strictly tighter than the rtol 5e-4
the reference tests allow when the flag is on (tests/lm2exp.py:21).
``ensure_reproducibility`` (triturus/utils.py:12-30) seeds python, numpy and
torch and makes the GPU the default device when one is present.
"""

from __future__ import annotations

import random

import numpy as np
import torch

_TRITURUS_TF32_ENABLED: bool = False


def ensure_reproducibility(
    *,
    seed: int = 42,
    determinism: bool = False,
    device: torch.device | int | str | None = None,
) -> None:
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if device is None:
        if torch.cuda.is_available():
            torch.set_default_device("cuda")
    else:
        torch.set_default_device(device)
    if determinism:
        # every kernel of this library is deterministic (fixed summation order,
        # no atomics); the flag only concerns torch's own ops
        torch.use_deterministic_algorithms(True, warn_only=True)


def set_tf32_enabled(allow_tf32: bool) -> None:
    global _TRITURUS_TF32_ENABLED
    _TRITURUS_TF32_ENABLED = bool(allow_tf32)


def is_triturus_tf32_enabled() -> bool:
    return _TRITURUS_TF32_ENABLED
