"""Global flags and seeding, same names as the reference's triturus/utils.py.

``set_tf32_enabled`` / ``is_triturus_tf32_enabled`` (triturus/utils.py:33-53):
gfx950 has no TF32/xf32 matrix instruction.  With the flag off the kernels
contract in IEEE fp32 on the fp32 matrix pipe; with it on they run on the bf16
matrix pipe with every fp32 operand cut into two bf16 pieces ("bf16x3": three
MFMAs per product, ~2^-16 relative error per product, fp32 accumulation) --
several times faster, and tighter than TF32 (2^-11) and than the rtol 5e-4 the
reference tests allow in that mode (tests/lm2exp.py:21).
``set_matrix_precision`` (no counterpart in the reference) picks the arithmetic
explicitly: "fp32", "bf16x3", or "bf16x6" (three pieces, six MFMAs, ~2^-23 per
product: as accurate as the fp32 pipe and faster); ``None`` follows the flag.
``ensure_reproducibility`` (triturus/utils.py:12-30) seeds python, numpy and
torch and makes the GPU the default device when one is present.
Both functions also write the same torch-side settings as the reference
(float32 matmul precision and the two ``allow_tf32`` backends; cudnn
benchmarking, the BLAS workspace variable and the dynamo recompile limit), so
that torch code run beside these kernels -- the "torch" line of a benchmark --
computes under the same settings as it does beside the reference.
"""

from __future__ import annotations

import os
import random

import numpy as np
import torch

_TRITURUS_TF32_ENABLED: bool = False
_MATRIX_PRECISION: str | None = None
MATRIX_PRECISIONS = ("fp32", "bf16x3", "bf16x6")


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
        # every kernel of this library is deterministic (fixed summation order; the
        # only atomics are the arrival counters of the max reductions, which decide who
        # combines the partial results, never the result); the flag only concerns torch's own ops
        torch.use_deterministic_algorithms(True, warn_only=True)
        torch.backends.cudnn.benchmark = False
        os.environ["CUBLAS_WORKSPACE_CONFIG"] = ":16:8"
    try:  # triturus/utils.py:30
        torch._dynamo.config.recompile_limit = 64
    except Exception:  # a torch build without dynamo: nothing to configure
        pass


def set_tf32_enabled(allow_tf32: bool) -> None:
    """triturus/utils.py:33-44: the library's own flag and torch's matmul settings together."""
    global _TRITURUS_TF32_ENABLED
    if allow_tf32:
        torch.set_float32_matmul_precision("high")
        torch.backends.cuda.matmul.allow_tf32 = True
        torch.backends.cudnn.allow_tf32 = True
        _TRITURUS_TF32_ENABLED = True
    else:
        torch.set_float32_matmul_precision("highest")
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        _TRITURUS_TF32_ENABLED = False


def is_torch_tf32_enabled() -> bool:
    """triturus/utils.py:47-48."""
    return bool(torch.backends.cuda.matmul.allow_tf32 and torch.backends.cudnn.allow_tf32)


def is_triturus_tf32_enabled() -> bool:
    return _TRITURUS_TF32_ENABLED


def set_matrix_precision(precision: str | None) -> None:
    """Arithmetic of the lm2exp / lt2exp contractions; None = follow the TF32 flag."""
    global _MATRIX_PRECISION
    if precision is not None and precision not in MATRIX_PRECISIONS:
        raise ValueError(f"unknown matrix precision {precision!r}: expected one of {MATRIX_PRECISIONS} or None")
    _MATRIX_PRECISION = precision


def pinned_matrix_precision() -> str | None:
    """What set_matrix_precision pinned, or None while the TF32 flag decides."""
    return _MATRIX_PRECISION


def matrix_precision() -> str:
    """The arithmetic the next lm2exp / lt2exp call will use."""
    if _MATRIX_PRECISION is not None:
        return _MATRIX_PRECISION
    return "bf16x3" if _TRITURUS_TF32_ENABLED else "fp32"
