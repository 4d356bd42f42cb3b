"""mm: fp32 matrix product on MI355X.

Same contract as the reference wrapper, triturus/mm.py:181-214: a is m x k, b is k x n, both
contiguous fp32 on one device; returns a fresh m x n tensor.  The contraction runs in IEEE
fp32 on the fp32 matrix pipe; with the reference's TF32 flag on (triturus/mm.py:198) it runs on
the bf16 matrix pipe with every operand cut into three bf16 pieces ("bf16x6": as accurate as
fp32, so the reference's own test tolerance still holds, and faster), or into two with
set_matrix_precision("bf16x3").  Not part of the log-space path: provided so that the
reference's module surface is complete.
"""

from __future__ import annotations

import torch

from triturus_amd import _lib
from triturus_amd.utils import is_triturus_tf32_enabled, pinned_matrix_precision


def mm(a: torch.Tensor, b: torch.Tensor, *, _precision: str | None = None) -> torch.Tensor:
    assert len(a.shape) == len(b.shape) == 2
    assert a.shape[1] == b.shape[0]
    assert a.dtype == b.dtype == torch.float32
    assert a.device == b.device
    assert a.is_contiguous() and b.is_contiguous()
    _lib.require_gpu(a, b)
    lib = _lib.load()
    m, k = a.shape
    n = b.shape[1]
    c = torch.empty((m, n), dtype=a.dtype, device=a.device)
    if c.numel() == 0:
        return c
    if k == 0:
        return c.zero_()
    # the flag alone selects three pieces: inside the reference's fp32-level test tolerance
    # (tests/mm.py:16 uses torch.allclose defaults with the flag on as well)
    precision = _precision or pinned_matrix_precision() or ("bf16x6" if is_triturus_tf32_enabled() else "fp32")
    with _lib.on_device(a.device):
        if precision == "fp32":
            status = lib.trt_mm_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, k, n, _lib.raw_stream(a.device))
        else:
            status = lib.trt_mm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, k, n,
                                     {"bf16x3": 2, "bf16x6": 3}[precision], _lib.raw_stream(a.device))
    if status:
        _lib.check(status, "trt_mm")
    return c
