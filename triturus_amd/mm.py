"""mm: fp32 matrix product on MI355X.

Same contract as the reference wrapper, triturus/mm.py:181-214: a is m x k, b is k x n, both
contiguous fp32 on one device; returns a fresh m x n tensor.  The contraction runs in IEEE
fp32 on the fp32 matrix pipe whatever the TF32 flag says (tighter than the flag asks for).
Not part of the log-space path: provided so that the reference's module surface is complete.
"""

from __future__ import annotations

import torch

from triturus_amd import _lib


def mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
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
    with _lib.on_device(a.device):
        status = lib.trt_mm_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, k, n, _lib.raw_stream(a.device))
    if status:
        _lib.check(status, "trt_mm_f32")
    return c
