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


_ws_bytes: dict = {}  # (m, k, n, row tile, cut) -> workspace bytes


def mm(a: torch.Tensor, b: torch.Tensor, *, _precision: str | None = None, _variant: int = 0,
       _splits: int = 0) -> torch.Tensor:
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
    # grids of few tiles are cut over k (the partial products meet in a workspace); _variant
    # and _splits force the row tile (1..4: 32..128 rows) and the cut (tests, timing)
    fp32 = precision == "fp32"
    key = (m, k, n, _variant if fp32 else 0, _splits if fp32 else 0)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = _ws_bytes[key] = lib.trt_mm_workspace_bytes(*key)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
    ws_ptr = ws.data_ptr() if ws_bytes else None
    with _lib.on_device(a.device):
        if fp32:
            status = lib.trt_mm_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, k, n, _variant, _splits,
                                    ws_ptr, ws_bytes, _lib.raw_stream(a.device))
        else:
            status = lib.trt_mm_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, k, n,
                                     {"bf16x3": 2, "bf16x6": 3}[precision], ws_ptr, ws_bytes,
                                     _lib.raw_stream(a.device))
    if status:
        _lib.check(status, "trt_mm")
    return c
