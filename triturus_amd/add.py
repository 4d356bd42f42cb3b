"""vadd: elementwise sum of two vectors on MI355X.

Same contract as the reference wrapper, triturus/add.py:32-46: x and y are 1-d, of one
shape, dtype and device, x contiguous; returns a fresh vector.  ``block_size`` is accepted
for signature compatibility and ignored.  Not part of the log-space path: provided so
that the reference's module surface is complete.
"""

from __future__ import annotations

import torch

from triturus_amd import _lib


def vadd(x: torch.Tensor, y: torch.Tensor, *, block_size: int = 512) -> torch.Tensor:
    assert len(x.shape) == len(y.shape) == 1
    assert x.shape == y.shape
    assert x.dtype == y.dtype
    assert x.device == y.device
    assert x.is_contiguous()
    _lib.require_gpu(x, y)
    lib = _lib.load()
    try:
        code = _lib.DTYPE_CODES[x.dtype]
    except KeyError:
        raise NotImplementedError(f"vadd supports fp32/fp64/fp16/bf16, got {x.dtype}") from None
    y = y.contiguous()
    r = torch.empty_like(x)
    n = x.shape[0]
    if n == 0:
        return r
    with _lib.on_device(x.device):
        status = lib.trt_vadd(x.data_ptr(), y.data_ptr(), r.data_ptr(), n, code, _lib.raw_stream(x.device))
    if status:
        _lib.check(status, "trt_vadd")
    return r
