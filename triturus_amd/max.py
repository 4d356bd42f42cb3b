"""vamax / vmax / matmax on MI355X.

Same contracts as the reference wrappers, triturus/max.py:35-59, 96-122,
171-226: contiguous floating-point input; ``vmax`` returns two 0-d tensors
(value, int64 index of the first maximum); ``matmax`` returns a 1-d tensor of
the maxima along ``axis``.  ``block_size`` is accepted for signature
compatibility and ignored: each reduction streams its input once.
NaN handling follows torch.amax / torch.max (NaN propagates).
"""

from __future__ import annotations

from ctypes import c_void_p

import torch

from triturus_amd import _lib


def _dtype_code(x: torch.Tensor) -> int:
    try:
        return _lib.DTYPE_CODES[x.dtype]
    except KeyError:
        raise NotImplementedError(f"max reductions support fp32/fp64/fp16/bf16, got {x.dtype}") from None


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor | None:
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def _vmax_impl(x: torch.Tensor, with_index: bool):
    _lib.require_gpu(x)
    lib = _lib.load()
    code = _dtype_code(x)
    n = x.shape[0]
    if n == 0:
        raise RuntimeError("max of an empty vector")
    val = torch.empty((), dtype=x.dtype, device=x.device)
    idx = torch.empty((), dtype=torch.int64, device=x.device) if with_index else None
    ws_bytes = lib.trt_vmax_workspace_bytes(n, code)
    ws = _workspace(ws_bytes, x.device)
    with _lib.on_device(x.device):
        status = lib.trt_vmax(
            c_void_p(x.data_ptr()), n, code, c_void_p(val.data_ptr()),
            c_void_p(idx.data_ptr() if idx is not None else None),
            c_void_p(ws.data_ptr() if ws is not None else None), ws_bytes,
            _lib.current_stream(x.device),
        )
    _lib.check(status, "trt_vmax")
    return val, idx


def vamax(x: torch.Tensor, *, block_size: int = 256) -> torch.Tensor:
    assert len(x.shape) == 1
    assert x.is_floating_point()
    assert x.is_contiguous()
    return _vmax_impl(x, False)[0]


def vmax(x: torch.Tensor, *, block_size: int = 256) -> tuple[torch.Tensor, torch.Tensor]:
    assert len(x.shape) == 1
    assert x.is_floating_point()
    assert x.is_contiguous()
    return _vmax_impl(x, True)


def matmax(x: torch.Tensor, axis: int = 0, *, block_size: int = 32) -> torch.Tensor:
    assert len(x.shape) == 2
    assert x.is_floating_point()
    assert x.is_contiguous()
    assert axis in {0, 1}
    _lib.require_gpu(x)
    lib = _lib.load()
    code = _dtype_code(x)
    m, n = x.shape
    if m == 0 or n == 0:
        raise RuntimeError("max of an empty matrix")
    y = torch.empty(n if axis == 0 else m, dtype=x.dtype, device=x.device)
    ws_bytes = lib.trt_matmax_workspace_bytes(m, n, axis, code)
    ws = _workspace(ws_bytes, x.device)
    with _lib.on_device(x.device):
        status = lib.trt_matmax(
            c_void_p(x.data_ptr()), c_void_p(y.data_ptr()), m, n, axis, code,
            c_void_p(ws.data_ptr() if ws is not None else None), ws_bytes,
            _lib.current_stream(x.device),
        )
    _lib.check(status, "trt_matmax")
    return y
