"""vamax / vmax / matmax on MI355X.

Same contracts as the reference wrappers, triturus/max.py:35-59, 96-122,
171-226: contiguous floating-point input; ``vmax`` returns two 0-d tensors
(value, int64 index of the first maximum); ``matmax`` returns a 1-d tensor of
the maxima along ``axis``.  ``block_size`` is accepted for signature
compatibility and ignored: each reduction streams its input once.
NaN handling follows torch.amax / torch.max (NaN propagates).
"""

from __future__ import annotations

import torch

from triturus_amd import _lib

_ws_bytes: dict = {}  # (op, shape..., dtype code) -> workspace bytes, as reported by the library
# (device index, raw stream) -> workspace of the reductions launched on that stream.  The library
# wants the arrival counters at the head of a max workspace zero before the first use and leaves
# them zero (one launch per reduction: the workgroup that finishes last combines the partial
# results), so the workspace is allocated once per stream, zero-filled, and kept: calls on one
# stream run one after the other, calls on different streams never share one.
_workspaces: dict = {}
# Workspaces that a larger one has replaced.  They are kept for the life of the process: a HIP
# graph captured while one of them was current still launches kernels that count in it.
_retired: list = []


def _workspace(dev: torch.device, nbytes: int):
    key = (dev.index, _lib.raw_stream(dev))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
            nbytes = max(nbytes, 2 * ws.numel())  # grow geometrically: what is retired stays below what is live
        ws = _workspaces[key] = torch.zeros(max(nbytes, 1 << 16), dtype=torch.uint8, device=dev)
    return ws


def _dtype_code(x: torch.Tensor) -> int:
    try:
        return _lib.DTYPE_CODES[x.dtype]
    except KeyError:
        raise NotImplementedError(f"max reductions support fp32/fp64/fp16/bf16, got {x.dtype}") from None


def _vmax_impl(x: torch.Tensor, with_index: bool):
    _lib.require_gpu(x)
    lib = _lib.load()
    code = _dtype_code(x)
    n = x.shape[0]
    if n == 0:
        raise RuntimeError("max of an empty vector")
    dev = x.device
    val = torch.empty((), dtype=x.dtype, device=dev)
    idx = torch.empty((), dtype=torch.int64, device=dev) if with_index else None
    key = ("v", n, code)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = _ws_bytes[key] = lib.trt_vmax_workspace_bytes(n, code)
    ws = _workspace(dev, ws_bytes) if ws_bytes else None
    with _lib.on_device(dev):
        status = lib.trt_vmax(
            x.data_ptr(), n, code, val.data_ptr(), idx.data_ptr() if with_index else None,
            ws.data_ptr() if ws_bytes else None, ws_bytes, _lib.raw_stream(dev),
        )
    if status:
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
    dev = x.device
    y = torch.empty(n if axis == 0 else m, dtype=x.dtype, device=dev)
    key = ("m", m, n, axis, code)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = _ws_bytes[key] = lib.trt_matmax_workspace_bytes(m, n, axis, code)
    ws = _workspace(dev, ws_bytes) if ws_bytes else None
    with _lib.on_device(dev):
        status = lib.trt_matmax(
            x.data_ptr(), y.data_ptr(), m, n, axis, code,
            ws.data_ptr() if ws_bytes else None, ws_bytes, _lib.raw_stream(dev),
        )
    if status:
        _lib.check(status, "trt_matmax")
    return y


def bmatmax(x: torch.Tensor, *, clamp: bool = False) -> torch.Tensor:
    """Batched column maxima: ``torch.amax(x, dim=1)`` of an R x J x K fp32 tensor, R x K.

    The reference reduces 2-D matrices only (``matmax``, triturus/max.py:125-188); this is the
    batched form along axis 1 that the contraction recipes start with
    (baselines/lm2exp.py:11, baselines/lt2exp.py:15,18).  With ``clamp`` the maxima are clamped
    to +-1e38 as there (baselines/lm2exp.py:12): the shift the contraction kernels subtract.
    """
    assert len(x.shape) == 3
    assert x.dtype == torch.float32
    _lib.require_gpu(x)
    lib = _lib.load()
    R, J, K = x.shape
    if R == 0 or K == 0:
        return torch.empty((R, K), dtype=x.dtype, device=x.device)
    if J == 0:
        raise RuntimeError("max over an empty axis")
    st = x.stride()
    if st[-1] != 1 or min(st) < 0:  # zero strides (an expanded operand) are read in place
        x = x.contiguous()
    m = torch.empty((R, K), dtype=x.dtype, device=x.device)
    key = ("b", R, J, K)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = _ws_bytes[key] = lib.trt_colmax_batched_workspace_bytes(R, J, K)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    with _lib.on_device(x.device):
        status = lib.trt_colmax_batched_f32(
            x.data_ptr(), m.data_ptr(), R, J, K, _lib.strides3(x), int(bool(clamp)),
            ws.data_ptr() if ws_bytes else None, ws_bytes, _lib.raw_stream(x.device),
        )
    if status:
        _lib.check(status, "trt_colmax_batched_f32")
    return m
