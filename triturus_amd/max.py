"""vamax / vmax / matmax on MI355X.

Same contracts as the reference wrappers, triturus/max.py:35-59, 96-122,
171-226: contiguous floating-point input; ``vmax`` returns two 0-d tensors
(value, int64 index of the first maximum); ``matmax`` returns a 1-d tensor of
the maxima along ``axis``.  ``block_size`` is accepted for signature
compatibility and ignored: each reduction streams its input once.
NaN handling follows torch.amax / torch.max (NaN propagates).
"""

from __future__ import annotations

import ctypes
import os
from collections import OrderedDict

import torch

from triturus_amd import _lib

_ws_bytes: dict = {}  # (op, shape..., dtype code) -> workspace bytes, as reported by the library

# The library wants the arrival counters at the head of a max workspace idle before the first
# use (trt_max_workspace_init) and leaves them idle (one launch per reduction: the workgroup
# that finishes last combines the partial results).  So a workspace is allocated and prepared
# once per device and stream and kept: calls on one stream run one after the other, calls on
# different streams never share one.  At most _MAX_STREAMS of them are kept, the least recently
# used one going first (the allocator hands its block to later work on the same stream only).
# The key is the raw stream handle: a stream created after another one was destroyed may get its
# handle and with it its workspace, which is as good as a new one -- every call leaves it idle.
_MAX_STREAMS = 16
_workspaces: "OrderedDict[tuple, torch.Tensor]" = OrderedDict()  # (device index, raw stream) -> workspace
# A stream that is being captured into a HIP graph gets a workspace of its own per capture,
# allocated inside the capture (from the graph's memory pool) and prepared by a kernel node of
# that graph: whatever is prepared while capturing is idle only once the graph runs, so it must
# never serve an eager call, and an eager workspace must never serve a graph (the replays would
# count in it while eager calls on the stream do).  (device index, raw stream) -> (capture id,
# workspace); the entry of a finished capture is dropped when the stream is next seen -- the
# graph's pool keeps the block for the replays.
_capture_workspaces: dict = {}
_CHECK = os.environ.get("TRITURUS_CHECK_WORKSPACE", "0") not in ("", "0")  # debugging: verify the counters before every call

try:
    _is_capturing = torch._C._cuda_isCurrentStreamCapturing
except AttributeError:  # pragma: no cover
    _is_capturing = torch.cuda.is_current_stream_capturing


def _new_workspace(dev: torch.device, nbytes: int, stream: int) -> torch.Tensor:
    ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=dev)
    with _lib.on_device(dev):
        _lib.check(_lib.load().trt_max_workspace_init(ws.data_ptr(), ws.numel(), stream), "trt_max_workspace_init")
    return ws


def _workspace(dev: torch.device, nbytes: int, stream: int):
    key = (dev.index, stream)
    if _is_capturing():  # the callers hold a tensor on `dev`, so the runtime is up
        cid = ctypes.c_ulonglong(0)
        _lib.check(_lib.load().trt_stream_capture_id(stream, ctypes.byref(cid)), "trt_stream_capture_id")
        if cid.value:
            held = _capture_workspaces.get(key)
            if held is None or held[0] != cid.value or held[1].numel() < nbytes:
                held = _capture_workspaces[key] = (cid.value, _new_workspace(dev, nbytes, stream))
            return held[1]
    if _capture_workspaces:
        _capture_workspaces.pop(key, None)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            nbytes = max(nbytes, 2 * ws.numel())  # grow geometrically
        ws = _workspaces[key] = _new_workspace(dev, nbytes, stream)
        while len(_workspaces) > _MAX_STREAMS:
            _workspaces.popitem(last=False)
    else:
        _workspaces.move_to_end(key)
        if _CHECK:
            with _lib.on_device(dev):
                _lib.check(_lib.load().trt_max_workspace_check(ws.data_ptr(), ws.numel(), stream),
                           "trt_max_workspace_check")
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
    stream = _lib.raw_stream(dev)
    ws = _workspace(dev, ws_bytes, stream) if ws_bytes else None
    with _lib.on_device(dev):
        status = lib.trt_vmax(
            x.data_ptr(), n, code, val.data_ptr(), idx.data_ptr() if with_index else None,
            ws.data_ptr() if ws_bytes else None, ws_bytes, stream,
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
    stream = _lib.raw_stream(dev)
    ws = _workspace(dev, ws_bytes, stream) if ws_bytes else None
    with _lib.on_device(dev):
        status = lib.trt_matmax(
            x.data_ptr(), y.data_ptr(), m, n, axis, code,
            ws.data_ptr() if ws_bytes else None, ws_bytes, stream,
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
