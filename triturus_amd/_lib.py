"""ctypes binding of the C-ABI library (include/triturus_hip.h).

The library is the only compute path.  If it has not been built, or a call
reports a non-zero status, a RuntimeError is raised: there is no fallback.
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, c_char_p, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libtriturus_hip.so"
ABI_VERSION = 9

TRT_F32, TRT_F64, TRT_F16, TRT_BF16 = 0, 1, 2, 3
MODE_AUTO, MODE_SPLIT, MODE_UNSPLIT = 0, 1, 2
STATIC_SCRATCH_BYTES = 16 << 20  # TRT_STATIC_SCRATCH_BYTES
E_SCRATCH = -5
E_STATE = -6

DTYPE_CODES = {
    torch.float32: TRT_F32,
    torch.float64: TRT_F64,
    torch.float16: TRT_F16,
    torch.bfloat16: TRT_BF16,
}

_I64x3 = c_int64 * 3

# name -> (restype, argtypes); mirrors include/triturus_hip.h one to one
SIGNATURES = {
    "trt_version": (c_int, []),
    "trt_error_string": (c_char_p, [c_int]),
    "trt_lm2exp_f32": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
         POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_lm2exp_bf16": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
         POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_lm2exp_bf16_variant_count": (c_int, []),
    "trt_lm2exp_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int, c_int]),
    "trt_lm2exp_variant_count": (c_int, []),
    "trt_lt2exp_f32": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
         c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_lt2exp_f32_static": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
         c_int, c_int, c_void_p],
    ),
    "trt_lt2exp_bf16": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
         POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
         c_int, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_lt2exp_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int]),
    "trt_lm2exp_bf16_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int, c_int]),
    "trt_lt2exp_bf16_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int]),
    "trt_lt2exp_variant_count": (c_int, []),
    "trt_matmax": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_matmax_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int, c_int]),
    "trt_vmax": (
        c_int,
        [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "trt_vmax_workspace_bytes": (c_size_t, [c_int64, c_int]),
    "trt_colmax_batched_f32": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int64, POINTER(c_int64), c_int, c_void_p, c_size_t, c_void_p],
    ),
    "trt_colmax_batched_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "trt_mm_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_size_t,
                           c_void_p]),
    "trt_mm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int, c_int]),
    "trt_mm_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t,
                            c_void_p]),
    "trt_vadd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "trt_copy_bytes": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "trt_max_workspace_init": (c_int, [c_void_p, c_size_t, c_void_p]),
    "trt_max_workspace_check": (c_int, [c_void_p, c_size_t, c_void_p]),
    "trt_stream_capture_id": (c_int, [c_void_p, POINTER(ctypes.c_ulonglong)]),
    "trt_lt2exp_kernel_name": (c_int, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_char_p, c_size_t]),
    "trt_lm2exp_kernel_name": (c_int, [c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_char_p, c_size_t]),
}

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None


def load() -> ctypes.CDLL:
    """Load the HIP library once; raise if it is missing or of another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m triturus_amd.build` "
                "(hipcc, gfx950). There is no CPU or eager fallback."
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if a declared symbol is absent
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.trt_version() != ABI_VERSION:
            raise RuntimeError(
                f"{LIB_PATH} has ABI version {lib.trt_version()}, expected {ABI_VERSION}: rebuild it"
            )
        _lib = lib
        return lib


def check(status: int, what: str) -> None:
    if status != 0:
        text = load().trt_error_string(status)
        raise RuntimeError(f"{what} failed with status {status}: {text.decode() if text else '?'}")


def kernel_name(op: str, *args: int) -> str:
    """Profiler name of the contraction kernel a call launches (trt_lt2exp_kernel_name / trt_lm2exp_kernel_name)."""
    buf = ctypes.create_string_buffer(160)
    check(getattr(load(), f"trt_{op}_kernel_name")(*args, buf, len(buf)), f"trt_{op}_kernel_name")
    return buf.value.decode()


_stride_arrays: dict = {}  # stride tuple -> ctypes array (read-only to the library, so shareable)


def strides3(t: torch.Tensor):
    return stride_array(t.stride())


def stride_array(st: tuple):
    """ctypes int64[3] of an element-stride tuple, cached: building one costs as much as a dict lookup
    saves on the small calls that are bound by the host."""
    arr = _stride_arrays.get(st)
    if arr is None:
        if len(_stride_arrays) > 4096:
            _stride_arrays.clear()
        arr = _stride_arrays[st] = _I64x3(*st)
    return arr


def current_stream(device: torch.device) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


try:  # the raw hipStream_t of torch's current stream without building a Stream object
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover - older / newer torch without the helper
    _raw_stream = None


def raw_stream(device: torch.device) -> int:
    """hipStream_t (as an integer) of torch's current stream on `device`."""
    if _raw_stream is not None:
        idx = device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


try:  # the current device ordinal without torch.cuda's lazy-init checks
    _get_device = torch._C._cuda_getDevice
except AttributeError:  # pragma: no cover
    _get_device = torch.cuda.current_device


def on_device(device: torch.device):
    """Context that makes `device` current for the launch; free when it already is."""
    idx = device.index
    if idx is None or idx == _get_device():
        return _NO_SWITCH
    return torch.cuda.device(device)



def require_gpu(*tensors: torch.Tensor) -> None:
    """The kernels run on HIP device memory only."""
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                f"triturus_amd runs on the GPU only: got a tensor on '{t.device}'. "
                "Move the inputs to the HIP device (there is no CPU fallback)."
            )
