"""ctypes front end of the plain C restatement (oracle_c.c).  Test infrastructure.

Each function takes CPU tensors / arrays as the kernels would get them (fp32, any strides:
they are made contiguous) and returns what the C loops computed in double precision.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_double, c_float, c_int, c_int64

import numpy as np
import torch

from oracle.build_c import LIB, build_oracle_c

_lib = None


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            build_oracle_c()
        lib = ctypes.CDLL(str(LIB))
        f32, f64, i64 = POINTER(c_float), POINTER(c_double), c_int64
        lib.lm2exp_c.argtypes = [f32, f32, f64, i64, i64, i64, i64]
        lib.lt2exp_c.argtypes = [f32, f32, f32, f64, i64, i64, i64, i64, i64]
        lib.vmax_c.argtypes = [f32, i64, f32, POINTER(c_int64)]
        lib.matmax_c.argtypes = [f32, f32, i64, i64, c_int]
        for fn in (lib.lm2exp_c, lib.lt2exp_c, lib.vmax_c, lib.matmax_c):
            fn.restype = None
        _lib = lib
    return _lib


def _f32(t) -> np.ndarray:
    return np.ascontiguousarray(torch.as_tensor(t).detach().to("cpu", torch.float32).numpy())


def _p(x: np.ndarray, ty):
    return x.ctypes.data_as(POINTER(ty))


def lm2exp_c(a, b) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    R, I, J = a.shape
    K = b.shape[2]
    assert b.shape[:2] == (R, J)
    c = np.empty((R, I, K), dtype=np.float64)
    _load().lm2exp_c(_p(a, c_float), _p(b, c_float), _p(c, c_double), R, I, J, K)
    return c


def lt2exp_c(w, a, b) -> np.ndarray:
    w, a, b = _f32(w), _f32(a), _f32(b)
    R, S, I, J = w.shape
    K = a.shape[2]
    assert a.shape[:2] == (R, I) and b.shape == (R, J, K)
    c = np.empty((R, S, K), dtype=np.float64)
    _load().lt2exp_c(_p(w, c_float), _p(a, c_float), _p(b, c_float), _p(c, c_double), R, S, I, J, K)
    return c


def vmax_c(x) -> tuple[float, int]:
    x = _f32(x).reshape(-1)
    val, idx = c_float(), c_int64()
    _load().vmax_c(_p(x, c_float), x.size, ctypes.byref(val), ctypes.byref(idx))
    return val.value, idx.value


def matmax_c(x, axis: int) -> np.ndarray:
    x = _f32(x)
    m, n = x.shape
    y = np.empty(n if axis == 0 else m, dtype=np.float32)
    _load().matmax_c(_p(x, c_float), _p(y, c_float), m, n, axis)
    return y
