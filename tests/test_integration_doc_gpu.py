"""The reference-side binding shown in the integration guide at the repository root is executed as
written: the first python
block (the lm2exp stub) and the second (the lt2exp fragment) must run against the built library
and reproduce the package's own results."""

import re
from pathlib import Path

import pytest
import torch

from triturus.lm2exp import lm2exp
from triturus.lt2exp import lt2exp
from triturus_amd import _lib

pytestmark = pytest.mark.gpu
DOC = (Path(__file__).resolve().parent.parent / "INTEGRATION.md").read_text()


def test_documented_ctypes_stubs_run(dev):
    blocks = re.findall(r"```python\n(.*?)```", DOC, flags=re.S)
    assert len(blocks) >= 2
    stub = blocks[0].replace('ctypes.CDLL("libtriturus_hip.so")', f'ctypes.CDLL("{_lib.LIB_PATH}")')
    ns: dict = {}
    exec(compile(stub, "INTEGRATION.md:lm2exp", "exec"), ns)
    g = torch.Generator().manual_seed(2)
    a = torch.rand(3, 50, 70, generator=g).to(dev)
    b = torch.randn(3, 70, 90, generator=g).to(dev)
    c = torch.empty(3, 50, 90, device=dev)
    ns["_launch_lm2exp"](a, b, c)
    assert torch.equal(c, lm2exp(a, b))
    # a transposed a goes through the stub as it is (the library reads it in place)
    at = a.transpose(1, 2).contiguous().transpose(1, 2)
    assert at.stride(2) != 1
    ct = torch.empty(3, 50, 90, device=dev)
    ns["_launch_lm2exp"](at, b, ct)
    assert torch.equal(ct, lm2exp(at, b)) and torch.allclose(ct, c, rtol=1e-5, atol=1e-6)
    # a shape that splits over J (needs the workspace the stub allocates)
    a2 = torch.rand(1, 128, 4096, generator=g).to(dev)
    b2 = torch.randn(1, 4096, 128, generator=g).to(dev)
    c2 = torch.empty(1, 128, 128, device=dev)
    ns["_launch_lm2exp"](a2, b2, c2)
    assert torch.equal(c2, lm2exp(a2, b2))

    # the lt2exp fragment: runs in the scope the reference wrapper has at triturus/lt2exp.py:549
    batch, m, j, k, n = 3, 75, 50, 50, 100
    w = torch.rand(batch, m, j, k, generator=g).to(dev)
    a3 = torch.randn(batch, j, n, generator=g).to(dev)
    b3 = torch.randn(batch, k, n, generator=g).to(dev)
    lib = ns["_lib"]
    lib.trt_lt2exp_f32.restype = ns["ctypes"].c_int
    lib.trt_lt2exp_workspace_bytes.restype = ns["ctypes"].c_size_t
    sig = _lib.SIGNATURES
    lib.trt_lt2exp_f32.argtypes = sig["trt_lt2exp_f32"][1]
    lib.trt_lt2exp_workspace_bytes.argtypes = sig["trt_lt2exp_workspace_bytes"][1]
    for mode in ("auto", "split", "unsplit"):
        c3 = torch.empty(batch, m, n, device=dev)
        scope = dict(ns, w=w.view(batch, m, -1), a=a3, b=b3, c=c3, batch=batch, m=m, j=j, k=k, n=n, mode=mode)
        exec(compile(blocks[1], "INTEGRATION.md:lt2exp", "exec"), scope)
        assert scope["status"] == 0
        assert torch.equal(c3, lt2exp(w, a3, b3, mode=mode))
    # every other element of a wider w: the flattened view keeps the stride, the library reads it in place
    wide = torch.zeros(batch, m, j, 2 * k, device=dev)
    wide[..., ::2] = w
    ws_ = wide[..., ::2]
    c4 = torch.empty(batch, m, n, device=dev)
    scope = dict(ns, w=ws_.view(batch, m, -1), a=a3, b=b3, c=c4, batch=batch, m=m, j=j, k=k, n=n, mode="unsplit")
    assert scope["w"].stride(2) == 2
    exec(compile(blocks[1], "INTEGRATION.md:lt2exp", "exec"), scope)
    assert scope["status"] == 0
    assert torch.equal(c4, lt2exp(ws_, a3, b3, mode="unsplit"))
    # (the dense w may run on another kernel than the strided view: the same values up to rounding)
    assert torch.allclose(c4, lt2exp(w, a3, b3, mode="unsplit"), rtol=1e-5, atol=1e-5)
