"""The library called from plain C: tests/c_abi/abi_caller.c knows only include/triturus_hip.h
and the HIP runtime (hipMalloc'd buffers, the null stream, no torch anywhere in its process).
What it writes back is checked against the float64 oracle and against the Python wrappers,
which reach the same entry points through ctypes: same library, same shape rules, so the same
bits.  A non-GPU test checks that the program was built and links against the in-tree library."""

import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import max_ref, oracle64

CALLER = Path(__file__).resolve().parent / "c_abi" / "abi_caller"


def run(tmp_path, op, *sizes, **operands):
    assert CALLER.exists(), "tests/c_abi/abi_caller is not built: run __graft_entry__.build()"
    for name, t in operands.items():
        np.ascontiguousarray(t.numpy()).tofile(tmp_path / f"{name}.bin")
    print("abi_caller", op, *sizes, flush=True)
    res = subprocess.run([str(CALLER), op, str(tmp_path), *map(str, sizes)], capture_output=True, text=True,
                         timeout=100)
    assert res.returncode == 0, res.stderr
    return lambda name, dtype=np.float32: torch.from_numpy(np.fromfile(tmp_path / f"{name}.bin", dtype=dtype))


def test_the_c_caller_is_built_against_the_in_tree_library():
    assert CALLER.exists(), "tests/c_abi/abi_caller is not built: run __graft_entry__.build()"
    out = subprocess.run(["ldd", str(CALLER)], capture_output=True, text=True).stdout
    lib = Path(__file__).resolve().parents[1] / "triturus_amd" / "lib" / "libtriturus_hip.so"
    found = [line.split("=>")[1].split()[0] for line in out.splitlines() if line.strip().startswith("libtriturus_hip.so")]
    assert found and Path(found[0]).resolve() == lib.resolve(), out


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(4, 64, 64, 64), (3, 70, 45, 130), (1, 512, 2048, 256)])
def test_lm2exp_from_c(dev, tmp_path, shape):
    from triturus.lm2exp import lm2exp

    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    b = torch.randn(R, J, K, generator=g) * 4 - 10
    b[0, :, 3] = float("-inf")
    c = run(tmp_path, "lm2exp", R, I, J, K, a=a, b=b)("c").view(R, I, K)
    r = oracle64.compare(c, oracle64.lm2exp64(a, b))
    assert r["ok"], r
    assert torch.equal(c, lm2exp(a.to(dev), b.to(dev)).cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("shape", [(2, 48, 32, 32, 256), (1, 40, 9, 21, 100), (1, 64, 64, 64, 512)])
def test_lt2exp_from_c(dev, tmp_path, shape, mode):
    from triturus.lt2exp import lt2exp

    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    a = torch.randn(R, I, K, generator=g) * 3 - 5
    b = torch.randn(R, J, K, generator=g) * 3 - 5
    a[0, :, 1] = float("-inf")
    c = run(tmp_path, "lt2exp", R, S, I, J, K, mode, w=w, a=a, b=b)("c").view(R, S, K)
    r = oracle64.compare(c, oracle64.lt2exp64(w, a, b))
    assert r["ok"], r
    # the wrapper's own front ends (copies for unaligned or short rows) are off: the C program
    # hands the operands over as they are
    ref = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=("auto", "split", "unsplit")[mode], _pad=False, _swap=False)
    assert torch.equal(c, ref.cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 1000, 1 << 20, (1 << 22) + 3])
def test_vmax_from_c(dev, tmp_path, n):
    g = torch.Generator().manual_seed(n)
    x = torch.randint(-50, 50, (n,), generator=g).float()  # ties: the first one is reported
    out = run(tmp_path, "vmax", n, x=x)
    val, idx = max_ref.vmax_ref_fast(x.numpy())
    assert float(out("val")[0]) == float(val)
    assert int(out("idx", np.int64)[0]) == int(idx)


@pytest.mark.gpu
@pytest.mark.parametrize("axis", [0, 1])
@pytest.mark.parametrize("shape", [(64, 4096), (4096, 4096), (1000, 37)])
def test_matmax_from_c(dev, tmp_path, shape, axis):
    m, n = shape
    g = torch.Generator().manual_seed(m + n + axis)
    x = torch.randn(m, n, generator=g)
    y = run(tmp_path, "matmax", m, n, axis, x=x)("y")
    assert torch.equal(y, torch.amax(x, dim=axis))
