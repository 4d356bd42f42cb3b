"""Operands beyond 4 GiB: 288 GB of HBM hold calls whose tensors no 32-bit byte offset spans,
so batch, row and element offsets must be 64-bit wherever they can grow that far.  The
batches at the far end of each operand are checked against the float64 oracle (a wrapped
offset would read or write the wrong batch there), the reductions against torch.  A single
batch slice beyond what the kernels index is refused with an error, never truncated."""

import pytest
import torch

from oracle import oracle64
from triturus.lm2exp import lm2exp
from triturus.lt2exp import lt2exp
from triturus.max import matmax, vamax, vmax
from triturus_amd.max import bmatmax

pytestmark = pytest.mark.gpu


@pytest.fixture
def big(dev):
    if torch.cuda.get_device_properties(dev).total_memory < (64 << 30):
        pytest.skip("needs 64 GB of device memory")
    yield dev
    torch.cuda.empty_cache()


@pytest.mark.parametrize("precision", ["fp32", "bf16x6"])
def test_lm2exp_with_b_and_c_beyond_4_gib(big, precision):
    R, I, J, K = 2048, 128, 256, 4096  # b: 8.6 GB, c: 4.3 GB
    a = torch.rand(R, I, J, device=big)
    b = torch.randn(R, J, K, device=big) * 5
    b[R - 1, :, 7] = float("-inf")
    c = lm2exp(a, b, _precision=precision)
    assert torch.isneginf(c[R - 1, :, 7]).all()
    for r0 in (0, 1023, R - 32):
        sl = slice(r0, r0 + 32)
        r = oracle64.compare(c[sl], oracle64.lm2exp64(a[sl], b[sl], device=big))
        assert r["ok"], (r0, r)


@pytest.mark.parametrize("precision", ["fp32", "bf16x6"])
def test_lt2exp_with_w_beyond_4_gib(big, precision):
    R, S, I, J, K = 4096, 64, 64, 64, 1024  # w: 4.3 GB
    w = torch.rand(R, S, I, J, device=big)
    a = torch.randn(R, I, K, device=big) * 3
    b = torch.randn(R, J, K, device=big) * 3
    c = lt2exp(w, a, b, _precision=precision)
    for r0 in (0, 2047, R - 8):
        sl = slice(r0, r0 + 8)
        r = oracle64.compare(c[sl], oracle64.lt2exp64(w[sl], a[sl], b[sl], batch_chunk=8, device=big))
        assert r["ok"], (r0, r)


def test_lt2exp_with_one_s_per_batch_and_w_beyond_4_gib(big):
    """The kernel that contracts j first (one s per batch): 64-bit batch offsets of w, a, b and c."""
    from triturus_amd import _lib

    R, S, I, J, K = 36000, 1, 128, 256, 16  # w: 4.7 GB
    assert "rows_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1)
    w = torch.rand(R, S, I, J, device=big)
    a = torch.randn(R, I, K, device=big) * 3
    b = torch.randn(R, J, K, device=big) * 3
    c = lt2exp(w, a, b)
    for r0 in (0, 17999, R - 8):
        sl = slice(r0, r0 + 8)
        r = oracle64.compare(c[sl], oracle64.lt2exp64(w[sl], a[sl], b[sl], batch_chunk=8, device=big))
        assert r["ok"], (r0, r)


def test_lm2exp_with_a_batch_of_b_beyond_2_gib(big):
    R, I, J, K = 2, 64, 8192, 70000  # 2.3 GB per batch of b
    a = torch.rand(R, I, J, device=big)
    b = torch.randn(R, J, K, device=big)
    c = lm2exp(a, b)
    r = oracle64.compare(c, oracle64.lm2exp64(a, b, device=big))
    assert r["ok"], r


def test_batches_beyond_the_index_range_are_refused(big):
    """One batch of b of 4.6 GB: an error, and nothing launched."""
    a = torch.rand(1, 32, 16384, device=big)
    b = torch.empty(1, 16384, 70000, device=big)
    with pytest.raises(RuntimeError, match="index range"):
        lm2exp(a, b)
    del a, b
    w = torch.empty(1, 1100, 1024, 1024, device=big)  # 4.6 GB in one batch
    a = torch.empty(1, 1024, 64, device=big)
    with pytest.raises(RuntimeError, match="index range"):
        lt2exp(w, a, a)


def test_vmax_beyond_2_to_the_32_elements(big):
    n = (1 << 32) + 12345
    x = torch.randn(n, device=big)
    first = (1 << 32) + 5
    x[first] = 9.0
    x[n - 7] = 9.0
    v, i = vmax(x)
    assert float(v) == 9.0 and int(i) == first
    assert float(vamax(x)) == 9.0


def test_matmax_and_bmatmax_beyond_4_gib(big):
    x = torch.randn(70001, 66000, device=big)  # 18.5 GB
    for axis in (0, 1):
        assert torch.equal(matmax(x, axis=axis), torch.amax(x, dim=axis))
    del x
    torch.cuda.empty_cache()
    x = torch.randn(3000, 700, 2100, device=big)  # 17.6 GB
    assert torch.equal(bmatmax(x), torch.amax(x, dim=1))
