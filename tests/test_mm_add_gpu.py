"""mm and vadd on the GPU: the reference's own tests (tests/mm.py:8-16, tests/add.py:6-12)
plus ragged and large shapes.  mm is checked against a float64 product (the oracle for a
plain matrix product is the product itself in higher precision) and against torch.mm."""

import pytest
import torch

from triturus.add import vadd
from triturus.mm import mm
from triturus.utils import set_tf32_enabled

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("allow_tf32", [False, True])
def test_mm(dev, allow_tf32):
    """The reference's test: 150 x 100 x 200, rand inputs, torch.allclose defaults."""
    set_tf32_enabled(allow_tf32)
    m, k, n = 150, 100, 200
    a = torch.rand(m, k, device=dev)
    b = torch.rand(k, n, device=dev)
    c = mm(a, b)
    assert c.shape == (m, n) and c.dtype == torch.float32
    assert torch.allclose(torch.mm(a, b), c)
    assert torch.allclose((a.double() @ b.double()).float(), c)


@pytest.mark.parametrize("shape", [(1, 1, 1), (33, 7, 31), (64, 64, 64), (300, 52, 129), (129, 1000, 257),
                                   (2048, 512, 1024), (4096, 300, 4096), (3072, 200, 3072), (285, 70, 16400)])
def test_mm_shapes(dev, shape):
    m, k, n = shape
    g = torch.Generator().manual_seed(m + k + n)
    a = torch.randn(m, k, generator=g).to(dev)
    b = torch.randn(k, n, generator=g).to(dev)
    c = mm(a, b)
    ref = a.double() @ b.double()
    # fp32 accumulation over k terms of magnitude ~1: error grows like sqrt(k) ulps
    assert torch.allclose(c.double(), ref, rtol=1e-5, atol=2e-6 * k ** 0.5 + 1e-6)
    # signs, zeros and exact small integers survive exactly
    ai = torch.randint(-3, 4, (m, k), generator=g).float().to(dev)
    bi = torch.randint(-3, 4, (k, n), generator=g).float().to(dev)
    assert torch.equal(mm(ai, bi), (ai.double() @ bi.double()).float())


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
@pytest.mark.parametrize("shape", [(2048, 512, 1024), (4096, 300, 4096), (1500, 1111, 2000), (8192, 64, 4096)])
def test_mm_on_the_bf16_pipe(dev, precision, shape):
    """Split-bf16 matrix product against float64: the error of a product is ~2^-16 (two
    pieces) or ~2^-23 (three) of |a||b|, so the bound scales with sum_k |a_ik| |b_kj|."""
    m, k, n = shape
    g = torch.Generator().manual_seed(m + k + n)
    a = torch.randn(m, k, generator=g).to(dev)
    b = torch.randn(k, n, generator=g).to(dev)
    c = mm(a, b, _precision=precision).double()
    ref = a.double() @ b.double()
    scale = a.abs().double() @ b.abs().double()
    eps = 2.0 ** -14 if precision == "bf16x3" else 2.0 ** -21
    assert torch.all((c - ref).abs() <= eps * scale + 1e-30)
    if precision == "bf16x6":  # as good as the fp32 pipe
        e32 = (mm(a, b, _precision="fp32").double() - ref).abs().max()
        assert (c - ref).abs().max() <= 2 * e32 + 1e-6
    ai = torch.randint(-3, 4, (m, k), generator=g).float().to(dev)
    bi = torch.randint(-3, 4, (k, n), generator=g).float().to(dev)
    assert torch.equal(mm(ai, bi, _precision=precision), (ai.double() @ bi.double()).float())


@pytest.mark.parametrize("shape", [(512, 512, 512), (256, 4096, 256), (128, 8192, 128), (85, 1594, 82),
                                   (33, 3001, 131), (64, 4096, 512), (768, 3072, 256), (1, 2000, 1)])
@pytest.mark.parametrize("tile, cut", [(0, 0), (1, 2), (2, 5), (3, 7), (4, 32), (0, 3)])
def test_mm_cut_over_k(dev, shape, tile, cut):
    """Products of few tiles under a long k are cut over k and the pieces summed in split order
    by a second launch (the rule's choice with tile = cut = 0, else forced): same bounds as the
    uncut product, exact on small integers, and the same bits call after call."""
    m, k, n = shape
    g = torch.Generator().manual_seed(m + k + n)
    a = torch.randn(m, k, generator=g).to(dev)
    b = torch.randn(k, n, generator=g).to(dev)
    c = mm(a, b, _variant=tile, _splits=cut)
    ref = a.double() @ b.double()
    # k products of magnitude ~1 added in fp32: the running sum grows like sqrt(j) and each
    # addition rounds it, so the error's deviation is ~eps k / 5 (5e-5 at k = 4096), its
    # maximum over the matrix 4-5 of those
    assert torch.allclose(c.double(), ref, rtol=1e-5, atol=1.5e-7 * k + 1e-6)
    assert torch.equal(c, mm(a, b, _variant=tile, _splits=cut))
    ai = torch.randint(-3, 4, (m, k), generator=g).float().to(dev)
    bi = torch.randint(-3, 4, (k, n), generator=g).float().to(dev)
    assert torch.equal(mm(ai, bi, _variant=tile, _splits=cut), (ai.double() @ bi.double()).float())


def test_mm_rule_cuts_long_products_of_few_tiles(dev):
    """What the rule decides shows in the workspace it asks for: none for a grid that fills the
    machine, some for 256 x 4096 x 256 (4 tiles of 128 columns and 32 rows each)."""
    from triturus_amd import _lib
    lib = _lib.load()
    assert lib.trt_mm_workspace_bytes(4096, 512, 4096, 0, 0) == 0
    assert lib.trt_mm_workspace_bytes(256, 4096, 256, 0, 0) >= 2 * 256 * 256 * 4
    assert lib.trt_mm_workspace_bytes(256, 4096, 256, 0, 1) == 0


def test_mm_rejects_what_the_reference_rejects(dev):
    a = torch.rand(4, 5, device=dev)
    with pytest.raises(AssertionError):
        mm(a, torch.rand(4, 5, device=dev))
    with pytest.raises(AssertionError):
        mm(a.t(), torch.rand(4, 5, device=dev))
    with pytest.raises(AssertionError):
        mm(a.double(), torch.rand(5, 4, device=dev).double())


def test_vadd(dev):
    """The reference's test: n = 2000, rand inputs."""
    n = 2000
    x = torch.rand(n, device=dev)
    y = torch.rand(n, device=dev)
    assert torch.allclose(x + y, vadd(x, y))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 3, 255, 4097, 1 << 20, (1 << 24) + 5])
def test_vadd_bit_exact(dev, dtype, n):
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n + 1, generator=g).to(dtype).to(dev)
    y = torch.randn(n + 1, generator=g).to(dtype).to(dev)
    assert torch.equal(vadd(x[:n], y[:n]), x[:n] + y[:n])
    # unaligned views take the scalar path
    assert torch.equal(vadd(x[1:], y[1:]), x[1:] + y[1:])
    assert torch.equal(vadd(x[:n], y[:n], block_size=64), x[:n] + y[:n])
