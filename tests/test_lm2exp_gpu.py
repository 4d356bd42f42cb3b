"""lm2exp on the GPU against the float64 oracle and the fp32 torch recipe.

Accuracy gate: |x - y| <= 1e-5 + 1e-4 |y| against float64, -inf positions exact,
no NaN (oracle64.compare); at the reference's own test shape additionally the
reference's bar, torch.allclose defaults (rtol 1e-5, atol 1e-8, tests/lm2exp.py:23)
against the fp32 torch recipe."""

from pathlib import Path

import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle64, torch_baseline
from triturus.lm2exp import lm2exp
from triturus.utils import set_tf32_enabled
from triturus_amd import _lib, workloads

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden"
NINF = float("-inf")
N_VARIANTS = 20
N_BF16_VARIANTS = 9
# Accuracy gates of the split-bf16 paths against the float64 oracle: two pieces (3 MFMAs per
# product) carry 16 significand bits -- looser than fp32, ten times tighter than the rtol 5e-4
# the reference allows its TF32 mode (tests/lm2exp.py:21); three pieces (6 MFMAs) carry 24 bits
# and must pass the fp32 gate unchanged.
BF16X3_GATE = {"rtol": 1e-4, "atol": 5e-5}
PRECISION_GATES = {"bf16x3": BF16X3_GATE, "bf16x6": {}}


def _check(out, a, b, **kw):
    r = oracle64.compare(out, oracle64.lm2exp64(a, b), **kw)
    assert r["ok"], r
    return r


@pytest.mark.parametrize("allow_tf32", [False, True])
def test_lm2exp(dev, allow_tf32):
    """The reference's test (tests/lm2exp.py:10-23): same shape, inputs and tolerances."""
    set_tf32_enabled(allow_tf32)
    batch, m, k, n = 24, 150, 100, 200
    a = torch.rand(batch, m, k)
    b = torch.randn(batch, k, n)
    gt = torch_baseline.lm2exp_fp32(a, b)
    c = lm2exp(a.to(dev), b.to(dev))
    assert c.shape == (batch, m, n) and c.dtype == torch.float32 and c.device.type == "cuda"
    if allow_tf32:
        # the flag selects the split-bf16 path (error ~2^-16 per product; TF32 has 2^-11)
        assert torch.allclose(gt, c.cpu(), rtol=5e-4)
        _check(c, a, b, **BF16X3_GATE)
    else:
        assert torch.allclose(gt, c.cpu())
        # and the same recipe evaluated by torch on the GPU
        assert torch.allclose(torch_baseline.lm2exp_fp32(a.to(dev), b.to(dev)), c)
        _check(c, a, b)


@pytest.mark.parametrize("name", ["lm2exp_small", "lm2exp_ragged"])
def test_golden(dev, name):
    z = np.load(GOLDEN / f"{name}.npz")
    out = lm2exp(torch.from_numpy(z["a"]).to(dev), torch.from_numpy(z["b"]).to(dev))
    r = oracle64.compare(out, z["c"])
    assert r["ok"] and r["n_neg_inf"] > 0, r


@pytest.mark.parametrize("variant", range(1, N_VARIANTS + 1))
@pytest.mark.parametrize("shape", [(3, 37, 41, 70), (2, 300, 52, 129), (1, 64, 64, 64), (2, 33, 7, 31)])
def test_every_tile_variant_on_ragged_shapes(dev, variant, shape):
    assert _lib.load().trt_lm2exp_variant_count() == N_VARIANTS
    R, I, J, K = shape
    g = torch.Generator().manual_seed(variant * 100 + I)
    a = torch.rand(R, I, J, generator=g)
    b = -5 + 4 * torch.randn(R, J, K, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.1] = NINF
    out = lm2exp(a.to(dev), b.to(dev), _variant=variant)
    _check(out, a, b)


@pytest.mark.parametrize(
    "shape",
    [(1, 1, 1, 1), (1, 1, 5, 1), (2, 1, 1, 9), (1, 5, 1, 3), (3, 2, 3, 1), (1, 31, 33, 35), (2, 257, 4, 65),
     (1, 513, 130, 260), (5, 16, 1000, 24), (1, 8, 4097, 16)],
)
def test_edge_shapes(dev, shape):
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    b = 2 * torch.randn(R, J, K, generator=g)
    _check(lm2exp(a.to(dev), b.to(dev)), a, b)


@pytest.mark.parametrize("splits", [2, 3, 5, 32])
@pytest.mark.parametrize("variant", [0, 1, 3, 4, 16, 18])
def test_split_contraction(dev, splits, variant):
    """The contraction over J cut over several workgroups and merged (no counterpart in the
    reference): same results as the single-workgroup path, also with -inf chunks, ragged J."""
    g = torch.Generator().manual_seed(splits * 31 + variant)
    R, I, J, K = 2, 70, 333, 150
    a = torch.rand(R, I, J, generator=g)
    b = -40 + 25 * torch.randn(R, J, K, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.2] = NINF
    b[0, :, 3] = NINF            # all -inf column
    b[1, :200, 7] = NINF         # -inf in every chunk of the first splits
    b[1, 40:, 9] = NINF          # finite only in the first split
    a[1, 5, :] = 0.0
    ag, bg = a.to(dev), b.to(dev)
    out = lm2exp(ag, bg, _variant=variant, _splits=splits)
    r = _check(out, a, b)
    assert r["n_neg_inf"] >= I + K
    assert torch.equal(out, lm2exp(ag, bg, _variant=variant, _splits=splits))  # deterministic
    assert torch.allclose(out, lm2exp(ag, bg, _variant=variant, _splits=1), rtol=1e-5, atol=1e-5)


def test_small_grid_long_contraction_splits_by_itself(dev):
    lib = _lib.load()
    assert lib.trt_lm2exp_workspace_bytes(1, 512, 2048, 384, 0, 0) > 0
    g = torch.Generator().manual_seed(77)
    a = torch.rand(1, 512, 2048, generator=g)
    b = torch.randn(1, 2048, 384, generator=g)
    out = lm2exp(a.to(dev), b.to(dev))
    _check(out, a, b)
    assert torch.allclose(torch_baseline.lm2exp_fp32(a, b), out.cpu())  # the reference's bar


@pytest.mark.parametrize(
    "shape",
    [(1, 768, 1536, 768), (2, 200, 704, 900), (5, 333, 992, 257), (1, 96, 2496, 1173), (12, 420, 2688, 273), (1, 1536, 1536, 1536)],
)
def test_small_grids_whose_tile_and_cut_are_chosen_together(dev, shape):
    """Shapes whose plan comes from the joint model of tile height and cut (every tile height,
    cuts of 1..8): against float64 on the GPU -- these are too large for the CPU oracle to be
    quick -- with -inf columns, zero rows and a batch-dependent offset in b."""
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g).to(dev)
    b = (5 * torch.randn(R, J, K, generator=g) - 30 * torch.arange(R).view(R, 1, 1)).to(dev)
    a[:, 3, :] = 0.0
    b[:, :, 7] = NINF
    out = lm2exp(a, b)
    ref = oracle64.lm2exp64(a, b, device=dev)  # float64 torch on the device
    r = oracle64.compare(out, ref)
    assert r["ok"] and r["n_neg_inf"] >= R * (I + K - 1), (shape, r)
    assert torch.equal(out, lm2exp(a, b))  # deterministic, cut or not


@pytest.mark.parametrize("shape", [(64, 700, 200, 180), (96, 390, 256, 144), (40, 1100, 260, 268),
                                   (64, 700, 201, 180), (96, 390, 131, 144),  # rows of a not 16-byte aligned
                                   (3, 2878, 587, 158), (6, 1159, 1000, 159)])  # smaller grids: 64 x 64 tiles
def test_large_grids_on_64_column_pair_tiles(dev, shape):
    """Shapes that the tile rule hands to the 64-column tiles of the paired kernel (K = 144, 180,
    268 on grids of some hundred tiles): against float64 on the GPU, with -inf columns and zero rows."""
    R, I, J, K = shape
    assert "pair_kernel" in _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, int(J % 4 == 0))
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g).to(dev)
    b = (4 * torch.randn(R, J, K, generator=g) - 10).to(dev)
    a[:, 5, :] = 0.0
    b[:, :, K - 1] = NINF
    out = lm2exp(a, b)
    r = oracle64.compare(out, oracle64.lm2exp64(a, b, device=dev))
    assert r["ok"] and r["n_neg_inf"] >= R * (I + K - 1), (shape, r)


@pytest.mark.parametrize("shape, kernel", [
    ((30, 283, 700, 10), "lm2exp_kernel<1, 1, 4, 1,"),     # 128 x 32 tiles, 90 of them, cut over J
    ((3, 170, 1500, 47), "lm2exp_kernel<1, 1, 2, 2,"),     # 64 x 64 tiles, 9 of them, cut over J
    ((101, 1510, 48, 48), "lm2exp_pair_kernel<2, 2,"),     # 128 x 64 paired tiles on a large grid
    ((14, 2464, 1001, 48), "lm2exp_pair_kernel<2, 2,"),    # ... under a long contraction, rows of a unaligned
    ((436, 89, 300, 46), "lm2exp_pair_kernel<2, 2,"),
])
def test_outputs_of_at_most_64_columns(dev, shape, kernel):
    """The narrow tiles that K <= 64 takes whatever the size of the grid, and the paired 128 x 64
    tile of large grids: against float64 on the GPU, with -inf columns and zero rows."""
    R, I, J, K = shape
    assert kernel in _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, int(J % 4 == 0))
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g).to(dev)
    b = (4 * torch.randn(R, J, K, generator=g) - 10).to(dev)
    a[:, 5, :] = 0.0
    b[:, :, K - 1] = NINF
    out = lm2exp(a, b)
    r = oracle64.compare(out, oracle64.lm2exp64(a, b, device=dev))
    assert r["ok"] and r["n_neg_inf"] >= R * (I + K - 1), (shape, r)
    assert torch.equal(out, lm2exp(a, b))


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
@pytest.mark.parametrize("shape", [(3, 37, 41, 70), (2, 130, 129, 257), (1, 64, 7, 64), (2, 33, 301, 31), (24, 150, 99, 200)])
def test_padded_rows_of_a(dev, precision, shape, monkeypatch):
    """J not a multiple of 4: the wrapper pads the rows of a (thresholds lowered so that small
    inputs take that path) and the kernels read them 16 bytes at a time, masking what lies past J."""
    import triturus_amd.lm2exp as mod

    monkeypatch.setattr(mod, "_PAD_MIN_K", 1)
    monkeypatch.setattr(mod, "_PAD_MIN_FLOPS", 0.0)
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    a[:, 0] = 0.0
    b = torch.randn(R, J, K, generator=g) * 6 - 2
    b[torch.rand(b.shape, generator=g) < 0.05] = NINF
    b[:, :, 0] = NINF
    for splits in (0, 1, 3):
        # (the fp32 path pads only on request; the bf16 paths by the lowered thresholds)
        out = lm2exp(a.to(dev), b.to(dev), _precision=precision, _splits=splits, _pad=True)
        r = _check(out, a, b, **PRECISION_GATES.get(precision, {}))
        assert r["n_neg_inf"] > 0
        _check(lm2exp(a.to(dev), b.to(dev), _precision=precision, _splits=splits, _pad=False), a, b,
               **PRECISION_GATES.get(precision, {}))
    # a caller's own padded rows (a view of a wider tensor) qualify as well
    wide = torch.full((R, I, J + (-J) % 4 + 4), float("nan"))
    wide[..., :J] = a
    out = lm2exp(wide.to(dev)[..., :J], b.to(dev), _precision=precision)
    _check(out, a, b, **PRECISION_GATES.get(precision, {}))


def test_empty_inputs(dev):
    assert lm2exp(torch.rand(0, 3, 4, device=dev), torch.rand(0, 4, 5, device=dev)).shape == (0, 3, 5)
    assert lm2exp(torch.rand(2, 0, 4, device=dev), torch.rand(2, 4, 5, device=dev)).shape == (2, 0, 5)
    assert lm2exp(torch.rand(2, 3, 4, device=dev), torch.rand(2, 4, 0, device=dev)).shape == (2, 3, 0)
    out = lm2exp(torch.rand(2, 3, 0, device=dev), torch.rand(2, 0, 5, device=dev))
    assert out.shape == (2, 3, 5) and torch.all(out == NINF)


def test_neg_inf_columns_zero_rows_and_range(dev):
    g = torch.Generator().manual_seed(5)
    a = torch.rand(3, 70, 90, generator=g)
    b = -50 + 20 * torch.randn(3, 90, 150, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.3] = NINF
    b[0, :, 17] = NINF
    b[2, :, 149] = NINF
    a[1, 33, :] = 0.0
    out = lm2exp(a.to(dev), b.to(dev))
    r = _check(out, a, b)
    assert r["n_neg_inf"] >= 2 * 70 + 150
    assert torch.all(out[0, :, 17] == NINF) and torch.all(out[1, 33, :] == NINF)
    assert not torch.isnan(out).any()
    # extreme magnitudes: columns near the clamp, and a column whose max is huge
    b = torch.full((1, 4, 64), -9e37)
    b[0, :, 1] = torch.tensor([-1e30, -2e30, NINF, -1e30])
    b[0, :, 2] = torch.tensor([80.0, -80.0, 0.0, 3.0])
    a = torch.rand(1, 6, 4, generator=g)
    out = lm2exp(a.to(dev), b.to(dev))
    _check(out, a, b)
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("variant", [0, 1, 3, 5, 16, 19])
def test_shift_moves_during_the_sweep(dev, variant):
    """Columns whose maximum keeps growing along J (ascending, step changes of 1e3 and 1e30,
    finite values only in the last rows): the single-sweep kernel must rescale its sums on
    the way and still match the two-sweep recipe."""
    g = torch.Generator().manual_seed(11)
    R, I, J, K = 2, 40, 300, 96
    a = torch.rand(R, I, J, generator=g) + 0.01
    b = torch.empty(R, J, K)
    ramp = torch.linspace(-500.0, 500.0, J)
    b[0] = ramp[:, None] + torch.randn(J, K, generator=g)              # ascending: rescales every chunk
    b[1] = -ramp[:, None] + torch.randn(J, K, generator=g)             # descending: never
    b[0, :, 5] = NINF
    b[0, J - 1, 5] = 3.0                                               # first finite value in the last row
    b[0, :, 6] = torch.where(torch.arange(J) < 150, -1e30, 1e30)       # jump of 2e30 mid-way
    b[1, :, 7] = torch.where(torch.arange(J) % 64 < 32, -1e3, 1e3)     # alternating by chunk
    b[1, :, 8] = NINF
    b[1, 100, 8] = -1e38                                               # at the clamp
    ag, bg = a.to(dev), b.to(dev)
    out = lm2exp(ag, bg, _variant=variant, _splits=1)
    r = _check(out, a, b)
    assert torch.isfinite(out[0, :, 5]).all() and torch.isfinite(out[0, :, 6]).all()
    assert torch.allclose(out.cpu(), torch_baseline.lm2exp_fp32(a, b), rtol=1e-5, atol=1e-5)
    out3 = lm2exp(ag, bg, _variant=variant, _splits=3)
    _check(out3, a, b)


@pytest.mark.parametrize("precision", ["fp32"])  # (the bf16 pipes give NaN here: inf times the negative low piece of an exp)
def test_an_infinite_weight_gives_infinity_like_the_torch_recipe(dev, precision):
    """a = +inf against a finite log-value: bmm gives +inf and so does the fp32 pipe."""
    g = torch.Generator().manual_seed(12)
    a = torch.rand(2, 70, 96, generator=g) + 0.1
    b = torch.randn(2, 96, 150, generator=g)
    a[0, 3, 17] = float("inf")
    a[1, 64, 95] = float("inf")
    ref = torch_baseline.lm2exp_fp32(a, b)
    for variant in (0, 1):
        out = lm2exp(a.to(dev), b.to(dev), _precision=precision, _variant=variant).cpu()
        assert not torch.isnan(out).any()
        assert torch.equal(torch.isposinf(out), torch.isposinf(ref))
        assert torch.isposinf(out[0, 3]).all() and torch.isposinf(out[1, 64]).all()
        fin = torch.isfinite(ref)
        assert torch.allclose(out[fin], ref[fin], rtol=5e-4 if precision == "bf16x3" else 1e-5, atol=1e-5)


def test_positive_infinity_follows_the_torch_recipe(dev):
    a = torch.rand(1, 4, 40) + 0.1
    b = torch.randn(1, 40, 33)
    b[0, 7, 2] = float("inf")
    b[0, 35, 3] = float("inf")
    out = lm2exp(a.to(dev), b.to(dev)).cpu()
    ref = torch_baseline.lm2exp_fp32(a, b)
    assert torch.equal(torch.isposinf(out), torch.isposinf(ref))
    assert torch.isposinf(out[0, :, 2]).all() and torch.isposinf(out[0, :, 3]).all()
    fin = torch.isfinite(ref)
    assert torch.allclose(out[fin], ref[fin], rtol=1e-5, atol=1e-6)


def test_nan_input_propagates_like_the_torch_recipe(dev):
    a = torch.rand(1, 8, 8)
    b = torch.randn(1, 8, 40)
    b[0, 3, 5] = float("nan")
    out = lm2exp(a.to(dev), b.to(dev)).cpu()
    ref = torch_baseline.lm2exp_fp32(a, b)
    assert torch.equal(torch.isnan(out), torch.isnan(ref))
    assert torch.isnan(out[0, :, 5]).all() and not torch.isnan(out[0, :, :5]).any()


def test_strided_inputs(dev):
    g = torch.Generator().manual_seed(6)
    a_big = torch.rand(4, 80, 96, generator=g)
    b_big = torch.randn(4, 96, 200, generator=g)
    # row / batch strided views with unit inner stride go to the kernel as they are
    a = a_big[::2, 5:61, 8:72]
    b = b_big[::2, 16:80, 3:143]
    out = lm2exp(a_big.to(dev)[::2, 5:61, 8:72], b_big.to(dev)[::2, 16:80, 3:143])
    _check(out, a, b)
    # transposed operands (inner stride != 1) and broadcast views
    at = torch.rand(2, 64, 56, generator=g)
    out = lm2exp(at.to(dev).transpose(1, 2), b_big.to(dev)[:2, :64])
    _check(out, at.transpose(1, 2), b_big[:2, :64])
    a1 = torch.rand(1, 56, 64, generator=g)
    out = lm2exp(a1.to(dev).expand(2, 56, 64), b_big.to(dev)[:2, :64])
    _check(out, a1.expand(2, 56, 64), b_big[:2, :64])
    # inputs are never modified
    ag, bg = a_big.to(dev), b_big.to(dev)
    lm2exp(ag[:, :, :96], bg)
    assert torch.equal(ag.cpu(), a_big) and torch.equal(bg.cpu(), b_big)


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
@pytest.mark.parametrize("shape", [(2, 256, 64, 128), (3, 300, 50, 129), (2, 70, 333, 40), (1, 130, 18, 257), (64, 16, 33, 7)])
def test_views_of_a_are_read_in_place(dev, shape, precision):
    """The reference hands any strides to its kernel (triturus/lm2exp.py:190-198).  A transposed,
    column-strided or expanded a must give the oracle's result without a copy: the call may
    allocate its output and nothing else."""
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    b = -5 + 4 * torch.randn(R, J, K, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.1] = NINF
    ref = oracle64.lm2exp64(a, b)
    gate = BF16X3_GATE if precision == "bf16x3" else {}
    lib = _lib.load()
    pieces = {"fp32": 0, "bf16x3": 2, "bf16x6": 3}[precision]
    ws_bytes = lib.trt_lm2exp_workspace_bytes(R, I, J, K, 0, 0)
    if pieces:
        ws_bytes = max(ws_bytes, lib.trt_lm2exp_bf16_workspace_bytes(R, I, J, K, pieces, 0))
    bg = b.to(dev)
    wide = torch.zeros(R, I, 2 * J + 1)
    wide[:, :, 1::2] = a
    views = {
        "transposed": a.transpose(1, 2).contiguous().to(dev).transpose(1, 2),
        "every other column": wide.to(dev)[:, :, 1::2],
        "batch first in memory": a.permute(1, 2, 0).contiguous().to(dev).permute(2, 0, 1),
    }
    if R == 1:
        del views["batch first in memory"]  # the trailing stride is the batch size
    for name, ag in views.items():
        assert ag.stride(2) != 1 and torch.equal(ag.cpu(), a), name
        lm2exp(ag, bg, _precision=precision)  # first call: library load, workspace query cache
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = lm2exp(ag, bg, _precision=precision)
        grown = torch.cuda.memory_allocated() - before
        r = oracle64.compare(out, ref, **gate)
        assert r["ok"], (name, r)
        assert grown <= out.numel() * 4 + ws_bytes + 1024, (name, grown, out.numel() * 4, ws_bytes)
    # an expanded operand (stride 0) is read in place as well
    a1 = a[:1]
    ag = a1.to(dev).expand(R, I, J)
    lm2exp(ag, bg, _precision=precision)
    before = torch.cuda.memory_allocated()
    out = lm2exp(ag, bg, _precision=precision)
    assert torch.cuda.memory_allocated() - before <= out.numel() * 4 + ws_bytes + 1024
    assert oracle64.compare(out, oracle64.lm2exp64(a1.expand(R, I, J), b), **gate)["ok"]


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
@pytest.mark.parametrize("shape", [(2, 256, 64, 128), (3, 300, 50, 129), (2, 70, 333, 40), (1, 130, 18, 257), (5, 16, 33, 7),
                                   (2, 256, 256, 384)])  # the last one: the paired-wavefront tile
def test_views_of_b_are_read_in_place(dev, shape, precision):
    """The log-space operand with a trailing stride other than 1 -- transposed (J contiguous),
    every other column of a wider tensor, one column expanded over K -- is read where it lies, as
    the reference forwards every stride to its kernel (triturus/lm2exp.py:190-198): the call may
    allocate its output (and the workspace of a cut contraction) and nothing else."""
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    b = -5 + 4 * torch.randn(R, J, K, generator=g)
    b[torch.rand(b.shape, generator=g) < 0.1] = NINF
    b[0, :, K // 2] = NINF
    ref = oracle64.lm2exp64(a, b)
    gate = {"rtol": 1e-4, "atol": 5e-5} if precision == "bf16x3" else {}
    ag = a.to(dev)
    wide = torch.zeros(R, J, 2 * K + 1)
    wide[:, :, 1::2] = b
    views = {
        "transposed": b.transpose(1, 2).contiguous().to(dev).transpose(1, 2),
        "every other column": wide.to(dev)[:, :, 1::2],
        "batch first in memory": b.permute(1, 2, 0).contiguous().to(dev).permute(2, 0, 1),
    }
    if R == 1:
        del views["batch first in memory"]
    lib = _lib.load()
    pieces = {"fp32": 0, "bf16x3": 2, "bf16x6": 3}[precision]
    ws_bytes = lib.trt_lm2exp_workspace_bytes(R, I, J, K, 0, 0)
    if pieces:
        ws_bytes = max(ws_bytes, lib.trt_lm2exp_bf16_workspace_bytes(R, I, J, K, pieces, 0))
    for name, bg in views.items():
        assert bg.stride(2) != 1 and torch.equal(bg.cpu(), b), name
        lm2exp(ag, bg, _precision=precision)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = lm2exp(ag, bg, _precision=precision)
        grown = torch.cuda.memory_allocated() - before
        r = oracle64.compare(out, ref, **gate)
        assert r["ok"], (name, r)
        assert grown <= out.numel() * 4 + ws_bytes + 2048, (name, grown, out.numel() * 4, ws_bytes)
    # one column of b for every k (stride 0): every output column is the same
    b1 = b[:, :, 1:2]
    out = lm2exp(ag, b1.to(dev).expand(R, J, K), _precision=precision)
    assert oracle64.compare(out, oracle64.lm2exp64(a, b1.expand(R, J, K)), **gate)["ok"]


def test_c_abi_takes_a_strided_b(dev):
    """trt_lm2exp_f32 itself (no Python wrapper in between) with sb[2] != 1."""
    lib = _lib.load()
    R, I, J, K = 2, 96, 40, 200
    g = torch.Generator().manual_seed(5)
    a = torch.rand(R, I, J, generator=g)
    bt = torch.randn(R, K, J, generator=g) * 3   # b[r, j, k] = bt[r, k, j]
    ag, btg = a.to(dev), bt.to(dev)
    c = torch.empty(R, I, K, device=dev)
    s3 = ctypes.c_int64 * 3
    with _lib.on_device(dev):
        st = lib.trt_lm2exp_f32(ag.data_ptr(), btg.data_ptr(), c.data_ptr(), R, I, J, K, s3(I * J, J, 1),
                                s3(K * J, 1, J), s3(I * K, K, 1), 0, 1, None, 0, _lib.raw_stream(dev))
    assert st == 0
    assert oracle64.compare(c, oracle64.lm2exp64(a, bt.transpose(1, 2)))["ok"]


def test_algebraic_properties_on_the_gpu(dev):
    g = torch.Generator().manual_seed(7)
    R, I, J, K = 2, 128, 96, 256
    a = torch.rand(R, I, J, generator=g).to(dev)
    b = (3 * torch.randn(R, J, K, generator=g)).to(dev)
    c = lm2exp(a, b)
    # identity weights return b
    eye = torch.eye(J, device=dev).expand(R, J, J).contiguous()
    assert torch.allclose(lm2exp(eye, b), b, rtol=1e-5, atol=1e-5)
    # power-of-two column shifts and row scalings are exact in floating point
    shift = 64.0 * torch.arange(K, device=dev).remainder(5)
    assert torch.allclose(lm2exp(a, b + shift), c + shift, rtol=1e-5, atol=1e-4)
    assert torch.allclose(lm2exp(4 * a, b), c + np.log(4.0), rtol=1e-5, atol=1e-5)
    # convex weights stay between the column extremes
    an = a / a.sum(2, keepdim=True)
    cn = lm2exp(an, b)
    assert torch.all(cn <= b.amax(1, keepdim=True) + 1e-4) and torch.all(cn >= b.amin(1, keepdim=True) - 1e-4)
    # deterministic
    assert torch.equal(lm2exp(a, b), c)


@pytest.mark.parametrize("name", ["c1", "c2"])
def test_benchmark_configurations_small(dev, name):
    cfg = workloads.CONFIGS[name]()
    a, b = cfg["a"], cfg["b"]
    out = lm2exp(a.to(dev), b.to(dev))
    r = _check(out, a, b)
    if name == "c2":
        assert r["n_neg_inf"] >= 16 * 512
        for rr in range(16):
            assert torch.all(out[rr, :, cfg["neg_inf_cols"][rr]] == NINF)
        assert torch.allclose(torch_baseline.lm2exp_fp32(a, b), out.cpu(), rtol=1e-5, atol=1e-6)


def test_benchmark_configuration_c3_full_size(dev):
    """R=64, I=J=256, K=4096, b ~ N(-50, 20) with 5% -inf: every output against float64."""
    cfg = workloads.c3()
    a, b = cfg["a"], cfg["b"]
    ag, bg = a.to(dev), b.to(dev)
    out = lm2exp(ag, bg)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    worst = 0.0
    for r0 in range(0, 64, 8):  # float64 oracle, 8 batches at a time
        r = oracle64.compare(out[r0:r0 + 8], oracle64.lm2exp64(a[r0:r0 + 8], b[r0:r0 + 8]))
        assert r["ok"], (r0, r)
        worst = max(worst, r["worst_err_over_tol"])
    # size-independent properties on the whole output
    assert torch.all(out <= bg.amax(1, keepdim=True) + 1e-3)
    for variant in (1, 2, 3, 5, 16, 17, 18):  # the online kernels and the other paired-wavefront tiles
        alt = lm2exp(ag, bg, _variant=variant)
        assert torch.allclose(alt, out, rtol=1e-5, atol=1e-5)
    shifted = lm2exp(ag, bg + 128.0)
    assert torch.allclose(shifted, out + 128.0, rtol=1e-5, atol=1e-3)


# ------------------------------------------------------------ split-bf16 matrix path
@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
@pytest.mark.parametrize("variant", range(0, N_BF16_VARIANTS + 1))
@pytest.mark.parametrize(
    "shape", [(24, 150, 100, 200), (3, 37, 41, 70), (2, 300, 52, 129), (1, 64, 64, 64), (2, 33, 7, 31),
              (1, 1, 1, 1), (2, 130, 128, 257)])
def test_bf16_paths_on_ragged_shapes(dev, precision, variant, shape):
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + variant)
    a = torch.rand(R, I, J, generator=g)
    b = torch.randn(R, J, K, generator=g) * 6 - 2
    b[torch.rand(b.shape, generator=g) < 0.05] = NINF
    b[:, :, 0] = NINF  # an all -inf column: -inf out, not NaN
    a[:, 0] = 0.0  # a zero row of weights: -inf out
    out = lm2exp(a.to(dev), b.to(dev), _precision=precision, _variant=variant)
    r = _check(out, a, b, **PRECISION_GATES[precision])
    assert r["n_neg_inf"] > 0


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
@pytest.mark.parametrize("splits", [2, 5, 32])
@pytest.mark.parametrize("shape", [(3, 37, 141, 70), (1, 64, 64, 64), (2, 130, 300, 257), (2, 33, 7, 31), (1, 96, 1000, 130)])
def test_bf16_paths_cut_over_the_contraction(dev, precision, splits, shape):
    """Every bf16 tile with its contraction cut over workgroups (each with its own running
    shift, merged afterwards): same gates, -inf columns and rows included, and the same
    result on a second call (the merge adds in a fixed order)."""
    R, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + splits)
    a = torch.rand(R, I, J, generator=g)
    b = torch.randn(R, J, K, generator=g) * 6 - 2
    b[:, : J // 2] += 40.0  # the pieces end with different shifts
    b[torch.rand(b.shape, generator=g) < 0.05] = NINF
    b[:, :, 0] = NINF
    a[:, 0] = 0.0
    ag, bg = a.to(dev), b.to(dev)
    for variant in range(0, N_BF16_VARIANTS + 1):
        out = lm2exp(ag, bg, _precision=precision, _variant=variant, _splits=splits)
        r = _check(out, a, b, **PRECISION_GATES[precision])
        assert r["n_neg_inf"] > 0, variant
        again = lm2exp(ag, bg, _precision=precision, _variant=variant, _splits=splits)
        assert torch.equal(out, again), variant


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
@pytest.mark.parametrize("variant", [0, 1, 4])
def test_bf16_paths_shift_moves_during_the_sweep(dev, precision, variant):
    """The inputs of test_shift_moves_during_the_sweep: the running shift must move (and the
    sums be rescaled) on the bf16 pipe as well."""
    g = torch.Generator().manual_seed(11)
    R, I, J, K = 2, 40, 300, 96
    a = torch.rand(R, I, J, generator=g) + 0.01
    b = torch.empty(R, J, K)
    ramp = torch.linspace(-500.0, 500.0, J)
    b[0] = ramp[:, None] + torch.randn(J, K, generator=g)
    b[1] = -ramp[:, None] + torch.randn(J, K, generator=g)
    b[0, :, 5] = NINF
    b[0, J - 1, 5] = 3.0
    b[0, :, 6] = torch.where(torch.arange(J) < 150, -1e30, 1e30)
    b[1, :, 7] = torch.where(torch.arange(J) % 64 < 32, -1e3, 1e3)
    b[1, :, 8] = NINF
    b[1, 100, 8] = -1e38
    out = lm2exp(a.to(dev), b.to(dev), _precision=precision, _variant=variant)
    _check(out, a, b, **PRECISION_GATES[precision])
    assert torch.isfinite(out[0, :, 5]).all() and torch.isfinite(out[0, :, 6]).all()


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_shift_moves_by_more_than_the_exponent_range(dev, precision):
    """A term summed just under the rescale margin above the old shift must survive when a later
    chunk lifts the shift by 88.5: exp(m_old - m_new) alone is below the smallest normal float
    (e^-87.3), the rescaled sum is not (the term lies at e^-80.6, or e^-56.6 with the wide margin
    of the two-piece path, of the new shift: inside the range of the two-sweep recipe too).  Same
    for the merge of a contraction cut over J, whose pieces end with shifts 88.5 apart."""
    margin = 32.0 if precision == "bf16x3" else 8.0
    R, I, J, K = 1, 40, 130, 70
    a = torch.zeros(R, I, J)
    a[:, :, 5] = 1000.0                      # the only weight: every output is b[5] + log 1000
    b = torch.full((R, J, K), -50.0)
    b[:, 0] = 0.0                            # first chunk's maximum, zero weight
    b[:, 5] = margin - 0.1                   # summed relative to the old shift, almost e^margin
    b[:, 100] = 88.5                         # a later chunk towers over it, zero weight
    ag, bg = a.to(dev), b.to(dev)
    n_variants = N_VARIANTS if precision == "fp32" else N_BF16_VARIANTS
    for variant in range(0, n_variants + 1):
        for splits in (0, 1, 3):
            out = lm2exp(ag, bg, _precision=precision, _variant=variant, _splits=splits)
            assert torch.isfinite(out).all(), (variant, splits)
            _check(out, a, b, **PRECISION_GATES.get(precision, {}))


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
def test_bf16_paths_strided_nan_and_magnitude(dev, precision):
    g = torch.Generator().manual_seed(5)
    R, I, J, K = 2, 45, 36, 70
    abig = torch.rand(R, I + 3, J + 4, generator=g)
    bbig = torch.randn(R, J + 2, K + 9, generator=g) * 3
    a, b = abig[:, 2 : I + 2, 4:], bbig[:, 1 : J + 1, 3 : K + 3]
    out = lm2exp(a.to(dev), b.to(dev), _precision=precision)
    _check(out, a, b, **PRECISION_GATES[precision])
    b2 = (b * 1e3 - 7e8).contiguous()
    out = lm2exp(a.to(dev), b2.to(dev), _precision=precision)
    assert torch.isfinite(out).all()
    assert torch.allclose(out.cpu().double(), oracle64.lm2exp64(a, b2), rtol=1e-6, atol=1e-3)
    b3 = b.clone()
    b3[1, 7, 9] = float("nan")
    out = lm2exp(a.to(dev), b3.to(dev), _precision=precision)
    assert torch.isnan(out[1, :, 9]).all()
    mask = torch.ones_like(out, dtype=torch.bool)
    mask[1, :, 9] = False
    assert not torch.isnan(out[mask]).any()


def test_bf16x6_is_as_accurate_as_the_fp32_kernel(dev):
    """Three bf16 pieces hold all 24 significand bits: against float64 the error of the
    6-MFMA path must stay within twice that of the fp32 MFMA kernel on the same inputs."""
    cfg = workloads.c2()
    a, b = cfg["a"], cfg["b"]
    ref = oracle64.lm2exp64(a, b)
    e32 = oracle64.compare(lm2exp(a.to(dev), b.to(dev)), ref)
    e6 = oracle64.compare(lm2exp(a.to(dev), b.to(dev), _precision="bf16x6"), ref)
    e3 = oracle64.compare(lm2exp(a.to(dev), b.to(dev), _precision="bf16x3"), ref, **BF16X3_GATE)
    assert e32["ok"] and e6["ok"] and e3["ok"], (e32, e6, e3)
    assert e6["max_abs_err"] <= 2 * e32["max_abs_err"] + 1e-6, (e6, e32)


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
def test_bf16_paths_c3_full_size(dev, precision):
    """R=64, I=J=256, K=4096 on the bf16 pipe: every output against float64, plus the
    size-independent bound c <= max_j b (rows of a sum to 1) and shift equivariance."""
    cfg = workloads.c3()
    a, b = cfg["a"], cfg["b"]
    ag, bg = a.to(dev), b.to(dev)
    out = lm2exp(ag, bg, _precision=precision)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    for r0 in range(0, 64, 8):
        r = oracle64.compare(out[r0:r0 + 8], oracle64.lm2exp64(a[r0:r0 + 8], b[r0:r0 + 8]),
                             **PRECISION_GATES[precision])
        assert r["ok"], (r0, r)
    assert torch.all(out <= bg.amax(1, keepdim=True) + 1e-3)
    shifted = lm2exp(ag, bg + 128.0, _precision=precision)
    assert torch.allclose(shifted, out + 128.0, rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("shape", [(16, 512, 1024, 1), (3, 70, 2048, 4), (64, 64, 4096, 1), (1, 5, 1500, 3),
                                   (2, 1000, 1028, 2)])
def test_at_most_4_columns_under_a_long_contraction_take_the_sweep(dev, shape):
    """K <= 4 and J >= 1024 with 16-byte aligned rows of a: the vector-ALU sweep of
    csrc/lt2exp_smallk.hpp with the rows of a as the weights, against the float64 oracle (zero
    rows, -inf and NaN columns) and against the matrix-pipe tile on the same operands."""
    R, I, J, K = shape
    assert "smallk_kernel" in _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1)
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    a[:, I // 2] = 0.0
    b = 6 * torch.randn(R, J, K, generator=g) - 20
    b[0, :, 0] = NINF
    b[R - 1, J // 3, K - 1] = NINF
    out = lm2exp(a.to(dev), b.to(dev))
    r = oracle64.compare(out, oracle64.lm2exp64(a, b))
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all() and torch.isneginf(out[:, I // 2]).all()
    assert torch.equal(out, lm2exp(a.to(dev), b.to(dev)))
    assert torch.allclose(out, lm2exp(a.to(dev), b.to(dev), _variant=12), rtol=1e-5, atol=1e-5)
    for prec in ("bf16x3", "bf16x6"):  # narrow outputs go to the fp32 entry, and so to the same sweep
        assert torch.equal(out, lm2exp(a.to(dev), b.to(dev), _precision=prec))
    bn = b.clone()
    bn[R // 2, 7, K // 2] = float("nan")
    outn = lm2exp(a.to(dev), bn.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])
    # a transposed a is not swept (its rows are not dense): same result from the paired tiles
    at = a.transpose(1, 2).contiguous().transpose(1, 2).to(dev)
    assert torch.allclose(out, lm2exp(at, b.to(dev)), rtol=1e-5, atol=1e-5)


LM_COLS_SHAPES = [(2000, 4, 4, 300), (1500, 8, 8, 1024), (900, 16, 16, 256), (4000, 64, 8, 130), (3000, 1, 16, 64),   # rows of 4, 8, 16
                  (3000, 5, 7, 100), (9000, 33, 3, 65), (4000, 9, 1, 200), (8000, 2, 11, 300)]                        # any J up to 16


@pytest.mark.parametrize("shape", LM_COLS_SHAPES)
def test_contractions_of_at_most_16_terms_over_many_batches_take_a_lane_per_column(dev, shape):
    """J <= 16 over many batches: the lane-per-column kernel of csrc/lt2exp_cols.hpp with the rows of
    a as the weights, against the float64 oracle (zero rows, -inf and NaN columns) and against
    lm2exp's own tiles on the same operands; a strided a and b are read in place."""
    R, I, J, K = shape
    assert _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1).startswith("trt::lt2exp_cols_kernel<1, ")
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    a[:, I // 2] = 0.0
    b = 6 * torch.randn(R, J, K, generator=g) - 20
    b[0, :, 0] = NINF
    b[R - 1, J // 3, K - 1] = NINF
    ref = oracle64.lm2exp64(a, b)
    out = lm2exp(a.to(dev), b.to(dev))
    r = oracle64.compare(out, ref)
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all() and torch.isneginf(out[:, I // 2]).all()
    assert torch.equal(out, lm2exp(a.to(dev), b.to(dev)))
    assert torch.allclose(out, lm2exp(a.to(dev), b.to(dev), _variant=12), rtol=1e-5, atol=1e-5)
    bn = b.clone()
    bn[R // 2, J // 2, K // 2] = float("nan")
    outn = lm2exp(a.to(dev), bn.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])
    at = a.transpose(1, 2).contiguous().transpose(1, 2).to(dev)          # J-major a
    bs = torch.nn.functional.pad(b, (0, 5)).to(dev)[:, :, :K]            # rows of b wider than K
    r = oracle64.compare(lm2exp(at, bs), ref)
    assert r["ok"], (shape, "strided", r)
    for prec in ("bf16x3", "bf16x6"):
        r = oracle64.compare(lm2exp(a.to(dev), b.to(dev), _precision=prec), ref, rtol=1e-4, atol=5e-5)
        assert r["ok"], (shape, prec, r)


JSPLIT_SHAPES = [(3000, 1, 256, 16), (900, 16, 256, 16), (700, 8, 64, 32), (500, 40, 128, 48), (3000, 33, 100, 64),   # one or two column blocks
                 (60, 4, 4096, 32), (40, 30, 500, 20), (1200, 5, 36, 9), (800, 32, 44, 33), (300, 7, 1000, 40),        # long and ragged contractions, small grids
                 (2000, 5, 73, 20), (1000, 7, 1001, 11), (1500, 16, 33, 9), (900, 12, 130, 25), (200, 3, 4099, 32),    # at most 16 rows and 32 columns: any J
                 (20000, 2, 32, 16), (700, 9, 515, 17), (600, 6, 120, 12), (500, 10, 380, 30), (500, 3, 509, 14),
                 (800, 14, 64, 20), (600, 13, 128, 30), (400, 15, 192, 16), (300, 16, 384, 32), (300, 12, 512, 10)]    # 12 to 16 rows: a read 16 bytes at a time


@pytest.mark.parametrize("shape", JSPLIT_SHAPES)
def test_narrow_outputs_of_few_rows_cut_the_contraction_over_the_wavefronts(dev, shape):
    """At most 64 columns under few rows per batch: lm2exp_jsplit_kernel and, for at most 16 rows and 32
    columns, lm2exp_jsplit16_kernel (csrc/lm2exp_jsplit.hpp) against the float64 oracle (zero rows, -inf and NaN columns, a strided b) and against lm2exp's own tiles."""
    R, I, J, K = shape
    kernel = _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1)
    assert kernel.startswith("trt::lm2exp_jsplit16_kernel<" if I <= 16 and K <= 32 else "trt::lm2exp_jsplit_kernel<")
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.rand(R, I, J, generator=g)
    a[:, I // 2] = 0.0
    b = 6 * torch.randn(R, J, K, generator=g) - 20
    b[0, :, 0] = NINF
    b[R - 1, J // 3, K - 1] = NINF
    ref = oracle64.lm2exp64(a, b)
    out = lm2exp(a.to(dev), b.to(dev))
    r = oracle64.compare(out, ref)
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all() and torch.isneginf(out[:, I // 2]).all()
    assert torch.equal(out, lm2exp(a.to(dev), b.to(dev)))                      # fixed order of the partial tiles
    assert torch.allclose(out, lm2exp(a.to(dev), b.to(dev), _variant=12), rtol=1e-5, atol=1e-5)
    bn = b.clone()
    bn[R // 2, J // 2, K // 2] = float("nan")
    outn = lm2exp(a.to(dev), bn.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])
    bs = torch.nn.functional.pad(b, (0, 5)).to(dev)[:, :, :K]                  # rows of b wider than K
    bt = b.transpose(1, 2).contiguous().transpose(1, 2).to(dev)                # K-major b
    for bv in (bs, bt):
        r = oracle64.compare(lm2exp(a.to(dev), bv), ref)
        assert r["ok"], (shape, "strided b", r)
    at = a.transpose(1, 2).contiguous().transpose(1, 2).to(dev)                # J-major a, and a off the 16-byte grid
    ao = torch.nn.functional.pad(a, (1, 2)).to(dev)[:, :, 1:J + 1]
    for av in (at, ao):
        r = oracle64.compare(lm2exp(av, bs), ref)
        assert r["ok"], (shape, "strided a", r)
    ai = a.clone()                                                             # an infinite weight in the row after
    if I > 1:
        ai[:, 1, 0] = float("inf")
        outi = lm2exp(ai.to(dev), b.to(dev))
        assert torch.equal(outi[:, 0], out[:, 0])
