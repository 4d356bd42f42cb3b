"""lt2exp on the GPU against the float64 oracle and the fp32 torch recipe.

Accuracy gate as for lm2exp (oracle64.compare: rtol 1e-4, atol 1e-5, -inf exact,
no NaN); at the reference's test shape additionally torch.allclose defaults
against the fp32 torch recipe (tests/lt2exp.py:36-40), for every ``mode``."""

import itertools
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle64, torch_baseline
from triturus.lm2exp import lm2exp
from triturus.lt2exp import lt2exp
from triturus.utils import set_tf32_enabled
from triturus_amd import _lib, workloads

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden"
NINF = float("-inf")
N_VARIANTS = 16
N_BF16_VARIANTS = 16  # 1..4, 9..12 tiles; 5..8, 13..16 the same tiles with the contraction cut over workgroups
# Accuracy gates of the split-bf16 paths against the float64 oracle.  Two pieces (3 MFMAs per
# product) carry 16 significand bits: looser than fp32, ten times tighter than the rtol 5e-4
# the reference allows its TF32 mode (tests/lt2exp.py:38).  Three pieces (6 MFMAs) carry 24
# bits and must pass the fp32 gate unchanged.
BF16X3_GATE = {"rtol": 1e-4, "atol": 5e-5}
PRECISION_GATES = {"bf16x3": BF16X3_GATE, "bf16x6": {}}


def _check(out, w, a, b, **kw):
    r = oracle64.compare(out, oracle64.lt2exp64(w, a, b), **kw)
    assert r["ok"], r
    return r


@pytest.mark.parametrize("mode,allow_tf32", itertools.product(["auto", "split", "unsplit"], [False, True]))
def test_lt2exp(dev, mode, allow_tf32):
    """The reference's test (tests/lt2exp.py:14-40): same shape, inputs and tolerances."""
    set_tf32_enabled(allow_tf32)
    batch, m, j, k, n = 3, 75, 50, 50, 100
    w = torch.rand(batch, m, j, k)
    a = torch.randn(batch, j, n)
    b = torch.randn(batch, k, n)
    gt = torch_baseline.lt2exp_fp32(w, a, b)
    c = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode)
    assert c.shape == (batch, m, n) and c.dtype == torch.float32 and c.device.type == "cuda"
    if allow_tf32:
        # the flag selects the split-bf16 path (error ~2^-16 per product; TF32 has 2^-11)
        assert torch.allclose(gt, c.cpu(), rtol=5e-4)
        _check(c, w, a, b, **BF16X3_GATE)
    else:
        assert torch.allclose(gt, c.cpu())
        assert torch.allclose(torch_baseline.lt2exp_fp32(w.to(dev), a.to(dev), b.to(dev)), c)
        _check(c, w, a, b)


@pytest.mark.parametrize("name", ["lt2exp_small", "lt2exp_ragged"])
@pytest.mark.parametrize("mode", ["unsplit", "split"])
def test_golden(dev, name, mode):
    z = np.load(GOLDEN / f"{name}.npz")
    out = lt2exp(*(torch.from_numpy(z[k]).to(dev) for k in "wab"), mode=mode)
    r = oracle64.compare(out, z["c"])
    assert r["ok"] and r["n_neg_inf"] > 0, r


@pytest.mark.parametrize("variant", range(1, N_VARIANTS + 1))
@pytest.mark.parametrize("mode", ["unsplit", "split"])
@pytest.mark.parametrize("shape", [(2, 35, 9, 13, 45), (1, 70, 20, 33, 300), (2, 16, 5, 72, 64), (1, 33, 3, 3, 31),
                                   (2, 40, 6, 48, 100), (1, 33, 5, 24, 70), (1, 65, 3, 16, 64), (1, 20, 4, 100, 130),
                                   # short rows of w that pack into chunks of 16 (variants 13, 14; last chunk ragged)
                                   (2, 70, 37, 8, 150), (2, 40, 50, 2, 100), (1, 33, 9, 4, 70), (1, 65, 64, 4, 40)])
def test_every_tile_variant_on_ragged_shapes(dev, variant, mode, shape):
    assert _lib.load().trt_lt2exp_variant_count() == N_VARIANTS
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(variant * 100 + S)
    w = torch.rand(R, S, I, J, generator=g)
    a = -3 + 2 * torch.randn(R, I, K, generator=g)
    b = -3 + 2 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.1] = NINF
    b[torch.rand(b.shape, generator=g) < 0.1] = NINF
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _variant=variant)
    _check(out, w, a, b)


@pytest.mark.parametrize(
    "shape",
    [(1, 1, 1, 1, 1), (2, 1, 3, 1, 5), (1, 3, 1, 4, 1), (1, 65, 2, 2, 257), (3, 8, 64, 4, 40), (1, 8, 4, 64, 40),
     (1, 129, 17, 65, 33), (1, 4, 300, 3, 16), (1, 4, 3, 300, 16),
     # a short j axis under a long i axis runs with the roles of (i, a) and (j, b) exchanged
     (2, 40, 150, 1, 200), (2, 40, 150, 2, 300), (1, 20, 64, 8, 260), (3, 33, 37, 5, 257), (1, 20, 16, 8, 300),
     # short rows that pack (J = 2, 4, 8 with I*J a multiple of 4), and one that does not (I*J = 6)
     (2, 100, 193, 8, 145), (1, 40, 77, 4, 130), (2, 70, 22, 2, 99), (1, 8, 3, 2, 40), (1, 8, 4, 8, 40)],
)
@pytest.mark.parametrize("mode", ["auto", "split"])
def test_edge_shapes(dev, shape, mode):
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    a = 2 * torch.randn(R, I, K, generator=g)
    b = 2 * torch.randn(R, J, K, generator=g)
    _check(lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode), w, a, b)
    for precision in ("bf16x3", "bf16x6"):
        _check(lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _precision=precision), w, a, b,
               **PRECISION_GATES[precision])


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
@pytest.mark.parametrize("shape", [(2, 40, 150, 2, 300), (1, 20, 64, 8, 260), (2, 33, 21, 7, 257), (2, 35, 9, 13, 45),
                                   (1, 70, 20, 33, 300), (2, 16, 5, 50, 64), (2, 40, 30, 3, 100), (1, 70, 9, 5, 64),
                                   (2, 33, 11, 6, 130), (2, 33, 9, 21, 130)])
def test_reshaping_front_ends(dev, precision, shape, monkeypatch):
    """The wrapper's two front ends -- roles of (i, a) and (j, b) exchanged on a transposed copy
    of w for a short j axis, and w / b padded to a multiple of 4 in J (for aligned rows, or for
    short rows that then pack) -- with their work
    thresholds lowered so that small inputs take them: same results, -inf and zero weights included."""
    import triturus_amd.lt2exp as mod

    monkeypatch.setattr(mod, "_RESHAPE_MIN_FLOPS", 0.0)
    monkeypatch.setattr(mod, "_PAD_MIN_K", 1)
    monkeypatch.setattr(mod, "_PACK_PAD_MIN_FLOPS", 0.0)
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    w[:, 0] = 0.0
    a = -3 + 2 * torch.randn(R, I, K, generator=g)
    b = -3 + 2 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.1] = NINF
    b[:, :, 0] = NINF
    for mode in ("auto", "split", "unsplit"):
        # (with the thresholds lowered the rules pad J = 21 for its chunk of 24 and, on the bf16
        # paths, exchange and pad the rest; the fp32 path weighs the copies against the work they
        # save, so small inputs take them on request)
        for pad, swap in ((None, None), (True, None), (None, True), (True, True)):
            out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _precision=precision, _pad=pad, _swap=swap)
            r = _check(out, w, a, b, **PRECISION_GATES.get(precision, {}))
            assert r["n_neg_inf"] > 0


def test_empty_inputs(dev):
    def z(*shape):
        return torch.rand(*shape, device=dev)

    assert lt2exp(z(0, 3, 4, 5), z(0, 4, 6), z(0, 5, 6)).shape == (0, 3, 6)
    assert lt2exp(z(2, 0, 4, 5), z(2, 4, 6), z(2, 5, 6)).shape == (2, 0, 6)
    assert lt2exp(z(2, 3, 4, 5), z(2, 4, 0), z(2, 5, 0)).shape == (2, 3, 0)
    out = lt2exp(z(2, 3, 0, 5), z(2, 0, 6), z(2, 5, 6))
    assert out.shape == (2, 3, 6) and torch.all(out == NINF)


def test_neg_inf_and_zero_weights(dev):
    g = torch.Generator().manual_seed(8)
    R, S, I, J, K = 2, 40, 24, 40, 130
    w = torch.rand(R, S, I, J, generator=g)
    a = -30 + 10 * torch.randn(R, I, K, generator=g)
    b = -30 + 10 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.3] = NINF
    b[torch.rand(b.shape, generator=g) < 0.3] = NINF
    a[0, :, 11] = NINF
    b[1, :, 129] = NINF
    w[1, 7] = 0.0
    for mode in ("unsplit", "split"):
        out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode)
        _check(out, w, a, b)
        assert torch.all(out[0, :, 11] == NINF) and torch.all(out[1, :, 129] == NINF)
        assert torch.all(out[1, 7] == NINF) and not torch.isnan(out).any()


def test_nan_and_extreme_inputs_follow_the_torch_recipe(dev):
    g = torch.Generator().manual_seed(12)
    w = torch.rand(1, 8, 6, 10, generator=g) + 0.1
    a = torch.randn(1, 6, 70, generator=g)
    b = torch.randn(1, 10, 70, generator=g)
    a[0, 2, 4] = float("nan")
    b[0, 9, 8] = float("nan")
    a[0, :, 10] = -9e37
    b[0, :, 11] = torch.linspace(-1e30, 1e30, 10)
    a[0, :, 12] = NINF
    a[0, 5, 12] = -1e38
    for mode in ("unsplit", "split"):
        out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode).cpu()
        ref = torch_baseline.lt2exp_fp32(w, a, b)
        assert torch.equal(torch.isnan(out), torch.isnan(ref))
        assert torch.isnan(out[0, :, 4]).all() and torch.isnan(out[0, :, 8]).all()
        ok = ~torch.isnan(ref)
        r = oracle64.compare(out[ok], oracle64.lt2exp64(w, a, b)[ok])
        assert r["ok"], r


def test_non_viewable_weights_raise_like_the_reference(dev):
    w = torch.rand(2, 3, 5, 4, device=dev).transpose(2, 3)  # I and J not jointly contiguous
    with pytest.raises(RuntimeError):
        lt2exp(w, torch.rand(2, 4, 6, device=dev), torch.rand(2, 5, 6, device=dev))


def test_strided_inputs(dev):
    g = torch.Generator().manual_seed(9)
    w_big = torch.rand(4, 50, 12, 20, generator=g)
    a_big = torch.randn(4, 12, 100, generator=g)
    b_big = torch.randn(4, 40, 100, generator=g)
    sl = (slice(None, None, 2), slice(3, 45))
    w, a, b = w_big[sl], a_big[::2, :, 7:90], b_big[::2, 10:30, 7:90]
    out = lt2exp(w_big.to(dev)[sl], a_big.to(dev)[::2, :, 7:90], b_big.to(dev)[::2, 10:30, 7:90])
    _check(out, w, a, b)
    # log-space operands with a trailing stride other than 1 are read in place as well
    at = torch.randn(2, 83, 12, generator=g)
    out = lt2exp(w_big.to(dev)[sl], at.to(dev).transpose(1, 2), b_big.to(dev)[::2, 10:30, 7:90])
    _check(out, w, at.transpose(1, 2), b)


@pytest.mark.parametrize("shape", [(2, 70, 12, 20, 130), (3, 33, 7, 5, 64), (1, 200, 4, 8, 40), (2, 64, 40, 1, 256),
                                   (2, 48, 3, 200, 96)])
@pytest.mark.parametrize("mode", ["unsplit", "split"])
def test_views_of_w_are_read_in_place(dev, shape, mode):
    """The reference hands the strides of the flattened w to its kernel (triturus/lt2exp.py:577-579,
    :612-614): a w whose (i, j) axes are jointly viewable but not dense -- every other element of
    a wider tensor -- or expanded over the batch must give the oracle's result without a copy
    (the call may allocate its output and, in split mode, its workspace, and nothing else)."""
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    w[torch.rand(w.shape, generator=g) < 0.2] = 0.0
    a = 3 * torch.randn(R, I, K, generator=g)
    b = -2 + 3 * torch.randn(R, J, K, generator=g)
    ref = oracle64.lt2exp64(w, a, b)
    ag, bg = a.to(dev), b.to(dev)
    wide = torch.zeros(R, S, I, 2 * J)
    wide[..., 1::2] = w
    views = {
        "every other element": wide.to(dev)[..., 1::2],
        "every third element": torch.zeros(R, S, I, 3 * J).index_copy_(3, torch.arange(J) * 3, w).to(dev)[..., ::3],
    }
    for name, wg in views.items():
        assert wg.stride(3) != 1 and torch.equal(wg.cpu(), w), name
        wg.view(R, S, I * J)  # viewable, as the reference requires
        lt2exp(wg, ag, bg, mode=mode)  # first call: library load, workspace query cache
        torch.cuda.synchronize()
        ws = _lib.load().trt_lt2exp_workspace_bytes(R, S, I, J, K, {"unsplit": _lib.MODE_UNSPLIT, "split": _lib.MODE_SPLIT}[mode])
        before = torch.cuda.memory_allocated()
        out = lt2exp(wg, ag, bg, mode=mode)
        grown = torch.cuda.memory_allocated() - before
        r = oracle64.compare(out, ref)
        assert r["ok"], (name, r)
        assert grown <= out.numel() * 4 + ws + 2048, (name, grown, out.numel() * 4, ws)
    w1 = w[:1]
    wg = w1.to(dev).expand(R, S, I, J)
    out = lt2exp(wg, ag, bg, mode=mode)
    assert oracle64.compare(out, oracle64.lt2exp64(w1.expand(R, S, I, J), a, b))["ok"]
    # on the bf16 matrix pipe such a view is staged element by element, in place as well
    for precision in ("bf16x3", "bf16x6"):
        wg = views["every other element"]
        lt2exp(wg, ag, bg, mode=mode, _precision=precision)
        torch.cuda.synchronize()
        ws = max(_lib.load().trt_lt2exp_workspace_bytes(R, S, I, J, K, {"unsplit": _lib.MODE_UNSPLIT, "split": _lib.MODE_SPLIT}[mode]),
                 _lib.load().trt_lt2exp_bf16_workspace_bytes(R, S, I, J, K, 2 if precision == "bf16x3" else 3,
                                                             {"unsplit": _lib.MODE_UNSPLIT, "split": _lib.MODE_SPLIT}[mode]))
        before = torch.cuda.memory_allocated()
        out = lt2exp(wg, ag, bg, mode=mode, _precision=precision)
        grown = torch.cuda.memory_allocated() - before
        assert oracle64.compare(out, ref, **PRECISION_GATES[precision])["ok"]
        if J >= 4 and not (J < I and K >= 256):  # (the wrapper may pad or exchange short rows of w on copies: not this test's subject)
            assert grown <= out.numel() * 4 + ws + 2048, (precision, grown, out.numel() * 4, ws)


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
@pytest.mark.parametrize("mode", ["unsplit", "split"])
@pytest.mark.parametrize("shape", [(2, 70, 12, 20, 130), (3, 33, 7, 5, 64), (1, 200, 4, 8, 40), (2, 64, 40, 1, 256),
                                   (2, 64, 32, 32, 256), (4, 64, 64, 64, 512)])  # the last two: paired wavefront groups
def test_views_of_a_and_b_are_read_in_place(dev, shape, mode, precision):
    """The log-space operands with trailing strides other than 1 -- transposed (the contracted
    axis contiguous), every other column of a wider tensor, batch innermost -- are read where they
    lie, as the reference forwards every stride to its kernels (triturus/lt2exp.py:606-620): the
    call may allocate its output and its workspace and nothing else."""
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    a = 3 * torch.randn(R, I, K, generator=g)
    b = -2 + 3 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.05] = NINF
    b[0, :, K // 3] = NINF
    ref = oracle64.lt2exp64(w, a, b)
    gate = PRECISION_GATES.get(precision, {})
    wg = w.to(dev)
    wide_a = torch.zeros(R, I, 2 * K + 1)
    wide_a[:, :, 1::2] = a
    pairs = {
        "both transposed": (a.transpose(1, 2).contiguous().to(dev).transpose(1, 2),
                            b.transpose(1, 2).contiguous().to(dev).transpose(1, 2)),
        "a every other column, b batch first in memory": (wide_a.to(dev)[:, :, 1::2],
                                                          b.permute(1, 2, 0).contiguous().to(dev).permute(2, 0, 1)),
        "a dense, b one column for all": (a.to(dev), None),
    }
    lib = _lib.load()
    mode_code = {"unsplit": _lib.MODE_UNSPLIT, "split": _lib.MODE_SPLIT}[mode]
    pieces = {"fp32": 0, "bf16x3": 2, "bf16x6": 3}[precision]
    ws = lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, mode_code)
    if pieces:
        ws = max(ws, lib.trt_lt2exp_bf16_workspace_bytes(R, S, I, J, K, pieces, mode_code))
    for name, (ag, bg) in pairs.items():
        want = ref
        if bg is None:
            b1 = b[:, :, 1:2]
            bg = b1.to(dev).expand(R, J, K)
            want = oracle64.lt2exp64(w, a, b1.expand(R, J, K))
        elif R > 1 or "batch" not in name:
            assert ag.stride(2) != 1 or bg.stride(2) != 1, name
        lt2exp(wg, ag, bg, mode=mode, _precision=precision)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = lt2exp(wg, ag, bg, mode=mode, _precision=precision)
        grown = torch.cuda.memory_allocated() - before
        r = oracle64.compare(out, want, **gate)
        assert r["ok"], (name, r)
        if J >= 4:  # (shorter rows of w may be padded or exchanged on copies by the wrapper: not this test's subject)
            assert grown <= out.numel() * 4 + ws + 2048, (name, grown, out.numel() * 4, ws)


def test_c_abi_takes_strided_a_and_b(dev):
    """trt_lt2exp_f32 itself (no Python wrapper in between) with sa[2] != 1 and sb[2] != 1."""
    import ctypes

    lib = _lib.load()
    R, S, I, J, K = 2, 40, 6, 20, 150
    g = torch.Generator().manual_seed(6)
    w = torch.rand(R, S, I, J, generator=g)
    at = torch.randn(R, K, I, generator=g) * 3      # a[r, i, k] = at[r, k, i]
    b2 = torch.randn(R, J, 2 * K, generator=g) * 3  # b = every other column of b2
    wg, atg, b2g = w.to(dev), at.to(dev), b2.to(dev)
    c = torch.empty(R, S, K, device=dev)
    s3 = ctypes.c_int64 * 3
    with _lib.on_device(dev):
        st = lib.trt_lt2exp_f32(wg.data_ptr(), atg.data_ptr(), b2g.data_ptr(), c.data_ptr(), R, S, I, J, K,
                                s3(S * I * J, I * J, 1), s3(K * I, 1, I), s3(J * 2 * K, 2 * K, 2), s3(S * K, K, 1),
                                _lib.MODE_UNSPLIT, 0, None, 0, _lib.raw_stream(dev))
    assert st == 0
    _check(c, w, at.transpose(1, 2), b2[:, :, ::2])


@pytest.mark.parametrize("precision", ["fp32"])  # (the bf16 pipes give NaN here: inf times the negative low piece of an exp)
def test_an_infinite_weight_gives_infinity_like_the_torch_recipe(dev, precision):
    g = torch.Generator().manual_seed(13)
    w = torch.rand(2, 40, 12, 32, generator=g) + 0.1
    a = torch.randn(2, 12, 130, generator=g)
    b = torch.randn(2, 32, 130, generator=g)
    w[0, 5, 3, 7] = float("inf")
    w[1, 39, 11, 31] = float("inf")
    ref = torch_baseline.lt2exp_fp32(w, a, b)
    for mode in ("unsplit", "split"):
        out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _precision=precision, _variant=2 if precision != "fp32" else 0).cpu()
        assert not torch.isnan(out).any()
        assert torch.equal(torch.isposinf(out), torch.isposinf(ref))
        assert torch.isposinf(out[0, 5]).all() and torch.isposinf(out[1, 39]).all()
        fin = torch.isfinite(ref)
        assert torch.allclose(out[fin], ref[fin], rtol=5e-4 if precision == "bf16x3" else 1e-5, atol=1e-5)


def test_reduces_to_lm2exp_and_factorises(dev):
    g = torch.Generator().manual_seed(10)
    R, S, I, J, K = 2, 64, 16, 24, 192
    w = torch.rand(R, S, I, J, generator=g).to(dev)
    a = (2 * torch.randn(R, I, K, generator=g)).to(dev)
    b = (2 * torch.randn(R, J, K, generator=g)).to(dev)
    c = lt2exp(w, a, b)
    ab = (a[:, :, None, :] + b[:, None, :, :]).reshape(R, I * J, K)
    assert torch.allclose(c, lm2exp(w.view(R, S, I * J), ab), rtol=1e-5, atol=1e-5)
    u = torch.rand(R, S, I, generator=g).to(dev)
    v = torch.rand(R, S, J, generator=g).to(dev)
    w1 = (u[:, :, :, None] * v[:, :, None, :]).contiguous()
    assert torch.allclose(lt2exp(w1, a, b), lm2exp(u, a) + lm2exp(v, b), rtol=1e-5, atol=1e-5)
    # split and unsplit agree, and both are deterministic
    cs = lt2exp(w, a, b, mode="split")
    assert torch.allclose(cs, c, rtol=1e-6, atol=1e-6)
    assert torch.equal(lt2exp(w, a, b, mode="split"), cs) and torch.equal(lt2exp(w, a, b), c)


def test_benchmark_configuration_c4(dev):
    cfg = workloads.c4()
    w, a, b = cfg["w"], cfg["a"], cfg["b"]
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev))
    _check(out, w, a, b)
    assert torch.allclose(torch_baseline.lt2exp_fp32(w, a, b), out.cpu(), rtol=1e-5, atol=1e-5)


def _all_batches_against_float64_on_the_gpu(out, wg, ag, bg, **gate):
    """Every batch of a full-size result against the float64 recipe evaluated by torch on the GPU
    (ATen / BLAS float64 routines: nothing of this library), 8 batches at a time."""
    worst = 0.0
    for r0 in range(0, wg.shape[0], 8):
        sl = slice(r0, r0 + 8)
        ref = oracle64.lt2exp64(wg[sl], ag[sl], bg[sl], device=wg.device)
        res = oracle64.compare(out[sl], ref, **gate)
        assert res["ok"], (r0, res)
        worst = max(worst, res["worst_err_over_tol"])
    return worst


def test_benchmark_configuration_c5_full_size(dev):
    """R=64, S=I=J=64, K=4096: all 64 batches against the float64 recipe (evaluated by torch on the
    GPU; 8 of them also on the CPU), then the lm2exp identity and shift equivariance on the
    whole output."""
    cfg = workloads.c5()
    w, a, b = cfg["w"], cfg["a"], cfg["b"]
    wg, ag, bg = w.to(dev), a.to(dev), b.to(dev)
    out = lt2exp(wg, ag, bg)
    torch.cuda.synchronize()
    assert out.shape == (64, 64, 4096) and torch.isfinite(out).all()
    _all_batches_against_float64_on_the_gpu(out, wg, ag, bg)
    for r in (0, 9, 18, 27, 36, 45, 54, 63):
        res = oracle64.compare(out[r:r + 1], oracle64.lt2exp64(w[r:r + 1], a[r:r + 1], b[r:r + 1]))
        assert res["ok"], (r, res)
    # and the reference's own bar against its fp32 recipe, evaluated by torch on the GPU
    # (tests/lt2exp.py:23-40: allclose defaults would be rtol 1e-5; the values here are ~ -50)
    for r0 in range(0, 64, 4):
        sl = slice(r0, r0 + 4)
        assert torch.allclose(torch_baseline.lt2exp_fp32(wg[sl], ag[sl], bg[sl]), out[sl], rtol=1e-5, atol=1e-5)
    # the same contraction through the other kernel, 16 batches at a time (1 GiB intermediate each)
    for r0 in range(0, 64, 16):
        sl = slice(r0, r0 + 16)
        ab = (ag[sl, :, None, :] + bg[sl, None, :, :]).reshape(16, 64 * 64, 4096)
        via = lm2exp(wg[sl].view(16, 64, 64 * 64), ab)
        assert torch.allclose(out[sl], via, rtol=1e-5, atol=1e-4)
        del ab, via
    assert torch.allclose(lt2exp(wg, ag + 64.0, bg - 32.0), out + 32.0, rtol=1e-5, atol=1e-3)
    for variant in (1, 3):
        alt = lt2exp(wg, ag, bg, _variant=variant)
        _all_batches_against_float64_on_the_gpu(alt, wg, ag, bg)
        assert torch.allclose(alt, out, rtol=1e-5, atol=1e-5)
    split = lt2exp(wg, ag, bg, mode="split")
    _all_batches_against_float64_on_the_gpu(split, wg, ag, bg)
    assert torch.allclose(split, out, rtol=1e-5, atol=1e-5)


def test_capturable_in_a_hip_graph(dev):
    """No allocation, synchronisation or host state inside the C ABI: a call captured in a
    HIP graph replays with new input values (replayed several times, with eager work and
    synchronisations in between, each replay checked against the eager result)."""
    g = torch.Generator().manual_seed(13)
    w = torch.rand(2, 64, 16, 32, generator=g).to(dev)
    a = torch.randn(2, 16, 256, generator=g).to(dev)
    b = torch.randn(2, 32, 256, generator=g).to(dev)
    a2 = torch.rand(2, 256, 32, generator=g).to(dev)
    w2 = w[:, :2].contiguous()                                   # two s per batch: j contracted first
    wl = torch.rand(2, 1, 245, 256, generator=g).to(dev)         # its factors take more than 64 KB of LDS
    al = torch.randn(2, 245, 40, generator=g).to(dev)
    bl = torch.randn(2, 256, 40, generator=g).to(dev)
    assert "rows_kernel" in _lib.kernel_name("lt2exp", 2, 2, 16, 32, 256, 0, 0, 1)
    assert "rows_kernel" in _lib.kernel_name("lt2exp", 2, 1, 245, 256, 40, 0, 0, 1)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        for _ in range(2):
            lt2exp(w, a, b)
            lm2exp(a2, b)
            lt2exp(w2, a, b)
            lt2exp(wl, al, bl)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_t = lt2exp(w, a, b)
        out_t_split = lt2exp(w, a, b, mode="split")
        out_m = lm2exp(a2, b)
        out_t3 = lt2exp(w, a, b, _precision="bf16x3", _variant=1)
        out_m6 = lm2exp(a2, b, _precision="bf16x6", _variant=3)
        out_r = lt2exp(w2, a, b)
        out_l = lt2exp(wl, al, bl)
    for rep in range(4):
        a.copy_(torch.randn(2, 16, 256, generator=g))
        b.copy_(torch.randn(2, 32, 256, generator=g) - rep)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_t, lt2exp(w, a, b))
        assert torch.equal(out_t_split, lt2exp(w, a, b, mode="split"))
        assert torch.equal(out_m, lm2exp(a2, b))
        assert torch.equal(out_t3, lt2exp(w, a, b, _precision="bf16x3", _variant=1))
        assert torch.equal(out_m6, lm2exp(a2, b, _precision="bf16x6", _variant=3))
        assert torch.equal(out_r, lt2exp(w2, a, b))
        assert torch.equal(out_l, lt2exp(wl, al, bl))
        torch.cuda.synchronize()


# ------------------------------------------------------------ split-bf16 matrix path
@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
@pytest.mark.parametrize("variant", range(0, N_BF16_VARIANTS + 1))
@pytest.mark.parametrize(
    "shape", [(3, 75, 50, 50, 100), (2, 35, 9, 13, 45), (1, 70, 20, 33, 300), (2, 16, 5, 72, 64), (1, 33, 3, 3, 31),
              (2, 64, 64, 64, 256), (1, 1, 1, 1, 1), (2, 130, 4, 128, 129), (2, 40, 6, 48, 100), (1, 65, 3, 16, 64)])
def test_bf16_paths_on_ragged_shapes(dev, precision, variant, shape):
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + variant)
    w = torch.rand(R, S, I, J, generator=g)
    a = torch.randn(R, I, K, generator=g) * 4 - 3
    b = torch.randn(R, J, K, generator=g) * 4 + 2
    a[torch.rand(a.shape, generator=g) < 0.05] = NINF
    b[:, :, 0] = NINF  # an all -inf column: -inf out, not NaN
    w[:, 0] = 0.0  # a zero row of weights: -inf out
    # variants 5..8 and 13..16 cut the contraction as far as the workspace allows: mode "split" sizes it
    cut = (variant - 1) % 8 >= 4 if variant else False
    mode = "split" if cut else "auto"
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _precision=precision, _variant=variant)
    r = _check(out, w, a, b, **PRECISION_GATES[precision])
    assert r["n_neg_inf"] > 0
    if cut:  # the cut is deterministic: same bits on a second call; and close to the uncut tile
        again = lt2exp(w.to(dev), a.to(dev), b.to(dev), mode=mode, _precision=precision, _variant=variant)
        assert torch.equal(out, again)
        uncut = lt2exp(w.to(dev), a.to(dev), b.to(dev), _precision=precision, _variant=variant - 4)
        fin = torch.isfinite(uncut)
        assert torch.equal(torch.isfinite(out), fin)
        assert torch.allclose(out[fin], uncut[fin], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
def test_bf16_paths_strided_and_extreme(dev, precision):
    g = torch.Generator().manual_seed(7)
    R, S, I, J, K = 2, 40, 12, 20, 70
    wbig = torch.rand(R, S + 3, I, J, generator=g)
    abig = torch.randn(R, I + 2, K + 5, generator=g)
    bbig = torch.randn(R, J, K + 9, generator=g)
    w, a, b = wbig[:, 1 : S + 1], abig[:, 1 : I + 1, 2 : K + 2], bbig[:, :, 3 : K + 3]
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev), _precision=precision)
    _check(out, w, a, b, **PRECISION_GATES[precision])
    # large magnitudes and a huge dynamic range: the shifts keep every piece finite
    a2 = a * 1e3 + 5e4
    b2 = b * 30 - 9e6
    out = lt2exp(w.to(dev), a2.contiguous().to(dev), b2.contiguous().to(dev), _precision=precision)
    ref = oracle64.lt2exp64(w, a2, b2)
    assert torch.isfinite(out).all()
    assert torch.allclose(out.cpu().double(), ref, rtol=1e-6, atol=1e-3)
    # NaN in a log-value poisons its column, nothing else
    b3 = b.clone()
    b3[0, 3, 5] = float("nan")
    out = lt2exp(w.to(dev), a.to(dev), b3.to(dev), _precision=precision)
    assert torch.isnan(out[0, :, 5]).all()
    mask = torch.ones_like(out, dtype=torch.bool)
    mask[0, :, 5] = False
    assert not torch.isnan(out[mask]).any()


def test_bf16x6_is_as_accurate_as_the_fp32_kernel(dev):
    """Three bf16 pieces hold all 24 significand bits: against float64 the error of the
    6-MFMA path must stay within twice that of the fp32 MFMA kernel on the same inputs."""
    c = workloads.c4()
    w, a, b = c["w"], c["a"], c["b"]
    ref = oracle64.lt2exp64(w, a, b)
    e32 = oracle64.compare(lt2exp(w.to(dev), a.to(dev), b.to(dev)), ref)
    e6 = oracle64.compare(lt2exp(w.to(dev), a.to(dev), b.to(dev), _precision="bf16x6"), ref)
    e3 = oracle64.compare(lt2exp(w.to(dev), a.to(dev), b.to(dev), _precision="bf16x3"), ref, **BF16X3_GATE)
    assert e32["ok"] and e6["ok"] and e3["ok"], (e32, e6, e3)
    assert e6["max_abs_err"] <= 2 * e32["max_abs_err"] + 1e-6, (e6, e32)


@pytest.mark.parametrize("precision", ["bf16x3", "bf16x6"])
def test_bf16_paths_c5_full_size(dev, precision):
    """All 64 batches against the float64 recipe (torch on the GPU; three of them on the CPU as
    well), and properties that need no oracle: shifting a column of a or b by t shifts the
    output column by t, scaling a row of w by 2^k adds k*log(2) exactly up to rounding."""
    c = workloads.c5()
    w, a, b = (c[k].to(dev) for k in "wab")
    out = lt2exp(w, a, b, _precision=precision)
    gate = PRECISION_GATES[precision]
    _all_batches_against_float64_on_the_gpu(out, w, a, b, **gate)
    for r in (0, 37, 63):
        ref = oracle64.lt2exp64(c["w"][r : r + 1], c["a"][r : r + 1], c["b"][r : r + 1])
        res = oracle64.compare(out[r : r + 1], ref, **gate)
        assert res["ok"], (r, res)
    t = torch.linspace(-7.0, 9.0, a.shape[2], device=dev)
    out_shift = lt2exp(w, a + t, b - 2 * t, _precision=precision)
    fin = torch.isfinite(out)
    assert torch.equal(torch.isfinite(out_shift), fin)
    assert torch.allclose(out_shift[fin], (out - t)[fin], rtol=1e-4, atol=2e-4)
    out_scaled = lt2exp(w * 8.0, a, b, _precision=precision)
    assert torch.allclose(out_scaled[fin], (out + float(np.log(8.0)))[fin], rtol=1e-6, atol=1e-5)


SWEEP_SHAPES = [
    (64, 64, 64, 64, 1), (64, 64, 64, 64, 8), (16, 100, 37, 28, 3), (8, 64, 64, 32, 5),     # a wavefront per row
    (200, 3, 50, 24, 2), (130, 1, 64, 64, 7), (3, 333, 60, 20, 4), (1, 700, 300, 8, 6),
    (4, 64, 64, 64, 4), (2, 70, 90, 12, 1), (1, 128, 7, 300, 8), (16, 8, 40, 40, 2),        # a workgroup per row
    (64, 64, 1, 1024, 2), (64, 64, 1024, 1, 2), (5, 130, 1024, 4, 3), (2, 300, 2, 1024, 8),  # J = 1 exchanged; long axes
    (1, 3, 64, 64, 2), (1, 1, 300, 300, 8), (8, 64, 16, 16, 5), (37, 17, 8, 16, 1), (300, 700, 4, 32, 3),  # few rows; short rows
    (64, 64, 64, 6, 3), (8, 300, 104, 10, 8), (3, 50, 4, 73, 1), (16, 128, 20, 13, 4), (2, 7, 100, 5, 2),  # J not a multiple of 4
    (5, 40, 160, 7, 6), (1, 600, 12, 301, 7), (33, 33, 2, 250, 1),
    (228, 3, 74, 147, 3), (16, 50, 15, 73, 5), (7, 33, 9, 31, 2), (2, 5, 1, 1001, 4), (3, 9, 7, 37, 1),  # rows not 16-byte aligned
]


@pytest.mark.parametrize("shape", SWEEP_SHAPES)
def test_outputs_of_at_most_8_columns_take_the_sweep(dev, shape):
    """K <= 8 with rows of w that can be read 16 bytes at a time: the vector-ALU sweep over w
    (csrc/lt2exp_smallk.hpp) against the float64 oracle, -inf and NaN columns included, and
    against the matrix-pipe kernel on the same operands."""
    R, S, I, J, K = shape
    assert "smallk_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, int((I * J) % 4 == 0))
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    w[:, S // 2] = 0.0
    a = 5 * torch.randn(R, I, K, generator=g) - 10
    b = 5 * torch.randn(R, J, K, generator=g) + 3
    a[0, :, 0] = NINF                       # a whole column of a: -inf out
    b[R - 1, J // 2, K - 1] = NINF          # a single -inf entry: finite out
    ref = oracle64.lt2exp64(w, a, b, batch_chunk=8)
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev))
    r = oracle64.compare(out, ref)
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all() and torch.isneginf(out[:, S // 2]).all()
    assert torch.equal(out, lt2exp(w.to(dev), a.to(dev), b.to(dev)))
    mfma = lt2exp(w.to(dev), a.to(dev), b.to(dev), _variant=4)
    assert torch.allclose(out, mfma, rtol=1e-5, atol=1e-5)
    for prec in ("bf16x3", "bf16x6"):        # handed over to the same sweep
        assert torch.equal(out, lt2exp(w.to(dev), a.to(dev), b.to(dev), _precision=prec))
    an = a.clone()
    an[R // 2, I // 2, K // 2] = float("nan")
    outn = lt2exp(w.to(dev), an.to(dev), b.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])


@pytest.mark.parametrize("offset", [1, 2, 3])
@pytest.mark.parametrize("shape", [(6, 40, 16, 32, 3), (2, 9, 99, 12, 8), (1, 1, 40, 40, 1)])
def test_the_sweep_on_a_w_that_starts_off_a_16_byte_boundary(dev, shape, offset):
    """A dense w whose first element sits 4, 8 or 12 bytes past a 16-byte boundary (a view into a
    larger buffer): rows are read from the boundary below them, the floats before a row's start and
    after its end weighing nothing.  The buffer around w is NaN, so a stray weight would show."""
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + offset)
    n = R * S * I * J
    buf = torch.full((n + 8,), float("nan"))
    buf[offset:offset + n] = torch.rand(n, generator=g)
    w = buf.to(dev)[offset:offset + n].view(R, S, I, J)
    assert w.data_ptr() % 16 == 4 * offset
    a = (3 * torch.randn(R, I, K, generator=g)).to(dev)
    b = (3 * torch.randn(R, J, K, generator=g)).to(dev)
    assert "smallk_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 0)
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=4))
    assert r["ok"], (shape, offset, r)


def test_the_sweep_reads_strided_a_and_b_and_sliced_w_in_place(dev):
    R, S, I, J, K = 12, 50, 24, 96, 5
    g = torch.Generator().manual_seed(5)
    wide = torch.rand(R, S + 3, I, J, generator=g).to(dev)
    w = wide[:, 2:S + 2]                                           # rows stay 16-byte aligned
    a = (3 * torch.randn(R, K, I, generator=g)).to(dev).transpose(1, 2)   # K-major
    b = (3 * torch.randn(R, J, 2 * K, generator=g)).to(dev)[:, :, ::2]    # every other column
    assert "smallk_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1)
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=4))
    assert r["ok"], r
    assert torch.equal(out, lt2exp(w.contiguous(), a.contiguous(), b.contiguous()))


ROWS_FIRST_SHAPES = [
    (2048, 1, 64, 64, 64), (130, 1, 64, 64, 12), (9, 1, 32, 8, 9), (1, 1, 31, 44, 17),       # one s per batch
    (7, 1, 300, 300, 20), (3, 2, 245, 256, 40), (16, 4, 500, 512, 20),                          # long axes: more LDS than 64 KB
    (5, 3, 33, 20, 70), (2, 2, 40, 12, 33), (6, 12, 29, 60, 45), (3, 9, 250, 28, 33),          # I not a multiple of 32; J = 4 (mod 8)
    (11, 2, 7, 200, 10), (1, 5, 33, 68, 65),
    (4, 7, 50, 36, 100), (2, 2, 64, 64, 300), (2, 5, 96, 100, 130), (2, 3, 128, 36, 257),      # several column tiles
    (1, 16, 256, 64, 100), (3, 40, 64, 64, 12), (2, 20, 64, 128, 24),                          # s in several workgroups
    (3, 1, 33, 9, 10), (5, 2, 40, 13, 33), (2, 3, 64, 66, 70), (4, 1, 31, 47, 130), (2, 5, 100, 175, 40),  # J not a multiple of 4:
    (3, 2, 245, 255, 20), (7, 4, 50, 10, 300), (40, 1, 64, 63, 64), (1, 9, 129, 30, 90),                  # rows read float by float
]


@pytest.mark.parametrize("shape", ROWS_FIRST_SHAPES)
def test_few_s_per_batch_contract_j_first(dev, shape):
    """Few s per batch: the kernel with the rows (s, i) of w on the rows of the MFMA
    (csrc/lt2exp_rows.hpp) against the float64 oracle, -inf and NaN columns included, and against
    the s-row tiles on the same operands.  An infinite weight in the first row of every s but the
    first must not leak into the s before it (rows past I of a tile are the next s's)."""
    R, S, I, J, K = shape
    assert _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, int(J % 4 == 0)).startswith(
        "trt::lt2exp_rows_kernel<") and _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, int(J % 4 == 0)).endswith(
        "true>" if J % 4 == 0 else "false>")
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    a = 5 * torch.randn(R, I, K, generator=g) - 10
    b = 5 * torch.randn(R, J, K, generator=g) + 3
    a[0, :, 0] = NINF                       # a whole column of a: -inf out
    b[R - 1, J // 2, K - 1] = NINF          # a single -inf entry: finite out
    ref = oracle64.lt2exp64(w, a, b, batch_chunk=8)
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev))
    r = oracle64.compare(out, ref)
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all()
    assert torch.equal(out, lt2exp(w.to(dev), a.to(dev), b.to(dev)))      # the sums are added in a fixed order
    tiles = lt2exp(w.to(dev), a.to(dev), b.to(dev), _variant=4)
    assert torch.allclose(out, tiles, rtol=1e-4, atol=1e-5)
    if S > 1:
        wi = w.clone()
        wi[:, 1:, 0, :] = float("inf")
        outi = lt2exp(wi.to(dev), a.to(dev), b.to(dev))
        assert torch.equal(outi[:, 0], out[:, 0])
        ok = torch.isposinf(outi[:, 1:]) | ~torch.isfinite(out[:, 1:])
        ok[R - 1, :, K - 1] = True             # (inf times the factor 0 of the -inf entry of b: NaN, as in the recipe)
        assert ok.all()
    an = a.clone()
    an[R // 2, I // 2, K // 2] = float("nan")
    outn = lt2exp(w.to(dev), an.to(dev), b.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])


def test_j_first_reads_strided_a_and_b_and_sliced_w_in_place(dev):
    R, S, I, J, K = 12, 3, 50, 96, 45
    g = torch.Generator().manual_seed(6)
    wide = torch.rand(R, S + 3, I, J, generator=g).to(dev)
    w = wide[:, 2:S + 2]                                           # rows stay 16-byte aligned
    a = (3 * torch.randn(R, K, I, generator=g)).to(dev).transpose(1, 2)   # K-major
    b = (3 * torch.randn(R, J, 2 * K, generator=g)).to(dev)[:, :, ::2]    # every other column
    assert "rows_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1)
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=4))
    assert r["ok"], r
    assert torch.equal(out, lt2exp(w.contiguous(), a.contiguous(), b.contiguous()))


@pytest.mark.parametrize("offset", [1, 2, 3])
@pytest.mark.parametrize("shape", [(6, 2, 40, 32, 30), (2, 5, 33, 12, 100), (1, 1, 70, 50, 17)])
def test_j_first_on_a_w_that_starts_off_a_16_byte_boundary(dev, shape, offset):
    """A dense w whose first element sits 4, 8 or 12 bytes past a 16-byte boundary (a view into a
    larger buffer of NaNs): the build that reads rows float by float, whatever J is."""
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + offset)
    n = R * S * I * J
    buf = torch.full((n + 8,), float("nan"))
    buf[offset:offset + n] = torch.rand(n, generator=g)
    w = buf.to(dev)[offset:offset + n].view(R, S, I, J)
    assert w.data_ptr() % 16 == 4 * offset
    a = (3 * torch.randn(R, I, K, generator=g)).to(dev)
    b = (3 * torch.randn(R, J, K, generator=g)).to(dev)
    assert _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 0).startswith("trt::lt2exp_rows_kernel<")
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=4))
    assert r["ok"], (shape, offset, r)


def test_few_s_per_batch_under_a_long_i_keep_w_as_it_lies(dev):
    """2 <= J < I would run on a transposed copy of w under the s-row tiles; j-first takes w as it is."""
    R, S, I, J, K = 40, 2, 300, 16, 40
    assert "rows_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1)
    g = torch.Generator().manual_seed(9)
    w = torch.rand(R, S, I, J, generator=g).to(dev)
    a = (3 * torch.randn(R, I, K, generator=g)).to(dev)
    b = (3 * torch.randn(R, J, K, generator=g)).to(dev)
    out = lt2exp(w, a, b)
    assert torch.equal(out, lt2exp(w, a, b, _swap=False, _pad=False))
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=4))
    assert r["ok"], r
    for prec in ("bf16x3", "bf16x6"):        # handed over to the same kernel
        assert torch.equal(out, lt2exp(w, a, b, _precision=prec, _swap=False))
    # J not a multiple of 4: no padded copies of w and b either
    w3, b3 = w[..., :15].contiguous(), b[:, :15].contiguous()
    assert torch.equal(lt2exp(w3, a, b3), lt2exp(w3, a, b3, _swap=False, _pad=False))
    r = oracle64.compare(lt2exp(w3, a, b3), oracle64.lt2exp64(w3.cpu(), a.cpu(), b3.cpu(), batch_chunk=4))
    assert r["ok"], r


COLS_SHAPES = [
    (512, 8, 8, 8, 256), (700, 4, 4, 4, 64), (400, 1, 16, 16, 512), (900, 16, 4, 8, 33), (2000, 2, 16, 4, 100),   # exact sizes
    (1500, 3, 5, 7, 64), (3000, 5, 1, 16, 40), (2500, 7, 16, 1, 90), (5000, 1, 3, 3, 1000), (1100, 2, 13, 2, 65),    # any I and J
]


@pytest.mark.parametrize("shape", COLS_SHAPES)
def test_few_units_over_many_batches_take_a_lane_per_column(dev, shape):
    """I and J of at most 16 over many batches: the kernel with a lane per output column and the
    batch's weights as scalar operands (csrc/lt2exp_cols.hpp) against the float64 oracle, -inf and
    NaN columns included, and against the MFMA tiles on the same operands."""
    R, S, I, J, K = shape
    assert _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1).startswith("trt::lt2exp_cols_kernel<")
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.rand(R, S, I, J, generator=g)
    w[:, S // 2] = 0.0
    a = 5 * torch.randn(R, I, K, generator=g) - 10
    b = 5 * torch.randn(R, J, K, generator=g) + 3
    a[0, :, 0] = NINF                       # a whole column of a: -inf out
    b[R - 1, J // 2, K - 1] = NINF          # a single -inf entry
    ref = oracle64.lt2exp64(w, a, b, batch_chunk=64)
    out = lt2exp(w.to(dev), a.to(dev), b.to(dev))
    r = oracle64.compare(out, ref)
    assert r["ok"], (shape, r)
    assert torch.isneginf(out[0, :, 0]).all() and torch.isneginf(out[:, S // 2]).all()
    assert torch.equal(out, lt2exp(w.to(dev), a.to(dev), b.to(dev)))
    tiles = lt2exp(w.to(dev), a.to(dev), b.to(dev), _variant=4)
    assert torch.allclose(out, tiles, rtol=1e-5, atol=1e-5)
    an = a.clone()
    an[R // 2, I // 2, K // 2] = float("nan")
    outn = lt2exp(w.to(dev), an.to(dev), b.to(dev))
    assert torch.isnan(outn[R // 2, :, K // 2]).all()
    mask = torch.ones_like(outn, dtype=torch.bool)
    mask[R // 2, :, K // 2] = False
    assert torch.equal(outn[mask], out[mask])


def test_a_lane_per_column_reads_strided_a_and_b_and_sliced_w_in_place(dev):
    R, S, I, J, K = 900, 6, 8, 8, 100
    g = torch.Generator().manual_seed(8)
    wide = torch.rand(R, S + 3, I, 2 * J, generator=g).to(dev)
    w = wide[:, 2:S + 2, :, ::2]                                   # every other weight of a wider tensor
    a = (3 * torch.randn(R, K, I, generator=g)).to(dev).transpose(1, 2)   # K-major
    b = (3 * torch.randn(R, J, 2 * K, generator=g)).to(dev)[:, :, ::2]    # every other column
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=64))
    assert r["ok"], r
    dense = lt2exp(w.contiguous(), a.contiguous(), b.contiguous())
    assert _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 1) == "trt::lt2exp_cols_kernel<8, 8, true>"
    assert torch.allclose(out, dense, rtol=1e-6, atol=1e-6)        # (the general build sums in the same order)
    for prec in ("bf16x3", "bf16x6"):
        r = oracle64.compare(lt2exp(w, a, b, _precision=prec), oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=64),
                             rtol=1e-4, atol=5e-5)
        assert r["ok"], (prec, r)


@pytest.mark.parametrize("offset", [1, 2, 3, 5])
@pytest.mark.parametrize("shape", [(600, 3, 8, 8, 100), (500, 2, 16, 16, 70), (900, 5, 4, 4, 200)])
def test_a_lane_per_column_on_a_w_that_starts_off_a_16_byte_boundary(dev, shape, offset):
    """The exact-size build fetches 16 weights to a scalar load: from any 4-byte boundary (a view into
    a larger buffer of NaNs)."""
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(sum(shape) + offset)
    n = R * S * I * J
    buf = torch.full((n + 8,), float("nan"))
    buf[offset:offset + n] = torch.rand(n, generator=g)
    w = buf.to(dev)[offset:offset + n].view(R, S, I, J)
    assert w.data_ptr() % 64 == 4 * offset
    a = (3 * torch.randn(R, I, K, generator=g)).to(dev)
    b = (3 * torch.randn(R, J, K, generator=g)).to(dev)
    assert _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 0).endswith("true>")
    assert "cols_kernel" in _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, 0)
    out = lt2exp(w, a, b)
    r = oracle64.compare(out, oracle64.lt2exp64(w.cpu(), a.cpu(), b.cpu(), batch_chunk=64))
    assert r["ok"], (shape, offset, r)
