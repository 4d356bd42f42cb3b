"""Seeded random shapes, strides and -inf patterns through every arithmetic of lm2exp and
lt2exp (fp32 matrix pipe, split-bf16 with 2 and 3 pieces), each checked against the float64
oracle.  Shapes are drawn around the tile boundaries (multiples of 16/32/64/128 +- 1) where
masking mistakes live; sizes stay small enough for the oracle to finish in milliseconds."""

import random

import pytest
import torch

from oracle import oracle64
from triturus.lm2exp import lm2exp
from triturus.lt2exp import lt2exp

pytestmark = pytest.mark.gpu
NINF = float("-inf")
GATES = {"fp32": {}, "bf16x3": {"rtol": 1e-4, "atol": 5e-5}, "bf16x6": {}}


def _dim(rng, hi):
    base = rng.choice([1, 2, 3, 8, 16, 31, 32, 33, 48, 63, 64, 65, 96, 127, 128, 129, 160, 200, 257])
    return max(1, min(hi, base + rng.choice([-1, 0, 0, 1])))


def _view(rng, t):
    """Random non-contiguous view with the same values: padded rows and/or an offset."""
    kind = rng.randrange(3)
    if kind == 0:
        return t
    pad = [0, rng.randrange(1, 4)] if kind == 1 else [rng.randrange(1, 3), rng.randrange(0, 3)]
    big = torch.nn.functional.pad(t, pad + [rng.randrange(0, 2), rng.randrange(0, 2)], value=7.0)
    sl = [slice(None)] * (t.dim() - 2)
    r0 = big.shape[-2] - t.shape[-2] - 0
    lo_r = 0 if big.shape[-2] == t.shape[-2] else rng.randrange(0, big.shape[-2] - t.shape[-2] + 1)
    v = big[(*sl, slice(lo_r, lo_r + t.shape[-2]), slice(pad[0], pad[0] + t.shape[-1]))]
    assert v.shape == t.shape and r0 >= 0
    v.copy_(t)
    return v


def _sprinkle(rng, g, b):
    p = rng.choice([0.0, 0.02, 0.3])
    if p:
        b[torch.rand(b.shape, generator=g) < p] = NINF
    if rng.random() < 0.5:
        b[..., rng.randrange(b.shape[-1])] = NINF  # an all -inf column
    return b


@pytest.mark.parametrize("seed", range(24))
@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_lm2exp_random(dev, seed, precision):
    rng = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(seed)
    R, I, J, K = rng.randrange(1, 4), _dim(rng, 200), _dim(rng, 257), _dim(rng, 257)
    a = torch.rand(R, I, J, generator=g) * rng.choice([1.0, 1e-3, 50.0])
    if rng.random() < 0.3:
        a[:, rng.randrange(I)] = 0.0
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 8.0, 40.0]) + rng.choice([0.0, -60.0, 90.0]))
    ref = oracle64.lm2exp64(a, b)
    ag, bg = _view(rng, a.to(dev)), _view(rng, b.to(dev))
    nvar = 0 if precision == "fp32" else 9
    variant = rng.randrange(0, nvar + 1)
    out = lm2exp(ag, bg, _precision=precision, _variant=variant)
    r = oracle64.compare(out, ref, **GATES[precision])
    assert r["ok"], (R, I, J, K, variant, r)


@pytest.mark.parametrize("seed", range(24))
@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_lt2exp_random(dev, seed, precision):
    rng = random.Random(2000 + seed)
    g = torch.Generator().manual_seed(seed)
    R, S, I, J, K = rng.randrange(1, 3), _dim(rng, 130), _dim(rng, 33), _dim(rng, 70), _dim(rng, 257)
    w = torch.rand(R, S, I, J, generator=g) * rng.choice([1.0, 1e-4, 30.0])
    if rng.random() < 0.3:
        w[:, rng.randrange(S)] = 0.0
    a = _sprinkle(rng, g, torch.randn(R, I, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, -40.0]))
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, 70.0]))
    ref = oracle64.lt2exp64(w, a, b)
    ag, bg = _view(rng, a.to(dev)), _view(rng, b.to(dev))
    wg = w.to(dev)
    if rng.random() < 0.5:  # padded rows of S: still viewable as R x S x (I*J)
        big = torch.zeros(R, S + 2, I, J, device=dev)
        big[:, 1 : S + 1] = wg
        wg = big[:, 1 : S + 1]
    mode = rng.choice(["auto", "split", "unsplit"])
    variant = 0 if precision == "fp32" else rng.randrange(0, 17)
    out = lt2exp(wg, ag, bg, mode=mode, _precision=precision, _variant=variant)
    r = oracle64.compare(out, ref, **GATES[precision])
    assert r["ok"], (R, S, I, J, K, mode, variant, r)


@pytest.mark.parametrize("seed", range(60))
def test_lt2exp_random_with_few_columns(dev, seed):
    """K = 1..9 on random shapes, a w that starts 0..12 bytes past a 16-byte boundary inside a
    buffer of NaNs, strided a and b: the sweep over w on the vector ALU wherever the library
    takes it (and the matrix pipe elsewhere), against the float64 oracle."""
    rng = random.Random(3000 + seed)
    g = torch.Generator().manual_seed(seed)
    R, S, I, J, K = rng.randrange(1, 5), _dim(rng, 130), _dim(rng, 129), _dim(rng, 200), rng.randrange(1, 10)
    off = rng.choice([0, 0, 1, 2, 3])
    n = R * S * I * J
    buf = torch.full((n + 8,), float("nan"))
    buf[off : off + n] = torch.rand(n, generator=g) * rng.choice([1.0, 1e-4, 30.0])
    w = buf.to(dev)[off : off + n].view(R, S, I, J)
    if rng.random() < 0.3:
        w[:, rng.randrange(S)] = 0.0
    a = _sprinkle(rng, g, torch.randn(R, I, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, -40.0]))
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, 70.0]))
    ref = oracle64.lt2exp64(w.cpu(), a, b)
    out = lt2exp(w, _view(rng, a.to(dev)), _view(rng, b.to(dev)), mode=rng.choice(["auto", "split", "unsplit"]))
    r = oracle64.compare(out, ref)
    assert r["ok"], (R, S, I, J, K, off, r)


@pytest.mark.parametrize("seed", range(60))
def test_lt2exp_random_with_few_s(dev, seed):
    """S = 1..12 on random shapes, rows of w of any length, a w that starts 0..12 bytes past a
    16-byte boundary, strided a and b, every precision: the kernel that contracts j first wherever
    the library takes it (the s-row tiles elsewhere), against the float64 oracle."""
    rng = random.Random(4000 + seed)
    g = torch.Generator().manual_seed(seed)
    R, S, I, K = rng.randrange(1, 40), rng.randrange(1, 13), _dim(rng, 300), _dim(rng, 400)
    J = 4 * rng.randrange(2, 80) if rng.random() < 0.5 else rng.randrange(8, 320)
    off = rng.choice([0, 0, 0, 1, 2, 3])
    n = R * S * I * J
    buf = torch.full((n + 8,), float("nan"))
    buf[off : off + n] = torch.rand(n, generator=g) * rng.choice([1.0, 1e-4, 30.0])
    w = buf[off : off + n].view(R, S, I, J)
    if rng.random() < 0.3:
        w[:, rng.randrange(S)] = 0.0
    a = _sprinkle(rng, g, torch.randn(R, I, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, -40.0]))
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, 70.0]))
    ref = oracle64.lt2exp64(w, a, b)
    precision = rng.choice(["fp32", "fp32", "bf16x3", "bf16x6"])
    wg = buf.to(dev)[off : off + n].view(R, S, I, J)
    wg.copy_(w)
    out = lt2exp(wg, _view(rng, a.to(dev)), _view(rng, b.to(dev)), mode=rng.choice(["auto", "split", "unsplit"]),
                 _precision=precision)
    r = oracle64.compare(out, ref, **GATES[precision])
    assert r["ok"], (R, S, I, J, K, off, precision, r)


@pytest.mark.parametrize("seed", range(40))
def test_lt2exp_random_with_few_units(dev, seed):
    """I, J = 1..16 over hundreds to thousands of batches, any S, strided a and b, a w that is a
    slice of a wider tensor now and then: the kernel with a lane per output column wherever the
    library takes it, against the float64 oracle."""
    rng = random.Random(5000 + seed)
    g = torch.Generator().manual_seed(seed)
    I, J, S, K = rng.randrange(1, 17), rng.randrange(1, 17), rng.choice([1, 2, 3, 5, 8, 16, 33]), _dim(rng, 300)
    R = rng.choice([50, 400, 1500, 4000])
    w = torch.rand(R, S, I, J, generator=g) * rng.choice([1.0, 1e-4, 30.0])
    a = _sprinkle(rng, g, torch.randn(R, I, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, -40.0]))
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, 70.0]))
    ref = oracle64.lt2exp64(w, a, b, batch_chunk=256)
    wg = w.to(dev)
    if rng.random() < 0.3:
        wide = torch.zeros(R, S, I, 2 * J, device=dev)
        wide[..., ::2] = wg
        wg = wide[..., ::2]
    precision = rng.choice(["fp32", "fp32", "bf16x3", "bf16x6"])
    out = lt2exp(wg, _view(rng, a.to(dev)), _view(rng, b.to(dev)), mode=rng.choice(["auto", "split", "unsplit"]),
                 _precision=precision)
    r = oracle64.compare(out, ref, **GATES[precision])
    assert r["ok"], (R, S, I, J, K, precision, r)


@pytest.mark.parametrize("seed", range(40))
def test_lm2exp_random_with_narrow_outputs(dev, seed):
    """At most 40 rows and 9..64 columns per batch over hundreds to thousands of batches, any J from
    32 on, strided a and b: the kernels that cut a batch's one tile over the wavefronts wherever the
    library takes them, against the float64 oracle."""
    rng = random.Random(7000 + seed)
    g = torch.Generator().manual_seed(seed)
    I, J, K = rng.randrange(1, 41), rng.choice([32, 33, 47, 64, 100, 129, 256, 380, 500, 515, 1000, 2050]), rng.randrange(9, 65)
    R = rng.choice([30, 300, 1200, 3000])
    a = torch.rand(R, I, J, generator=g) * rng.choice([1.0, 1e-4, 30.0])
    a[torch.rand(R, I, J, generator=g) < 0.1] = 0.0
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([1.0, 10.0]) + rng.choice([0.0, 70.0, -90.0]))
    ref = oracle64.lm2exp64(a, b)
    precision = rng.choice(["fp32", "fp32", "fp32", "bf16x3"])
    out = lm2exp(_view(rng, a.to(dev)), _view(rng, b.to(dev)), _precision=precision)
    r = oracle64.compare(out, ref, **GATES[precision])
    assert r["ok"], (R, I, J, K, precision, r)


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_results_are_bit_reproducible(dev, precision):
    """Fixed summation order everywhere (no atomics, merges in split order): the same call on
    the same inputs gives the same bits, run after run, whatever else the GPU is doing --
    including the paths that cut the contraction over several workgroups."""
    g = torch.Generator().manual_seed(99)
    w = torch.rand(3, 75, 50, 50, generator=g).to(dev)
    a = torch.randn(3, 50, 100, generator=g).to(dev)
    b = torch.randn(3, 50, 100, generator=g).to(dev)
    a2 = torch.rand(2, 96, 700, generator=g).to(dev)
    b2 = (torch.randn(2, 700, 130, generator=g) * 20).to(dev)
    big_w = torch.rand(8, 64, 32, 32, generator=g).to(dev)
    big_a = torch.randn(8, 32, 2048, generator=g).to(dev)
    big_b = torch.randn(8, 32, 2048, generator=g).to(dev)
    calls = [
        lambda: lt2exp(w, a, b, mode="split", _precision=precision),
        lambda: lt2exp(w, a, b, mode="unsplit", _precision=precision),
        lambda: lt2exp(big_w, big_a, big_b, _precision=precision),
        lambda: lm2exp(a2, b2, _precision=precision),
        lambda: lm2exp(a2, b2, _precision=precision, _splits=5),
    ]
    first = [f().clone() for f in calls]
    noise = torch.randn(4096, 4096, device=dev)
    for rep in range(3):
        (noise @ noise).sum()  # unrelated work in between
        for f, ref in zip(calls, first):
            assert torch.equal(f(), ref)


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_very_long_column_axis(dev, precision):
    """K = 2^20 + 3 columns (8193 column tiles, offsets beyond 2^22 elements per row): every
    column against the float64 oracle."""

    g = torch.Generator().manual_seed(5)
    K = (1 << 20) + 3
    a = torch.rand(1, 40, 24, generator=g).to(dev)
    b = (torch.randn(1, 24, K, generator=g) * 6).to(dev)
    b[0, :, K - 1] = NINF
    out = lm2exp(a, b, _precision=precision)
    ref = oracle64.lm2exp64(a.cpu(), b.cpu())
    assert oracle64.compare(out, ref, **GATES[precision])["ok"]
    w = torch.rand(1, 20, 6, 10, generator=g).to(dev)
    a2 = (torch.randn(1, 6, K, generator=g) * 3).to(dev)
    b2 = (torch.randn(1, 10, K, generator=g) * 3).to(dev)
    out = lt2exp(w, a2, b2, _precision=precision)
    ref = oracle64.lt2exp64(w.cpu(), a2.cpu(), b2.cpu())
    assert oracle64.compare(out, ref, **GATES[precision])["ok"]


def test_measured_tile_selection(dev):
    """Opt-in tuning (the reference autotunes per shape key): the first call times the
    candidate tiles, later calls reuse the choice; results stay within the gate."""
    from triturus_amd import autotune

    g = torch.Generator().manual_seed(3)
    a = torch.rand(8, 200, 96, generator=g)
    b = torch.randn(8, 96, 300, generator=g) * 4
    w = torch.rand(4, 70, 24, 40, generator=g)
    a2 = torch.randn(4, 24, 500, generator=g)
    b2 = torch.randn(4, 40, 500, generator=g)
    ref_m = oracle64.lm2exp64(a, b)
    ref_t = oracle64.lt2exp64(w, a2, b2)
    autotune.clear()
    autotune.set_autotune(True)
    try:
        for precision in ("fp32", "bf16x3"):
            for _ in range(2):
                out = lm2exp(a.to(dev), b.to(dev), _precision=precision)
                assert oracle64.compare(out, ref_m, **GATES[precision])["ok"]
                out = lt2exp(w.to(dev), a2.to(dev), b2.to(dev), _precision=precision)
                assert oracle64.compare(out, ref_t, **GATES[precision])["ok"]
        picked = autotune.chosen()
        assert ("lm2exp", 8, 200, 96, 300, "fp32") in picked
        assert ("lt2exp", 4, 70, 24, 40, 500, "auto", "bf16x3") in picked
        assert all(isinstance(v, int) and v >= 0 for v in picked.values())
    finally:
        autotune.set_autotune(False)
        autotune.clear()
    assert autotune.pick(("x",), (0, 1), lambda v: None) == 0  # off: the library's rule


# ---- sparse weights under a wide spread of log-values: the dominant log-value often meets a
# zero weight, so an output rests on terms far below its column's maximum.  fp32 arithmetic can
# hold a term only while it stays above 2^-126 of the shift; the check therefore brackets every
# output between the exact float64 value and the value with all terms more than `cut` below the
# column maximum dropped (a result may lose those terms, nothing else).
def _lm_bracket(a, b, cut):
    a, b = a.double(), b.double()
    m = torch.clamp(torch.amax(b, dim=1, keepdim=True), -1e38, 1e38)
    t = b - m
    e = torch.exp(t)
    pos = a[a > 0]
    slack = min(0.0, float(torch.log(pos.min()))) if pos.numel() else 0.0
    hi = m + torch.log(torch.bmm(a, e))
    lo = m + torch.log(torch.bmm(a, torch.where(t < -(cut + slack), torch.zeros_like(e), e)))
    return lo, hi


def _lt_bracket(w, a, b, cut):
    w, a, b = w.double(), a.double(), b.double()
    R, S, I, J = w.shape
    K = a.shape[2]
    ma = torch.clamp(torch.amax(a, dim=1, keepdim=True), -1e38, 1e38)
    mb = torch.clamp(torch.amax(b, dim=1, keepdim=True), -1e38, 1e38)
    ta, tb = a - ma, b - mb
    t = ta.unsqueeze(2) + tb.unsqueeze(1)
    e = torch.exp(t)
    pos = w[w > 0]
    slack = min(0.0, float(torch.log(pos.min()))) if pos.numel() else 0.0
    drop = (t < -(cut + slack)) | (ta.unsqueeze(2) < -cut) | (tb.unsqueeze(1) < -cut)
    wf = w.reshape(R, S, I * J)
    shift = ma + mb
    hi = shift + torch.log(torch.bmm(wf, e.reshape(R, I * J, K)))
    lo = shift + torch.log(torch.bmm(wf, torch.where(drop, torch.zeros_like(e), e).reshape(R, I * J, K)))
    return lo, hi


def _inside(x, lo, hi, rtol=1e-4, atol=1e-5):
    x = x.detach().cpu().double()
    tol_hi = atol + rtol * torch.nan_to_num(hi.abs(), posinf=0.0)
    tol_lo = atol + rtol * torch.nan_to_num(lo.abs(), posinf=0.0)
    fragile = ~((hi - lo).abs() <= tol_hi)  # rests on terms that fp32 may flush or hold as denormals
    up = x <= hi + tol_hi + torch.where(fragile, 0.75, 0.0)
    down = (x >= lo - tol_lo) | (lo == NINF)
    bad = ~(up & down) | torch.isnan(x)
    return int(bad.sum()), int(fragile.sum())


@pytest.mark.parametrize("seed", range(16))
@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_sparse_weights_under_a_wide_spread(dev, seed, precision):
    rng = random.Random(3000 + seed)
    g = torch.Generator().manual_seed(3000 + seed)
    cut = 75.0 if precision == "fp32" else 60.0
    R, I, J, K = rng.randrange(1, 4), _dim(rng, 200), _dim(rng, 257), _dim(rng, 257)
    a = torch.rand(R, I, J, generator=g) * rng.choice([1.0, 1e-3, 50.0, 1e20])
    a[torch.rand(a.shape, generator=g) < 0.8] = 0.0
    b = torch.randn(R, J, K, generator=g) * rng.choice([40.0, 300.0]) + rng.choice([0.0, 1e4, -1e6])
    b = _sprinkle(rng, g, b)
    lo, hi = _lm_bracket(a, b, cut)
    nvar = 20 if precision == "fp32" else 9
    variant, splits = rng.randrange(0, nvar + 1), rng.choice([0, 1, 3])
    out = lm2exp(_view(rng, a.to(dev)), _view(rng, b.to(dev)), _precision=precision, _variant=variant, _splits=splits)
    bad, _ = _inside(out, lo, hi, **GATES[precision])
    assert bad == 0, ("lm2exp", R, I, J, K, variant, splits, bad)

    R, S, I, J, K = rng.randrange(1, 3), _dim(rng, 130), _dim(rng, 33), _dim(rng, 70), _dim(rng, 257)
    w = torch.rand(R, S, I, J, generator=g) * rng.choice([1.0, 1e-4, 1e20])
    w[torch.rand(w.shape, generator=g) < 0.8] = 0.0
    a = _sprinkle(rng, g, torch.randn(R, I, K, generator=g) * rng.choice([10.0, 100.0]) + rng.choice([0.0, 1e5]))
    b = _sprinkle(rng, g, torch.randn(R, J, K, generator=g) * rng.choice([10.0, 100.0]) + rng.choice([0.0, -1e5]))
    lo, hi = _lt_bracket(w, a, b, cut)
    mode = rng.choice(["auto", "split", "unsplit"])
    variant = rng.randrange(0, 5)
    if precision == "fp32" and rng.random() < 0.4:  # the tiles with j-chunks of 16, 24 and 48, the narrow tiles
        variant = rng.randrange(5, 13)
    out = lt2exp(w.to(dev), _view(rng, a.to(dev)), _view(rng, b.to(dev)), mode=mode, _precision=precision,
                 _variant=variant)
    bad, _ = _inside(out, lo, hi, **GATES[precision])
    assert bad == 0, ("lt2exp", R, S, I, J, K, mode, variant, bad)


def test_concurrent_streams(dev):
    """The library keeps no state between calls: launches interleaved on two streams (default
    priority), each with its own split-mode workspace, give the results of the same calls made
    one after the other."""
    g = torch.Generator().manual_seed(17)
    a = torch.rand(2, 96, 700, generator=g).to(dev)
    b = (torch.randn(2, 700, 130, generator=g) * 20).to(dev)
    w = torch.rand(3, 75, 50, 50, generator=g).to(dev)
    x = torch.randn(3, 50, 100, generator=g).to(dev)
    y = torch.randn(3, 50, 100, generator=g).to(dev)
    ref_m = lm2exp(a, b, _splits=5)
    ref_t = lt2exp(w, x, y, mode="split")
    ref_m6 = lm2exp(a, b, _precision="bf16x6")
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)
    outs = []
    for _ in range(20):
        with torch.cuda.stream(s1):
            o1 = lm2exp(a, b, _splits=5)
            o3 = lm2exp(a, b, _precision="bf16x6")
        with torch.cuda.stream(s2):
            o2 = lt2exp(w, x, y, mode="split")
        outs.append((o1, o2, o3))
    torch.cuda.synchronize()
    for o1, o2, o3 in outs:
        assert torch.equal(o1, ref_m) and torch.equal(o2, ref_t) and torch.equal(o3, ref_m6)


@pytest.mark.parametrize("precision", ["fp32", "bf16x3", "bf16x6"])
def test_against_the_c_restatement(dev, precision):
    """The HIP path against the plain C loops (oracle/oracle_c.c), the checker that shares no
    code with torch: benchmark input distributions at small sizes, -inf included."""
    from oracle import oracle_c
    from triturus_amd import workloads

    c2 = workloads.c2(R=2, n=96)
    out = lm2exp(c2["a"].to(dev), c2["b"].to(dev), _precision=precision)
    assert oracle64.compare(out, oracle_c.lm2exp_c(c2["a"], c2["b"]), **GATES[precision])["ok"]
    c4 = workloads.c4(R=2, K=200)
    for mode in ("unsplit", "split"):
        out = lt2exp(c4["w"].to(dev), c4["a"].to(dev), c4["b"].to(dev), mode=mode, _precision=precision)
        assert oracle64.compare(out, oracle_c.lt2exp_c(c4["w"], c4["a"], c4["b"]), **GATES[precision])["ok"]
