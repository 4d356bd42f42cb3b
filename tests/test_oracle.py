"""Pins the CPU oracle (oracle/) without the GPU.

The float64 recipe oracles are checked against formulations that share no code
with them: scipy's logsumexp over the explicitly broadcast tensor, pure-Python
fsum loops on tiny inputs, and algebraic special cases chosen so that a dropped
term, a wrong axis or a transposed operand fails at least one of them.
"""

import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import max_ref, oracle64, torch_baseline
from triturus_amd import workloads

GOLDEN = Path(__file__).resolve().parent / "golden"
NINF = float("-inf")


def _rand_lm(seed, R, I, J, K, p_inf=0.0):
    g = torch.Generator().manual_seed(seed)
    a = torch.rand(R, I, J, generator=g, dtype=torch.float64)
    b = 3.0 * torch.randn(R, J, K, generator=g, dtype=torch.float64)
    if p_inf:
        b[torch.rand(b.shape, generator=g) < p_inf] = NINF
    return a, b


def _rand_lt(seed, R, S, I, J, K, p_inf=0.0):
    g = torch.Generator().manual_seed(seed)
    w = torch.rand(R, S, I, J, generator=g, dtype=torch.float64)
    a = 3.0 * torch.randn(R, I, K, generator=g, dtype=torch.float64)
    b = 3.0 * torch.randn(R, J, K, generator=g, dtype=torch.float64)
    if p_inf:
        a[torch.rand(a.shape, generator=g) < p_inf] = NINF
        b[torch.rand(b.shape, generator=g) < p_inf] = NINF
    return w, a, b


def _close(x, y, tol=1e-11):
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    assert x.shape == y.shape
    assert np.array_equal(np.isneginf(x), np.isneginf(y))
    assert not np.isnan(x).any() and not np.isnan(y).any()
    fin = np.isfinite(y)
    np.testing.assert_allclose(x[fin], y[fin], rtol=tol, atol=tol)


# ------------------------------------------------------------------ lm2exp
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 3, 4, 5), (3, 17, 9, 33), (2, 8, 64, 8)])
@pytest.mark.parametrize("p_inf", [0.0, 0.3])
def test_lm2exp_recipe_matches_closed_form(shape, p_inf):
    a, b = _rand_lm(1, *shape, p_inf=p_inf)
    _close(oracle64.lm2exp64(a, b), oracle64.lm2exp_lse(a, b))


def test_lm2exp_brute_force_loops():
    R, I, J, K = 2, 3, 4, 5
    a, b = _rand_lm(2, R, I, J, K)
    b[1, 2, 3] = NINF
    got = oracle64.lm2exp64(a, b)
    for r in range(R):
        for i in range(I):
            for k in range(K):
                s = math.fsum(float(a[r, i, j]) * math.exp(float(b[r, j, k])) for j in range(J))
                assert math.isclose(float(got[r, i, k]), math.log(s), rel_tol=1e-12, abs_tol=1e-12)


def test_lm2exp_operand_roles_not_transposed():
    # a selects rows of b: with a one-hot a[r,i,:] = e_{p(i)}, c[r,i,:] = b[r,p(i),:]
    R, I, J, K = 2, 5, 5, 7
    _, b = _rand_lm(3, R, I, J, K)
    perm = torch.tensor([3, 0, 4, 1, 2])
    a = torch.zeros(R, I, J, dtype=torch.float64)
    a[:, torch.arange(I), perm] = 1.0
    _close(oracle64.lm2exp64(a, b), b[:, perm, :])


def test_lm2exp_special_cases():
    R, I, J, K = 2, 6, 5, 4
    a, b = _rand_lm(4, R, I, J, K)
    c = oracle64.lm2exp64(a, b)
    # J = 1: c = log a + b
    _close(oracle64.lm2exp64(a[:, :, :1], b[:, :1, :]), torch.log(a[:, :, :1]) + b[:, :1, :])
    # constant b and rows of a summing to one: c is that constant
    an = a / a.sum(2, keepdim=True)
    _close(oracle64.lm2exp64(an, torch.full_like(b, -7.25)), torch.full((R, I, K), -7.25))
    # column shift equivariance and row scaling
    t = torch.linspace(-50, 50, K, dtype=torch.float64)
    _close(oracle64.lm2exp64(a, b + t), c + t, tol=1e-10)
    _close(oracle64.lm2exp64(2.5 * a, b), c + math.log(2.5))
    # convex weights: min_j b <= c <= max_j b
    cn = oracle64.lm2exp64(an, b)
    assert torch.all(cn <= b.amax(1, keepdim=True) + 1e-12)
    assert torch.all(cn >= b.amin(1, keepdim=True) - 1e-12)


def test_lm2exp_neg_inf_columns_and_zero_rows_give_neg_inf_not_nan():
    a, b = _rand_lm(5, 2, 4, 6, 5)
    b[0, :, 2] = NINF
    a[1, 3, :] = 0.0
    c = oracle64.lm2exp64(a, b)
    assert not torch.isnan(c).any()
    assert torch.all(c[0, :, 2] == NINF)
    assert torch.all(c[1, 3, :] == NINF)
    assert torch.isfinite(c[0, :, :2]).all()
    # huge dynamic range: the shift keeps everything finite
    b2 = torch.tensor([[[-1e30], [-2e30]]], dtype=torch.float64)
    a2 = torch.ones(1, 1, 2, dtype=torch.float64)
    assert float(oracle64.lm2exp64(a2, b2)) == -1e30


# ------------------------------------------------------------------ lt2exp
@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (2, 3, 4, 5, 6), (2, 9, 7, 3, 17)])
@pytest.mark.parametrize("p_inf", [0.0, 0.3])
def test_lt2exp_recipe_matches_closed_form(shape, p_inf):
    w, a, b = _rand_lt(6, *shape, p_inf=p_inf)
    _close(oracle64.lt2exp64(w, a, b), oracle64.lt2exp_lse(w, a, b))
    _close(oracle64.lt2exp64(w, a, b, batch_chunk=2), oracle64.lt2exp_lse(w, a, b))


def test_lt2exp_brute_force_loops():
    R, S, I, J, K = 2, 2, 3, 4, 3
    w, a, b = _rand_lt(7, R, S, I, J, K)
    got = oracle64.lt2exp64(w, a, b)
    for r in range(R):
        for s in range(S):
            for k in range(K):
                tot = math.fsum(
                    float(w[r, s, i, j]) * math.exp(float(a[r, i, k])) * math.exp(float(b[r, j, k]))
                    for i in range(I)
                    for j in range(J)
                )
                assert math.isclose(float(got[r, s, k]), math.log(tot), rel_tol=1e-12, abs_tol=1e-12)


def test_lt2exp_reduces_to_lm2exp_on_the_outer_sum():
    R, S, I, J, K = 2, 5, 3, 4, 6
    w, a, b = _rand_lt(8, R, S, I, J, K, p_inf=0.2)
    ab = (a[:, :, None, :] + b[:, None, :, :]).reshape(R, I * J, K)
    _close(oracle64.lt2exp64(w, a, b), oracle64.lm2exp64(w.reshape(R, S, I * J), ab))


def test_lt2exp_matches_the_einsum_formulation():
    """The reference states the recipe a second way, as a three-operand einsum over the shifted
    exponentials (baselines/lt2exp.py:28-45); in float64 the two agree to rounding."""
    R, S, I, J, K = 3, 5, 4, 6, 7
    w, a, b = _rand_lt(12, R, S, I, J, K, p_inf=0.2)
    w64, a64, b64 = w.double(), a.double(), b.double()
    ma = torch.clamp(torch.amax(a64, dim=1, keepdim=True), -1e38, 1e38)
    mb = torch.clamp(torch.amax(b64, dim=1, keepdim=True), -1e38, 1e38)
    r = torch.einsum("brij,bis,bjs->brs", w64, torch.exp(a64 - ma), torch.exp(b64 - mb))
    _close(oracle64.lt2exp64(w, a, b), ma + mb + torch.log(r))


def test_lt2exp_rank_one_weights_factorise():
    R, S, I, J, K = 2, 4, 3, 5, 6
    _, a, b = _rand_lt(9, R, S, I, J, K)
    g = torch.Generator().manual_seed(10)
    u = torch.rand(R, S, I, generator=g, dtype=torch.float64)
    v = torch.rand(R, S, J, generator=g, dtype=torch.float64)
    w = u[:, :, :, None] * v[:, :, None, :]
    _close(oracle64.lt2exp64(w, a, b), oracle64.lm2exp64(u, a) + oracle64.lm2exp64(v, b), tol=1e-10)


def test_lt2exp_index_roles_not_swapped():
    # one-hot w[r,s,i,j] picks a[r,i(s),k] + b[r,j(s),k]; I != J catches a swap
    R, S, I, J, K = 1, 4, 3, 5, 6
    _, a, b = _rand_lt(11, R, S, I, J, K)
    ii = torch.tensor([2, 0, 1, 2])
    jj = torch.tensor([4, 3, 0, 1])
    w = torch.zeros(R, S, I, J, dtype=torch.float64)
    w[0, torch.arange(S), ii, jj] = 1.0
    _close(oracle64.lt2exp64(w, a, b), a[:, ii, :] + b[:, jj, :])


def test_lt2exp_neg_inf():
    w, a, b = _rand_lt(12, 2, 3, 4, 5, 6)
    a[0, :, 1] = NINF
    b[1, :, 2] = NINF
    w[1, 2] = 0.0
    c = oracle64.lt2exp64(w, a, b)
    assert not torch.isnan(c).any()
    assert torch.all(c[0, :, 1] == NINF) and torch.all(c[1, :, 2] == NINF) and torch.all(c[1, 2] == NINF)


# ------------------------------------------------ fp32 recipes vs the oracle
def test_fp32_recipes_within_the_accuracy_gate():
    c = workloads.c1()
    r = oracle64.compare(torch_baseline.lm2exp_fp32(c["a"], c["b"]), oracle64.lm2exp64(c["a"], c["b"]))
    assert r["ok"], r
    c = workloads.c2(R=2, n=128)
    out = torch_baseline.lm2exp_fp32(c["a"], c["b"])
    r = oracle64.compare(out, oracle64.lm2exp64(c["a"], c["b"]))
    assert r["ok"] and r["n_neg_inf"] >= 2 * 128, r
    for rr in range(2):
        assert torch.all(out[rr, :, c["neg_inf_cols"][rr]] == NINF)
    c = workloads.c4(R=2, K=128)
    full = torch_baseline.lt2exp_fp32(c["w"], c["a"], c["b"])
    r = oracle64.compare(full, oracle64.lt2exp64(c["w"], c["a"], c["b"]))
    assert r["ok"], r
    assert torch.allclose(full, torch_baseline.lt2exp_fp32_chunked(c["w"], c["a"], c["b"], 1), rtol=1e-5, atol=1e-6)


def test_compare_gate_catches_errors():
    y = torch.tensor([1.0, NINF, 3.0], dtype=torch.float64)
    assert oracle64.compare(y.float(), y)["ok"]
    assert not oracle64.compare(torch.tensor([1.0, -1e30, 3.0]), y)["ok"]
    assert not oracle64.compare(torch.tensor([1.0, NINF, float("nan")]), y)["ok"]
    assert not oracle64.compare(torch.tensor([1.001, NINF, 3.0]), y)["ok"]
    assert not oracle64.compare(torch.tensor([NINF, NINF, 3.0]), y)["ok"]


def test_workload_shapes_and_normalisation():
    c = workloads.c1()
    assert c["a"].shape == (4, 64, 64) and torch.allclose(c["a"].sum(2), torch.ones(4, 64))
    c = workloads.c4(R=2, K=64)
    assert torch.allclose(c["w"].sum((2, 3)), torch.ones(2, 64))
    c = workloads.c5(R=1, K=32)
    assert c["w"].shape == (1, 64, 64, 64) and torch.allclose(c["w"].sum((2, 3)), torch.ones(1, 64))
    c3 = workloads.c3(R=1, K=64)
    frac = torch.isinf(c3["b"]).float().mean().item()
    assert 0.03 < frac < 0.07
    assert workloads.lt2exp_flops(64, 64, 64, 64, 4096) == 137438953472
    assert workloads.lm2exp_flops(64, 256, 256, 4096) == 34359738368
    assert workloads.lm2exp_bytes(64, 256, 256, 4096) == 553648128
    assert workloads.lt2exp_bytes(64, 64, 64, 64, 4096) == 268435456


# --------------------------------------------------------------------- max
def test_max_ref_against_torch():
    g = torch.Generator().manual_seed(13)
    for n in (1, 2, 17, 2000):
        x = torch.randn(n, generator=g)
        v, i = torch.max(x, 0)
        assert max_ref.vmax_ref(x.numpy()) == (v.item(), i.item())
        assert max_ref.vmax_ref_fast(x.numpy()) == (v.item(), i.item())
    x = torch.tensor([1.0, 5.0, 5.0, -2.0, 5.0])
    assert max_ref.vmax_ref(x.numpy()) == (5.0, 1)
    x = torch.tensor([1.0, float("nan"), 7.0, float("nan")])
    v, i = max_ref.vmax_ref(x.numpy())
    tv, ti = torch.max(x, 0)
    assert math.isnan(v) and math.isnan(tv.item()) and i == ti.item() == 1
    x = torch.full((5,), NINF)
    assert max_ref.vmax_ref(x.numpy()) == (NINF, 0) and torch.max(x, 0)[1].item() == 0
    m = torch.randn(23, 31, generator=g)
    for ax in (0, 1):
        assert np.array_equal(max_ref.matmax_ref(m.numpy(), ax), torch.amax(m, ax).numpy())


# ----------------------------------------------------------------- goldens
@pytest.mark.parametrize("name", ["lm2exp_small", "lm2exp_ragged"])
def test_golden_lm2exp_oracle(name):
    z = np.load(GOLDEN / f"{name}.npz")
    _close(oracle64.lm2exp64(z["a"], z["b"]), z["c"])
    _close(oracle64.lm2exp_lse(z["a"], z["b"]), z["c"], tol=1e-10)
    assert np.isneginf(z["c"]).sum() > 0


@pytest.mark.parametrize("name", ["lt2exp_small", "lt2exp_ragged"])
def test_golden_lt2exp_oracle(name):
    z = np.load(GOLDEN / f"{name}.npz")
    _close(oracle64.lt2exp64(z["w"], z["a"], z["b"]), z["c"])
    _close(oracle64.lt2exp_lse(z["w"], z["a"], z["b"]), z["c"], tol=1e-10)
    assert np.isneginf(z["c"]).sum() > 0


def test_golden_max_oracle():
    z = np.load(GOLDEN / "vmax_ties.npz")
    v, i = torch.max(torch.from_numpy(z["x"]), 0)
    assert v.item() == z["value"] and i.item() == z["index"]
    z = np.load(GOLDEN / "matmax_small.npz")
    x = torch.from_numpy(z["x"])
    assert np.array_equal(torch.amax(x, 0).numpy(), z["axis0"])
    assert np.array_equal(torch.amax(x, 1).numpy(), z["axis1"])


# ---- the plain C restatement (oracle/oracle_c.c) against the torch / NumPy oracle: two
# implementations that share no code (libm scalar loops on one side, ATen on the other)
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 5, 7, 6), (3, 17, 33, 20)])
@pytest.mark.parametrize("p_inf", [0.0, 0.3])
def test_c_restatement_lm2exp(shape, p_inf):
    from oracle import oracle_c

    a, b = (t.float() for t in _rand_lm(21, *shape, p_inf=p_inf))  # fp32 values, as the kernels get them
    b[0, :, 0] = NINF  # an all -inf column: -inf out, never NaN
    got, want = oracle_c.lm2exp_c(a, b), oracle64.lm2exp64(a, b).numpy()
    assert np.array_equal(np.isneginf(got), np.isneginf(want)) and not np.isnan(got).any()
    _close(torch.from_numpy(got), torch.from_numpy(want))
    _close(torch.from_numpy(got), torch.from_numpy(oracle64.lm2exp_lse(a, b)))


@pytest.mark.parametrize("shape", [(1, 1, 1, 1, 1), (2, 3, 4, 5, 6), (2, 9, 7, 3, 17)])
@pytest.mark.parametrize("p_inf", [0.0, 0.3])
def test_c_restatement_lt2exp(shape, p_inf):
    from oracle import oracle_c

    w, a, b = (t.float() for t in _rand_lt(22, *shape, p_inf=p_inf))
    got, want = oracle_c.lt2exp_c(w, a, b), oracle64.lt2exp64(w, a, b).numpy()
    assert np.array_equal(np.isneginf(got), np.isneginf(want)) and not np.isnan(got).any()
    _close(torch.from_numpy(got), torch.from_numpy(want))
    _close(torch.from_numpy(got), torch.from_numpy(oracle64.lt2exp_lse(w, a, b)))


def test_c_restatement_clamp_and_nan():
    from oracle import oracle_c

    a = torch.tensor([[[1.0, 2.0]]])
    b = torch.tensor([[[NINF, 3.0, float("nan")], [NINF, 1.0, 0.0]]])
    got = oracle_c.lm2exp_c(a, b)[0, 0]
    assert np.isneginf(got[0])                       # all -inf column: the clamp keeps exp(-inf - m) = 0
    assert abs(got[1] - math.log(math.exp(3.0) + 2 * math.exp(1.0))) < 1e-12
    assert np.isnan(got[2])                          # a NaN poisons its column, as in the torch recipe


def test_c_restatement_max():
    from oracle import max_ref, oracle_c

    g = torch.Generator().manual_seed(23)
    x = (torch.randn(37, 53, generator=g) * 3).round()  # many ties
    for axis in (0, 1):
        assert np.array_equal(oracle_c.matmax_c(x, axis), torch.amax(x, axis).numpy())
    flat = x.reshape(-1)
    assert oracle_c.vmax_c(flat) == max_ref.vmax_ref_fast(flat.numpy())
    v, i = torch.max(flat, 0)
    assert oracle_c.vmax_c(flat) == (v.item(), i.item())
    flat[100] = float("nan")
    flat[7] = float("nan")
    v, i = oracle_c.vmax_c(flat)
    assert math.isnan(v) and i == 7                  # the first NaN
    y = x.clone()
    y[3, 4] = float("nan")
    assert np.isnan(oracle_c.matmax_c(y, 0)[4]) and np.isnan(oracle_c.matmax_c(y, 1)[3])
