"""matmax / vmax / vamax on the GPU: bit-exact against torch.amax / torch.max
(the reference's own ground truth, tests/max.py:13,22,32) and against the
brute-force NumPy rule in oracle/max_ref.py."""

import itertools
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import max_ref
from triturus.max import matmax, vamax, vmax
from triturus_amd import _lib

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).resolve().parent / "golden"


def _same(got: torch.Tensor, want: torch.Tensor):
    got = got.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    assert torch.equal(torch.nan_to_num(got, nan=0.0), torch.nan_to_num(want, nan=0.0))


# ---- the reference's own tests (tests/max.py), same shapes and parameters
@pytest.mark.parametrize("block_size", [2, 32, 128])
def test_max_vamax(dev, block_size):
    x = torch.randn(2000)
    m = vamax(x.to(dev), block_size=block_size)
    assert m.shape == () and torch.all(torch.amax(x, dim=0) == m.cpu())


@pytest.mark.parametrize("block_size", [2, 32, 128])
def test_max_vmax(dev, block_size):
    x = torch.randn(2000)
    gt_m, gt_i = torch.max(x, dim=0)
    m, i = vmax(x.to(dev), block_size=block_size)
    assert m.shape == () and i.shape == () and i.dtype == torch.int64
    assert torch.all(gt_m == m.cpu()) and torch.all(gt_i == i.cpu())


@pytest.mark.parametrize("block_size,axis", itertools.product([2, 32, 128], [0, 1]))
def test_max_matmax(dev, block_size, axis):
    x = torch.randn(200, 150)
    m = matmax(x.to(dev), axis=axis, block_size=block_size)
    assert torch.all(torch.amax(x, dim=axis) == m.cpu())


# ---- sizes, alignment, ties, special values
@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 63, 64, 65, 255, 1023, 1025, 4099, 100003, 1 << 20, (1 << 22) + 7])
def test_vmax_sizes(dev, n):
    x = torch.randn(n)
    v, i = vmax(x.to(dev))
    rv, ri = max_ref.vmax_ref_fast(x.numpy())
    assert (v.item(), i.item()) == (rv, ri)
    assert vamax(x.to(dev)).item() == rv


@pytest.mark.parametrize("n,offset", [((1 << 23) + 5, 0), (9_000_001, 3), (1 << 24, 0), (20_000_000, 1)])
def test_vmax_of_vectors_too_large_for_the_cache(dev, n, offset):
    """Operands of 32 MiB and more are swept with read-once loads, each workgroup over a run of
    consecutive blocks: ties (lowest index wins), a NaN (first one wins) and all -inf are placed
    across the seams of those runs."""
    g = torch.Generator().manual_seed(n)
    base = torch.round(torch.randn(n + offset, generator=g) * 4) / 4  # many ties
    x = base[offset:]
    xg = base.to(dev)[offset:]
    gv, gi = torch.max(x, 0)
    v, i = vmax(xg)
    assert (v.item(), i.item()) == (gv.item(), gi.item())
    assert vamax(xg).item() == gv.item()
    # one maximum, planted at the seams of the workgroups' runs and at both ends
    top = gv.item() + 1.0
    for pos in (0, 1, 2047 * 4, 2048 * 4, n // 512, n // 512 + 1, n // 2 - 1, n // 2, n - 2049 * 4, n - 2, n - 1):
        y = xg.clone()
        y[pos] = top
        v, i = vmax(y)
        assert (v.item(), i.item()) == (top, pos), pos
    # two equal maxima in different runs: the first is reported
    y = xg.clone()
    y[n - 3] = top
    y[n // 3] = top
    v, i = vmax(y)
    assert (v.item(), i.item()) == (top, n // 3)
    # a NaN wins, the first of two is reported
    y = xg.clone()
    y[n - 7] = float("nan")
    y[n // 5] = float("nan")
    v, i = vmax(y)
    assert math.isnan(v.item()) and i.item() == n // 5
    assert math.isnan(vamax(y).item())
    # nothing but -inf: index 0
    y = torch.full_like(xg, float("-inf"))
    v, i = vmax(y)
    assert (v.item(), i.item()) == (float("-inf"), 0)


@pytest.mark.parametrize("offset", [1, 2, 3, 5])
def test_vmax_unaligned_views(dev, offset):
    base = torch.randn(5000)
    xg = base.to(dev)[offset:]
    gv, gi = torch.max(base[offset:], 0)
    v, i = vmax(xg)
    assert (v.item(), i.item()) == (gv.item(), gi.item())
    assert vamax(xg[: 4096 - offset]).item() == base[offset:4096].max().item()


def test_vmax_ties_go_to_the_lowest_index(dev):
    z = np.load(GOLDEN / "vmax_ties.npz")
    v, i = vmax(torch.from_numpy(z["x"]).to(dev))
    assert v.item() == z["value"] and i.item() == z["index"]
    # the maximum repeated across wavefronts, workgroups and vector lanes
    x = torch.zeros(1 << 20)
    for first in (0, 3, 64, 255, 256, 1027, 70001, (1 << 20) - 1):
        y = x.clone()
        y[first:] = 1.0
        y[first::7] = 2.0
        v, i = vmax(y.to(dev))
        assert (v.item(), i.item()) == (2.0, first)
    v, i = vmax(torch.full((300001,), -3.5).to(dev))
    assert (v.item(), i.item()) == (-3.5, 0)


def test_vmax_special_values(dev):
    ninf = float("-inf")
    v, i = vmax(torch.full((70000,), ninf).to(dev))
    assert (v.item(), i.item()) == (ninf, 0)
    x = torch.full((70000,), ninf)
    x[69999] = -1e38
    v, i = vmax(x.to(dev))
    assert (v.item(), i.item()) == (x[69999].item(), 69999)
    x = torch.randn(100000)
    x[[777, 50000]] = float("inf")
    v, i = vmax(x.to(dev))
    assert (v.item(), i.item()) == (float("inf"), 777)
    # NaN wins and reports the first NaN, like torch.max
    x = torch.randn(100000)
    x[[99999, 4242, 65000]] = float("nan")
    x[10] = float("inf")
    gv, gi = torch.max(x, 0)
    v, i = vmax(x.to(dev))
    assert math.isnan(v.item()) and math.isnan(gv.item()) and i.item() == gi.item() == 4242
    assert math.isnan(vamax(x.to(dev)).item())
    x = torch.tensor([0.0, -0.0, 0.0])
    v, i = vmax(x.to(dev))
    assert v.item() == 0.0 and i.item() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n", [3, 9, 41, 75, 8875, 70001, (1 << 20) + 3, 3790651])
def test_vmax_of_nothing_but_minus_infinity(dev, dtype, n):
    """Every element -inf: index 0 whatever the length -- also when the vector ends in elements
    that do not fill a 16-byte piece, or starts off a 16-byte boundary -- and a finite value or a
    later -inf must not disturb the first-occurrence rule."""
    ninf = float("-inf")
    for off in (0, 1, 3):
        base = torch.full((n + off,), ninf, dtype=dtype)
        v, i = vmax(base.to(dev)[off:])
        assert (v.item(), i.item()) == (ninf, 0), (n, off)
        base[off + n - 1] = -3.0  # the only finite value: last element (in the scalar tail for most n)
        v, i = vmax(base.to(dev)[off:])
        assert (v.item(), i.item()) == (-3.0, n - 1), (n, off)
        assert vamax(base.to(dev)[off:]).item() == -3.0


@pytest.mark.parametrize("dtype", [torch.float64, torch.float16, torch.bfloat16])
def test_other_float_dtypes(dev, dtype):
    x = torch.randn(50001).to(dtype)
    gv, gi = torch.max(x.float() if dtype != torch.float64 else x, 0)
    v, i = vmax(x.to(dev))
    assert v.dtype == dtype and v.item() == gv.item() and i.item() == gi.item()
    assert vamax(x.to(dev)).item() == gv.item()
    m = torch.randn(301, 257).to(dtype)
    for axis in (0, 1):
        _same(matmax(m.to(dev), axis), torch.amax(m, axis))
    m = torch.randn(256, 512).to(dtype)
    for axis in (0, 1):
        _same(matmax(m.to(dev), axis), torch.amax(m, axis))


@pytest.mark.parametrize("dtype", [torch.float64, torch.float16, torch.bfloat16])
def test_other_float_dtypes_beyond_the_cache(dev, dtype):
    """Operands of 32 MiB and more take the read-once loads in every element width."""
    wide = dtype == torch.float64
    n = 5_000_003 if wide else 18_000_005
    g = torch.Generator().manual_seed(3)
    x = torch.randn(n, generator=g).to(dtype)
    ref = x if wide else x.float()
    gv, gi = torch.max(ref, 0)
    xg = x.to(dev)
    v, i = vmax(xg)
    assert v.dtype == dtype and v.item() == gv.item() and i.item() == gi.item()
    assert vamax(xg).item() == gv.item()
    rows, cols = (2100, 2048) if wide else (4200, 4096)
    m = xg[: rows * cols].view(rows, cols)
    mref = ref[: rows * cols].view(rows, cols)
    for axis in (0, 1):
        _same(matmax(m, axis), torch.amax(mref, axis).to(dtype))
    m[rows // 2, 17] = float("nan")
    m[3, cols - 1] = float("-inf")
    mref = m.cpu() if wide else m.cpu().float()
    for axis in (0, 1):
        _same(matmax(m, axis), torch.amax(mref, axis).to(dtype))


@pytest.mark.parametrize(
    "shape",
    [(1, 1), (1, 7), (7, 1), (23, 31), (64, 64), (65, 127), (200, 150), (1000, 3), (3, 1000), (2, 300000),
     (300000, 2), (513, 1024), (4096, 256), (5, 65536), (65537, 5), (65536, 256), (40000, 64), (5000, 130),
     (16400, 4100), (8200, 8196)],  # 256 MiB and more: two 16-byte pieces per lane along axis 0, ragged last block
)
def test_matmax_shapes(dev, shape):
    x = torch.randn(*shape)
    for axis in (0, 1):
        y = matmax(x.to(dev), axis)
        assert y.is_contiguous()
        _same(y, torch.amax(x, axis))
        assert np.array_equal(y.cpu().numpy(), max_ref.matmax_ref(x.numpy(), axis))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1024, 4096), (1500, 4100), (1025, 8200), (2048, 16384)])
def test_matmax_long_rows(dev, dtype, shape):
    """Many rows of at least 16 KiB take the workgroup-per-row kernel along axis 1 (whole
    blocks, a partial block and a scalar tail, depending on the row length)."""
    m, n = shape
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, n, generator=g).to(dtype)
    x[3, n - 1] = 50.0          # maximum in the scalar tail
    x[4, 0] = 60.0
    x[7, n // 2] = float("nan")
    x[9, :] = float("-inf")
    xg = x.to(dev)
    for axis in (0, 1):
        _same(matmax(xg, axis), torch.amax(x, axis))
    # the same rows through a view that is only element-aligned (other kernel path)
    base = torch.zeros(m * n + 1, dtype=dtype)
    base[1:] = x.reshape(-1)
    _same(matmax(base.to(dev)[1:].view(m, n), 1), torch.amax(x, 1))


def test_matmax_golden_and_views(dev):
    z = np.load(GOLDEN / "matmax_small.npz")
    x = torch.from_numpy(z["x"]).to(dev)
    assert np.array_equal(matmax(x, 0).cpu().numpy(), z["axis0"])
    assert np.array_equal(matmax(x, 1).cpu().numpy(), z["axis1"])
    # contiguous but 4-byte aligned storage (a view into a larger buffer)
    base = torch.randn(1 + 300 * 129)
    v = base[1:].view(300, 129)
    for axis in (0, 1):
        _same(matmax(base.to(dev)[1:].view(300, 129), axis), torch.amax(v, axis))


def test_matmax_special_values(dev):
    x = torch.randn(300, 500)
    x[5, :] = float("-inf")
    x[:, 7] = float("-inf")
    x[17, 33] = float("nan")
    x[200, 400] = float("inf")
    for axis in (0, 1):
        _same(matmax(x.to(dev), axis), torch.amax(x, axis))


def test_max_on_the_large_lt2exp_operand(dev):
    """matmax along both axes and vmax with indices on the 64 x 64 x 4096 log-space
    operand of the large lt2exp configuration, bit-exact against torch."""
    from triturus_amd import workloads

    b = workloads.c5()["b"]
    bg = b.to(dev)
    flat = b.view(4096, 4096)
    for axis in (0, 1):
        _same(matmax(bg.view(4096, 4096), axis), torch.amax(flat, axis))
    for r in (0, 31, 63):
        for axis in (0, 1):
            _same(matmax(bg[r], axis), torch.amax(b[r], axis))
    gv, gi = torch.max(b.view(-1), 0)
    v, i = vmax(bg.view(-1))
    assert (v.item(), i.item()) == (gv.item(), gi.item())
    # duplicate the maximum later in the vector: the first one must still win
    b2 = b.clone().view(-1)
    b2[-1] = gv
    v, i = vmax(b2.to(dev))
    assert (v.item(), i.item()) == (gv.item(), gi.item())
    assert vamax(bg.view(-1)).item() == gv.item()


def test_runs_on_the_current_stream_without_synchronising(dev):
    x = torch.randn(1 << 20)
    xg = x.to(dev)
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        v, i = vmax(xg)
        y = matmax(xg.view(1024, 1024), 1)
    s.synchronize()
    assert (v.item(), i.item()) == tuple(t.item() for t in torch.max(x, 0))
    _same(y, torch.amax(x.view(1024, 1024), 1))


def test_a_captured_graph_survives_the_growth_of_its_workspace(dev):
    """A graph captured on a stream launches kernels that count in the workspace that was current
    for the stream at capture time.  A later call on that stream that needs a larger workspace
    must not hand the old one back to the allocator while the graph can still be replayed."""
    x = torch.randn(1 << 21)
    xg = x.to(dev)
    want = tuple(t.item() for t in torch.max(x, 0))
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        vmax(xg)  # the stream's first workspace: the small one of vmax
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        v, i = vmax(xg)
    wide = torch.randn(4096, 8192, device=dev)
    with torch.cuda.stream(s):
        y = matmax(wide, 0)  # partial rows of 32 splits: a larger workspace replaces the first
        fill = [torch.full((1 << 14,), float(k), device=dev) for k in range(64)]  # would land in a freed block
    s.synchronize()
    _same(y, torch.amax(wide, 0).cpu())
    for _ in range(3):
        g.replay()
        torch.cuda.synchronize()
        assert (v.item(), i.item()) == want
    for k, f in enumerate(fill):
        assert torch.all(f == float(k))


def test_c_abi_with_a_workspace_prepared_by_the_library(dev):
    """A C caller's workspace: garbage from the allocator, its arrival counters zeroed once by
    trt_max_workspace_init; several calls of both reductions then share it (every call leaves
    the counters zero)."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3000, 4100, generator=g)
    x[17, 33] = float("nan")
    xg = x.to(dev)
    n = x.numel()
    need = max(lib.trt_vmax_workspace_bytes(n, _lib.TRT_F32), lib.trt_matmax_workspace_bytes(3000, 4100, 0, _lib.TRT_F32),
               lib.trt_matmax_workspace_bytes(3000, 4100, 1, _lib.TRT_F32))
    ws = torch.full((need,), 0xAB, dtype=torch.uint8, device=dev)
    stream = _lib.raw_stream(dev)
    with _lib.on_device(dev):
        _lib.check(lib.trt_max_workspace_init(ws.data_ptr(), need, stream), "trt_max_workspace_init")
        for _ in range(3):
            val = torch.empty((), device=dev)
            idx = torch.empty((), dtype=torch.int64, device=dev)
            _lib.check(lib.trt_vmax(xg.data_ptr(), n, _lib.TRT_F32, val.data_ptr(), idx.data_ptr(), ws.data_ptr(), need,
                                    stream), "trt_vmax")
            gv, gi = torch.max(x.view(-1), 0)
            assert torch.isnan(val).item() and idx.item() == gi.item()
            for axis in (0, 1):
                y = torch.empty(x.shape[1 - axis], device=dev)
                _lib.check(lib.trt_matmax(xg.data_ptr(), y.data_ptr(), 3000, 4100, axis, _lib.TRT_F32, ws.data_ptr(),
                                          need, stream), "trt_matmax")
                _same(y, torch.amax(x, axis))
    assert lib.trt_max_workspace_check(ws.data_ptr(), need, stream) == 0  # the counters are idle again
    assert lib.trt_vmax(xg.data_ptr(), n, _lib.TRT_F32, val.data_ptr(), idx.data_ptr(), ws.data_ptr() + 4, need - 4,
                        stream) == -2  # a workspace that is not 16-byte aligned is refused
    assert lib.trt_matmax(xg.data_ptr(), y.data_ptr(), 3000, 4100, 0, _lib.TRT_F32, ws.data_ptr() + 8, need - 8,
                          stream) == -2


@pytest.mark.parametrize("dirt", ["never prepared", "zeroed", "one counter zeroed", "random bytes"])
def test_a_workspace_with_foreign_counters_shows_in_the_result(dev, dirt):
    """Counters that no call of the library left behind (written here from the host side with torch;
    every kernel still runs to its end): the reductions then return NaN -- vmax with index -1 --
    instead of leaving garbage, trt_max_workspace_check reports TRT_E_STATE, and after
    trt_max_workspace_init the same workspace serves again."""
    lib = _lib.load()
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2048, 4096, generator=g)
    xg = x.to(dev)
    n = x.numel()
    need = max(lib.trt_vmax_workspace_bytes(n, _lib.TRT_F32), lib.trt_matmax_workspace_bytes(2048, 4096, 0, _lib.TRT_F32))
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    stream = _lib.raw_stream(dev)
    val = torch.empty((), device=dev)
    idx = torch.empty((), dtype=torch.int64, device=dev)
    y = torch.empty(4096, device=dev)

    def run_both():
        val.fill_(123.0), idx.fill_(123), y.fill_(123.0)
        with _lib.on_device(dev):
            _lib.check(lib.trt_vmax(xg.data_ptr(), n, _lib.TRT_F32, val.data_ptr(), idx.data_ptr(), ws.data_ptr(), need,
                                    stream), "trt_vmax")
            _lib.check(lib.trt_matmax(xg.data_ptr(), y.data_ptr(), 2048, 4096, 0, _lib.TRT_F32, ws.data_ptr(), need,
                                      stream), "trt_matmax")
        torch.cuda.synchronize()

    with _lib.on_device(dev):
        _lib.check(lib.trt_max_workspace_init(ws.data_ptr(), need, stream), "trt_max_workspace_init")
    head = ws[:65536]
    if dirt == "never prepared":
        head.fill_(0xAB)
    elif dirt == "zeroed":
        head.zero_()
    elif dirt == "one counter zeroed":  # the first group of vmax, the first column block of matmax
        head[:8].zero_()
    else:
        head.copy_(torch.randint(0, 256, (65536,), generator=g, dtype=torch.uint8))
    torch.cuda.synchronize()
    assert lib.trt_max_workspace_check(ws.data_ptr(), need, stream) == _lib.E_STATE
    run_both()
    gv, gi = torch.max(x.view(-1), 0)
    right = (val.item(), idx.item()) == (gv.item(), gi.item())
    assert right or (torch.isnan(val).item() and idx.item() == -1), (val.item(), idx.item())
    col_right = y.cpu() == torch.amax(x, 0)
    assert bool(torch.all(col_right | torch.isnan(y.cpu())))
    assert not (right and bool(col_right.all()))  # this dirt is not survivable: it must show
    with _lib.on_device(dev):
        _lib.check(lib.trt_max_workspace_init(ws.data_ptr(), need, stream), "trt_max_workspace_init")
    run_both()
    assert (val.item(), idx.item()) == (gv.item(), gi.item())
    _same(y, torch.amax(x, 0))
    assert lib.trt_max_workspace_check(ws.data_ptr(), need, stream) == 0


def test_the_first_reduction_of_a_stream_inside_a_graph_capture(dev):
    """A stream whose first reduction ever is recorded into a HIP graph: the workspace prepared
    during the capture is idle only when that graph runs, so neither an eager call on the stream
    nor a second graph may count in it before the first replay."""
    import triturus_amd.max as tmax

    x = torch.randn(1 << 22)
    x2 = torch.randn(3000, 1000)
    xg, x2g = x.to(dev), x2.to(dev)
    want = tuple(t.item() for t in torch.max(x, 0))
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    key = (dev.index, s.cuda_stream)
    assert key not in tmax._workspaces
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1, stream=s):
        v1, i1 = vmax(xg)
        y1 = matmax(x2g, 0)
    assert key not in tmax._workspaces  # nothing prepared under capture is kept for eager calls
    with torch.cuda.stream(s):
        v, i = vmax(xg)  # eager, before the first replay
        y = matmax(x2g, 0)
    s.synchronize()
    assert (v.item(), i.item()) == want
    _same(y, torch.amax(x2, 0))
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=s):
        v2, i2 = vmax(xg)
    for _ in range(3):
        g2.replay()
        torch.cuda.synchronize()
        assert (v2.item(), i2.item()) == want
        with torch.cuda.stream(s):
            v, i = vmax(xg)
        s.synchronize()
        assert (v.item(), i.item()) == want
        g1.replay()
        torch.cuda.synchronize()
        assert (v1.item(), i1.item()) == want
        _same(y1, torch.amax(x2, 0))


def test_workspaces_are_kept_for_a_bounded_number_of_streams(dev):
    import triturus_amd.max as tmax

    x = torch.randn(1 << 18)
    xg = x.to(dev)
    want = tuple(t.item() for t in torch.max(x, 0))
    streams = [torch.cuda.Stream(device=dev) for _ in range(tmax._MAX_STREAMS + 8)]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(s):
            v, i = vmax(xg)
        s.synchronize()
        assert (v.item(), i.item()) == want
    assert len(tmax._workspaces) <= tmax._MAX_STREAMS


@pytest.mark.parametrize("seed", range(8))
def test_random_vectors_and_matrices(dev, seed):
    """A bracketed version of a one-off randomized scan (which found the all -inf tail case
    above): lengths and shapes drawn log-uniformly, four dtypes, views off a 16-byte boundary,
    ties, NaN, +inf and vectors of nothing but -inf, against torch.max / torch.amax."""
    import random

    rng = random.Random(1000 + seed)
    dtypes = [torch.float32, torch.float64, torch.float16, torch.bfloat16]

    def logu(lo, hi):
        return int(round(2 ** rng.uniform(math.log2(lo), math.log2(hi))))

    for case in range(40):
        dt = rng.choice(dtypes)
        g = torch.Generator().manual_seed(rng.randrange(1 << 30))
        wide = (lambda t: t.float()) if dt in (torch.float16, torch.bfloat16) else (lambda t: t)
        if case % 2 == 0:
            n, off = logu(1, 1 << 21), rng.choice([0, 0, 1, 2, 3, 5])
            x = torch.randn(n + off, generator=g)
            if rng.random() < 0.3:
                x = torch.round(x * 2) / 2  # many ties
            if rng.random() < 0.2 and n > 2:
                x[rng.randrange(n + off)] = float("nan")
            if rng.random() < 0.15:
                x[:] = float("-inf")
            x = x.to(dt)
            gv, gi = torch.max(wide(x[off:]), 0)
            v, i = vmax(x.to(dev)[off:])
            assert i.item() == gi.item(), (dt, n, off)
            _same(v.float(), gv.float())
            _same(vamax(x.to(dev)[off:]).float(), gv.float())
        else:
            m, n = logu(1, 6000), logu(1, 6000)
            off = rng.choice([0, 0, 0, 1, 4])
            base = torch.randn(m * n + off, generator=g)
            if rng.random() < 0.3 and m * n > 2:
                base[rng.randrange(m * n + off)] = float("nan")
            if rng.random() < 0.2:
                base[rng.randrange(m * n + off)] = float("inf")
            base = base.to(dt)
            x = base[off:].view(m, n)
            xg = base.to(dev)[off:].view(m, n)
            for axis in (0, 1):
                _same(matmax(xg, axis), torch.amax(wide(x), axis).to(dt))


# ---- batched column maxima: the front end of the contraction recipes
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 7, 5), (4, 64, 256), (2, 300, 1000), (64, 64, 4096), (5, 33, 257),
                                   (1, 4096, 300), (2, 1000, 70), (16, 512, 512), (1, 129, 3),  # these four are cut over J
                                   (1, 70000, 40), (2, 9000, 300),  # more than 128 pieces: combined in two levels
                                   (66, 75, 2048), (2, 40000, 128), (3, 1111, 3000)])  # 32 MiB and more: read-once loads
@pytest.mark.parametrize("clamp", [False, True])
def test_bmatmax(dev, shape, clamp):
    from triturus_amd.max import bmatmax

    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(*shape, generator=g) * 50
    x[torch.rand(shape, generator=g) < 0.1] = float("-inf")
    x[0, :, 0] = float("-inf")                      # an all -inf column
    if shape[2] > 2:
        x[0, shape[1] // 2, 2] = float("nan")       # a NaN wins, as in torch.amax
        x[-1, 0, 1] = float("inf")
    want = torch.amax(x, dim=1)
    if clamp:
        want = torch.clamp(want, -1e38, 1e38)       # baselines/lm2exp.py:12
    _same(bmatmax(x.to(dev), clamp=clamp), want)
    # strided input: padded rows and a batch gap
    big = torch.full((shape[0] * 2, shape[1] + 3, shape[2] + 5), 1e30)
    v = big[::2, 1 : 1 + shape[1], 2 : 2 + shape[2]]
    v.copy_(x)
    bigg = big.to(dev)
    _same(bmatmax(bigg[::2, 1 : 1 + shape[1], 2 : 2 + shape[2]], clamp=clamp), want)


def test_bmatmax_is_the_shift_of_the_contraction(dev):
    """m = clamp(amax(b, 1)) is what lm2exp subtracts: m + log(a @ exp(b - m)) from it equals lm2exp."""
    from triturus.lm2exp import lm2exp
    from triturus_amd.max import bmatmax

    g = torch.Generator().manual_seed(8)
    a = torch.rand(3, 40, 90, generator=g).to(dev)
    b = (torch.randn(3, 90, 130, generator=g) * 10).to(dev)
    b[1, :, 7] = float("-inf")
    m = bmatmax(b, clamp=True).unsqueeze(1)
    recipe = m + torch.log(torch.bmm(a, torch.exp(b - m)))
    out = lm2exp(a, b)
    assert torch.equal(torch.isneginf(out), torch.isneginf(recipe))
    fin = torch.isfinite(recipe)
    assert torch.allclose(out[fin], recipe[fin], rtol=1e-5, atol=1e-5)
