"""The entry point that allocates nothing, trt_lt2exp_f32_static, through the C ABI: its
split-mode workspace is a device array inside the library.  Its output must equal that of
trt_lt2exp_f32 (which takes a caller's workspace) bit for bit, and pass the accuracy gate
against the float64 oracle, on two calls in a row, the second on a smaller input."""

import ctypes

import pytest
import torch

from oracle import oracle64
from triturus_amd import _lib

pytestmark = pytest.mark.gpu


def _inputs(shape, seed, dev):
    R, S, I, J, K = shape
    g = torch.Generator().manual_seed(seed)
    w = torch.rand(R, S, I, J, generator=g)
    w = w / w.sum(dim=(2, 3), keepdim=True)
    a = -20 + 5 * torch.randn(R, I, K, generator=g)
    b = -20 + 5 * torch.randn(R, J, K, generator=g)
    a[torch.rand(a.shape, generator=g) < 0.05] = float("-inf")
    b[:, :, 3] = float("-inf")
    return (w, a, b), tuple(t.to(dev) for t in (w, a, b))


def _call(lib, static, wg, ag, bg, mode):
    R, S, I, J = wg.shape
    K = ag.shape[2]
    w3 = wg.view(R, S, I * J)
    c = torch.full((R, S, K), float("nan"), device=wg.device)
    common = (w3.data_ptr(), ag.data_ptr(), bg.data_ptr(), c.data_ptr(), R, S, I, J, K,
              _lib.strides3(w3), _lib.strides3(ag), _lib.strides3(bg), _lib.strides3(c), mode, 0)
    stream = _lib.raw_stream(wg.device)
    if static:
        status = lib.trt_lt2exp_f32_static(*common, stream)
    else:
        need = lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, mode)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=wg.device)
        status = lib.trt_lt2exp_f32(*common, ws.data_ptr() if need else None, need, stream)
    torch.cuda.synchronize()
    return status, c


def test_static_scratch_entry_point_matches_the_workspace_entry_point(dev):
    lib = _lib.load()
    # the reference's test shape first (a long contraction under a small grid: split mode cuts
    # it), then a smaller input: the scratch array still holds the first call's partial sums
    for n, shape in enumerate([(3, 75, 50, 50, 100), (2, 40, 30, 20, 70)]):
        (w, a, b), (wg, ag, bg) = _inputs(shape, 100 + n, dev)
        ref = oracle64.lt2exp64(w, a, b)
        for mode in (_lib.MODE_SPLIT, _lib.MODE_AUTO, _lib.MODE_UNSPLIT):
            R, S, I, J, K = shape
            need = lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, mode)
            assert need <= _lib.STATIC_SCRATCH_BYTES and (need > 0 or mode != _lib.MODE_SPLIT)
            before = torch.cuda.memory_allocated()
            st1, c1 = _call(lib, True, wg, ag, bg, mode)
            grown = torch.cuda.memory_allocated() - before
            st0, c0 = _call(lib, False, wg, ag, bg, mode)
            assert st1 == 0 and st0 == 0, (shape, mode, st1, st0)
            assert grown <= c1.numel() * 4 + 1024  # the output of the test itself, nothing else
            assert torch.equal(c1, c0), (shape, mode)
            r = oracle64.compare(c1, ref)
            assert r["ok"] and r["n_neg_inf"] >= R * S, (shape, mode, r)
    assert lib.trt_lt2exp_workspace_bytes(3, 75, 50, 50, 100, _lib.MODE_SPLIT) > 0  # the scratch array was in use


def test_static_scratch_entry_point_takes_no_memory_from_the_driver(dev):
    """torch's own counters cannot see a hipMalloc made inside the library: the free memory that
    the driver reports must be the same before and after a call whose tensors all exist already
    (a warm-up call first: the first call on a device looks up the scratch array's address)."""
    lib = _lib.load()
    shape = (3, 75, 50, 50, 100)
    R, S, I, J, K = shape
    (w, a, b), (wg, ag, bg) = _inputs(shape, 100, dev)
    w3 = wg.view(R, S, I * J)
    c = torch.empty(R, S, K, device=dev)
    args = (w3.data_ptr(), ag.data_ptr(), bg.data_ptr(), c.data_ptr(), R, S, I, J, K,
            _lib.strides3(w3), _lib.strides3(ag), _lib.strides3(bg), _lib.strides3(c), _lib.MODE_SPLIT, 0)
    stream = _lib.raw_stream(dev)
    assert lib.trt_lt2exp_f32_static(*args, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    reserved_before = torch.cuda.memory_reserved(dev)
    for _ in range(3):
        assert lib.trt_lt2exp_f32_static(*args, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert torch.cuda.memory_reserved(dev) == reserved_before  # torch took nothing from the driver in between
    assert free_after == free_before, (free_before, free_after)
    assert oracle64.compare(c, oracle64.lt2exp64(w, a, b))["ok"]


def test_static_scratch_entry_point_refuses_what_does_not_fit(dev):
    lib = _lib.load()
    shape = (64, 512, 8, 8, 1024)  # split mode: some ten copies of a 128 MiB output
    R, S, I, J, K = shape
    assert lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, _lib.MODE_SPLIT) > _lib.STATIC_SCRATCH_BYTES
    # real tensors of that shape (were the refusal to regress, the kernels would run on valid memory)
    wg = torch.rand(R, S, I * J, device=dev)
    ag, bg = torch.randn(R, I, K, device=dev), torch.randn(R, J, K, device=dev)
    c = torch.full((R, S, K), 7.0, device=dev)
    s3 = (ctypes.c_int64 * 3)
    args = (wg.data_ptr(), ag.data_ptr(), bg.data_ptr(), c.data_ptr(), R, S, I, J, K,
            s3(S * I * J, I * J, 1), s3(I * K, K, 1), s3(J * K, K, 1), s3(S * K, K, 1))
    assert lib.trt_lt2exp_f32_static(*args, _lib.MODE_SPLIT, 0, _lib.raw_stream(dev)) == _lib.E_SCRATCH
    torch.cuda.synchronize()
    assert bool((c == 7.0).all())  # nothing was enqueued
    assert b"scratch" in lib.trt_error_string(_lib.E_SCRATCH)
    # unsplit needs no scratch at all, whatever the size
    (w, a, b), (wg, ag, bg) = _inputs((2, 33, 5, 7, 40), 7, dev)
    st, c = _call(lib, True, wg, ag, bg, _lib.MODE_UNSPLIT)
    assert st == 0 and oracle64.compare(c, oracle64.lt2exp64(w, a, b))["ok"]
