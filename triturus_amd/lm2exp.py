"""lm2exp: batched ``log(a @ exp(b))`` on MI355X.

Same contract as the reference wrapper, triturus/lm2exp.py:167-206:
a is R x I x J (linear space), b is R x J x K (log space), both fp32 on one
device; returns a fresh R x I x K tensor, enqueued on the current stream
without synchronising.

Arithmetic: IEEE fp32 on the fp32 matrix pipe; with the reference's TF32 flag on
(is_triturus_tf32_enabled(), read at triturus/lm2exp.py:185) the bf16 matrix pipe with operands
cut into two bf16 pieces, see triturus_amd.utils.  The underscore keywords
(tile variant, split count, arithmetic) are for tests and experiments.
"""

from __future__ import annotations

import torch

from triturus_amd import _lib, autotune
from triturus_amd.utils import MATRIX_PRECISIONS, matrix_precision


_ws_bytes: dict = {}  # (R, I, J, K, variant, splits, pieces) -> workspace bytes, as reported by the library


def _unit_inner(t: torch.Tensor) -> torch.Tensor:
    # The kernels take any non-negative batch and row strides (zero included: an expanded
    # operand is read in place) but want a unit trailing stride; only a tensor without one is
    # materialised.  (A trailing axis of one element has no stride to speak of: reshaping it
    # gives it the unit stride without a copy.)
    st = t.stride()
    if st[-1] == 1 and min(st) >= 0:
        return t
    if t.shape[-1] == 1 and min(st[:-1]) >= 0:
        return t.as_strided(t.shape, (*st[:-1], 1), t.storage_offset())
    return t.contiguous()


_PIECES = {"bf16x3": 2, "bf16x6": 3}
# from this output width and this much work on, rows of a that are not a multiple of 4 long are
# padded on the bf16 paths (tests lower the thresholds, or pass _pad, to reach that path on small inputs)
_PAD_MIN_K = 2048
_PAD_MIN_FLOPS = 2e9
# tile variants worth timing when tuning is on (0 = the library's rule)
_FP32_CANDIDATES = (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17)
_BF16_CANDIDATES = (0, 1, 2, 3, 4, 8, 9)


def lm2exp(
    a: torch.Tensor, b: torch.Tensor, *, _variant: int = 0, _splits: int = 0, _precision: str | None = None,
    _pad: bool | None = None,
) -> torch.Tensor:
    ash, bsh = a.shape, b.shape
    assert len(ash) == len(bsh) == 3
    assert ash[0] == bsh[0]
    assert ash[2] == bsh[1]
    assert a.dtype == b.dtype == torch.float32
    dev = a.device
    assert dev == b.device
    if not a.is_cuda:
        _lib.require_gpu(a, b)
    lib = _lib._lib or _lib.load()

    R, I, J = ash
    K = bsh[2]
    c = a.new_empty((R, I, K))
    if R * I * K == 0:
        return c
    if J == 0:
        # empty contraction: log(0)
        return c.fill_(float("-inf"))
    if _precision is None:
        _precision = matrix_precision()
    elif _precision not in MATRIX_PRECISIONS:
        raise ValueError(f"unknown matrix precision {_precision!r}")
    fp32 = _precision == "fp32"
    # Operands go to the kernels with whatever non-negative strides they have, as the reference
    # forwards them (triturus/lm2exp.py:190-198): b in every kernel (a lane owns a column of b,
    # so a trailing stride only scales its offsets) and a (on the fp32 pipe the paired-wavefront
    # tiles read a transposed or strided a in place -- a forced tile of another family wants
    # unit-stride rows --, on the bf16 pipe the element-staging builds do).  Only negative
    # strides always need a copy.
    sa, sb = a.stride(), b.stride()
    pair_tile = _variant == 0 or _variant > lib.trt_lm2exp_variant_count() - 5
    if (fp32 and not pair_tile and sa[2] != 1) or min(sa) < 0:
        a = _unit_inner(a)
        sa = a.stride()
    if min(sb) < 0:
        b = b.contiguous()
        sb = b.stride()
    if _variant == 0 and _splits == 0 and sa[2] == 1 and autotune.is_autotune_enabled():
        cands = _FP32_CANDIDATES if fp32 else _BF16_CANDIDATES
        _variant = autotune.pick(("lm2exp", R, I, J, K, _precision), cands,
                                 lambda v: lm2exp(a, b, _variant=v, _splits=-1, _precision=_precision))
    # Rows of a are read 16 bytes at a time when they start aligned; with J not a multiple of 4 a
    # contiguous a does not qualify and the kernels stage it element by element.  The bf16 paths
    # then run a call with enough work on a copy of a whose rows are padded to a multiple of 4; on
    # the fp32 path the copy no longer pays (timed on 50 shapes with J = 9..1347: of the nine the
    # work thresholds would have padded, six ran 3-18 % slower and three 1-3 % faster).
    # _pad: True / False force the copy / its absence (tests, timing).
    pad = (not fp32 and K >= _PAD_MIN_K and 2 * R * I * J * K >= _PAD_MIN_FLOPS) if _pad is None else _pad
    if J % 4 != 0 and J > 4 and sa[2] == 1 and pad:
        a = torch.nn.functional.pad(a, (0, (-J) % 4))[..., :J]
        sa = a.stride()
    if _splits < 0:  # tuning launch: the library decides the split for this tile
        _splits = 0
    # small grids with a long contraction are cut over J; the partial sums need a workspace
    fp32_variant = _variant if fp32 else 0
    pieces = 0 if fp32 else _PIECES[_precision]
    key = (R, I, J, K, fp32_variant, _splits, pieces)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = lib.trt_lm2exp_workspace_bytes(R, I, J, K, fp32_variant, _splits)
        if pieces:  # the bf16 entry may cut a small grid itself
            ws_bytes = max(ws_bytes, lib.trt_lm2exp_bf16_workspace_bytes(R, I, J, K, pieces, _splits))
        _ws_bytes[key] = ws_bytes
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        ws_ptr = ws.data_ptr()
    else:
        ws_ptr = None
    stride_array = _lib.stride_array
    with _lib.on_device(dev):
        if fp32:
            status = lib.trt_lm2exp_f32(
                a.data_ptr(), b.data_ptr(), c.data_ptr(),
                R, I, J, K, stride_array(sa), stride_array(sb), stride_array((I * K, K, 1)),
                _variant, _splits, ws_ptr, ws_bytes, _lib.raw_stream(dev),
            )
        else:
            # bf16 matrix pipe; a grid too small for it has its contraction cut over J or goes
            # back to the fp32 kernels (which may cut it as well: hence the workspace)
            status = lib.trt_lm2exp_bf16(
                a.data_ptr(), b.data_ptr(), c.data_ptr(),
                R, I, J, K, stride_array(sa), stride_array(sb), stride_array((I * K, K, 1)),
                pieces, _variant, _splits, ws_ptr, ws_bytes, _lib.raw_stream(dev),
            )
    if status:
        _lib.check(status, "trt_lm2exp_f32" if fp32 else "trt_lm2exp_bf16")
    return c
