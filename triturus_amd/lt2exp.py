"""lt2exp: batched log-space Tucker-2 contraction on MI355X.

Same contract as the reference wrapper, triturus/lt2exp.py:519-630:
w is R x S x I x J (linear space), a is R x I x K, b is R x J x K (log space),
all fp32 on one device; returns a fresh R x S x K tensor.  ``mode`` is
"auto" | "split" | "unsplit"; anything else raises ValueError.  w must be
viewable as R x S x (I*J) (``w.view`` raises RuntimeError otherwise, as in the
reference).

Arithmetic: IEEE fp32 on the fp32 matrix pipe; with the reference's TF32 flag on
(is_triturus_tf32_enabled(), read at triturus/lt2exp.py:551) the bf16 matrix pipe with operands
cut into two bf16 pieces, see triturus_amd.utils.  The underscore keywords
(tile variant, split count, arithmetic) are for tests and experiments.
"""

from __future__ import annotations

import torch

from triturus_amd import _lib, autotune
from triturus_amd.lm2exp import _unit_inner
from triturus_amd.utils import MATRIX_PRECISIONS, matrix_precision

_ws_bytes: dict = {}  # (R, S, I, J, K, mode, pieces) -> workspace bytes, as reported by the library

_MODES = {"auto": _lib.MODE_AUTO, "split": _lib.MODE_SPLIT, "unsplit": _lib.MODE_UNSPLIT}


def launches_split(R: int, S: int, I: int, J: int, K: int, mode: str) -> bool:
    """The reference's mode rule, triturus/lt2exp.py:534-541."""
    if mode == "auto":
        return R * S * K < 1048576 and I * J > 512
    if mode == "split":
        return True
    if mode == "unsplit":
        return False
    raise ValueError(f"Uknown mode '{mode}' for the l2exp kernel")


_PIECES = {"bf16x3": 2, "bf16x6": 3}
# tile variants worth timing when tuning is on (0 = the library's rule)
_FP32_CANDIDATES = (0, 1, 2, 4, 5, 6, 7, 8, 9, 10, 13, 14)
_BF16_CANDIDATES = (0, 1, 2, 3, 4, 9, 10, 11, 12)


# Thresholds of the two reshaping front ends below (tests lower them to reach those paths on
# small inputs): padded work that repays a copy kernel, and the output width from which padding
# J to a multiple of 4 pays.
_RESHAPE_MIN_FLOPS = 4e9
_PAD_MIN_K = 1024
_PACK_PAD_MIN_FLOPS = 2e10  # padded work from which rows of 3, 5, 6, 7 are worth padding to 4 or 8 (fp32)


def _padded(n: int) -> int:
    """Length of a contracted axis of n once padded to whole j-chunks of the size that fits it best."""
    return min(-(-n // c) * c for c in (16, 24, 32, 48))


def _padded_by_element(n: int) -> int:
    """The same for rows of w that are not 16-byte aligned: staged by element, in chunks of 16 or 32 only."""
    return min(-(-n // c) * c for c in (16, 32))


def _kernel_us(R: int, S: int, I: int, J: int, K: int) -> float:
    """Rough time of the fp32 contraction kernel on these sizes, for weighing one front end
    against another (microseconds, without the launch): the padded work -- S to tiles of 32
    rows, K to one 64-column tile or tiles of 128, J to whole chunks -- at 109 TFLOP/s, less on
    a grid that leaves compute units idle (fill ** 0.38) and on rows of w that are not 16-byte
    aligned (0.89), or w streamed at 2.65 TB/s where that takes longer."""
    tiles = R * -(-S // 32) * (1 if K <= 64 else -(-K // 128))
    fill = min(1.0, tiles / 256.0)
    padded_j = _padded(J) if J % 4 == 0 else _padded_by_element(J)
    flops = 2.0 * R * (-(-S // 32) * 32) * I * padded_j * (64 if K <= 64 else -(-K // 128) * 128)
    compute = flops / (109e6 * fill ** 0.38 * (1.0 if J % 4 == 0 else 0.89))
    stream = R * S * I * J * 4 / 2.65e6
    return max(compute, stream)


def _exchange_pays(R: int, S: int, I: int, J: int, K: int) -> bool:
    """fp32 path: is the call faster with the roles of (i, a) and (j, b) exchanged, transposed
    copy of w included?
    Rows of at most 8 values: by the model above, the copy at 6.2 us and its traffic at 9.7 TB/s
    (w is often still in cache).  The constants here and in _kernel_us were fitted to 378 shapes
    timed both ways (R = 1..256, S = 4..1024, J = 2..24 under I = 3..400, K = 1..4096); on the
    220 of them with J <= 8 and 74 others the rule's choice is 0.6-0.8 % (mean) behind the faster
    of the two, where the rule below stood 8-10 % behind -- it leaves out narrow and short
    outputs, which pad S and K (R=227, S=4, I=31, J=3, K=891: 65 -> 26 us; R=36, S=44, I=355,
    J=2, K=47: 54 -> 24).
    Longer rows: the padded work saved, of a kernel priced at 80 TFLOP/s, against w read and
    written at 2.5 TB/s plus 8 us, with a margin of 20 % (0.6-1.1 % behind the faster of the two
    on 278 shapes with J = 9..249, where the model above, which does not see what rows that are
    not 16-byte aligned cost on either side of the exchange, stood 1.4-7.5 % behind)."""
    if J <= 8:
        return _kernel_us(R, S, J, I, K) + 6.2 + 8.0 * R * S * I * J / 9.7e6 < _kernel_us(R, S, I, J, K)
    saved = 1.0 - (J * _padded(I)) / (I * _padded(J))
    kernel_s = 2.0 * R * S * I * _padded(J) * K / 80e12
    copy_s = 8.0 * R * S * I * J / 2.5e12 + 8e-6
    return saved * kernel_s >= 1.2 * copy_s


def _sweeps(R: int, S: int, I: int, J: int, K: int, w: torch.Tensor) -> bool:
    """Outputs of at most 8 columns whose w the library streams once on the vector ALU
    (csrc/lt2exp_smallk.hpp, same conditions as smallk_applies there): no front end below can
    make such a call cheaper, a copy of w costs more than the call."""
    if K > 8:
        return False
    kc = 1 if K <= 1 else 4 if K <= 4 else 8
    if ((I + (J + 3) // 4 * 4) * kc + 4 + 256 + 16) * 4 > 48 * 1024:
        return False
    sw = w.stride()
    if J % 4 == 0 and sw[2] == 1 and sw[0] % 4 == 0 and sw[1] % 4 == 0 and w.data_ptr() % 16 == 0:
        return I * J >= (256 if K > 4 else 128)
    return sw[2] == 1 and J > 4 and I * J >= (1024 if K > 4 else 256)


_IN_PLACE_KERNELS = ("trt::lt2exp_rows_kernel", "trt::lt2exp_cols_kernel")


def _rows_first(R: int, S: int, I: int, J: int, K: int, w: torch.Tensor) -> bool:
    """Would the library run this call on one of its kernels that read any w in place -- the one for
    few s per batch, the one for few units with a lane per column?  (Asked of the library itself,
    host side only: the rules are fitted ones and live there.)"""
    sw = w.stride()
    if sw[2] != 1:
        return False
    aligned = sw[0] % 4 == 0 and sw[1] % 4 == 0 and w.data_ptr() % 16 == 0
    return _lib.kernel_name("lt2exp", R, S, I, J, K, 0, 0, int(aligned)).startswith(_IN_PLACE_KERNELS)


def _packs(I: int, J: int) -> bool:
    """Rows of w short enough for the fp32 kernel to walk (i, j) as one flat axis (no padding of j)."""
    return J in (2, 4, 8) and (I * J) % 4 == 0 and I * J >= 32


def lt2exp(
    w: torch.Tensor, a: torch.Tensor, b: torch.Tensor, *, mode: str = "auto", _variant: int = 0,
    _precision: str | None = None, _tuning: bool = False, _pad: bool | None = None, _swap: bool | None = None,
) -> torch.Tensor:
    wsh, ash, bsh = w.shape, a.shape, b.shape
    assert len(wsh) == 4
    assert len(ash) == len(bsh) == 3
    assert wsh[0] == ash[0] == bsh[0]
    assert wsh[2] == ash[1]
    assert wsh[3] == bsh[1]
    assert ash[2] == bsh[2]
    assert w.dtype == a.dtype == b.dtype == torch.float32
    assert w.device == a.device == b.device
    R, S, I, J = wsh
    K = ash[2]
    mode_code = _MODES.get(mode)
    if mode_code is None:
        launches_split(R, S, I, J, K, mode)  # raises the reference's ValueError
    if not w.is_cuda:
        _lib.require_gpu(w, a, b)
    lib = _lib._lib or _lib.load()

    c = a.new_empty((R, S, K))
    # the reference flattens with w.view(batch, m, -1) (triturus/lt2exp.py:549); naming the
    # size keeps the same RuntimeError for non-viewable w and also accepts empty tensors
    w = w.view(R, S, I * J)
    if R * S * K == 0:
        return c
    if I * J == 0:
        return c.fill_(float("-inf"))
    # The kernels walk j in chunks of at least 16 and i one at a time: a short j axis under a
    # long i axis wastes most of every chunk.  The contraction is symmetric in (i, a) and (j, b),
    # so such a call runs with the roles exchanged on a transposed copy of w (J = 1 needs no
    # copy: the library does that exchange itself) when the padded work that saves is worth the
    # copy (_exchange_pays: fp32) / a third of the padded work on a wide enough output (bf16 paths).
    # Not for forced tiles (tests, tuning), nor where the fp32 kernel packs the short rows itself.
    # _swap: True / False force the exchange / its absence (tests, timing).
    if _precision is None:
        _precision = matrix_precision()
    elif _precision not in MATRIX_PRECISIONS:
        raise ValueError(f"unknown matrix precision {_precision!r}")
    fp32 = _precision == "fp32"
    if K <= 8 and _variant == 0 and _swap is None and _pad is None and _sweeps(R, S, I, J, K, w):
        _swap = _pad = False
    # (the shape tests come first: most calls meet none of them and pay for no rule)
    if _variant == 0 and 2 <= J < I and not (fp32 and _packs(I, J)):
        if _swap is not None:
            swap = _swap
        elif fp32:
            # (few s per batch: the library contracts j first, over the rows (s, i) of w as they lie
            # -- csrc/lt2exp_rows.hpp -- and wants no exchange; asked only where one would be made)
            swap = _exchange_pays(R, S, I, J, K) and not (K > 8 and _rows_first(R, S, I, J, K, w))
        else:
            swap = (K >= 256 and 2 * I * _padded(J) >= 3 * J * _padded(I)
                    and 2 * R * S * I * _padded(J) * K >= _RESHAPE_MIN_FLOPS)  # worth a copy kernel: some 40 us of work
        if swap:
            w = w.view(R, S, I, J).transpose(2, 3).contiguous().view(R, S, I * J)
            a, b = b, a
            I, J = J, I
    # Rows of w are read 16 bytes at a time only when J is a multiple of 4 (every (s, i) row then
    # starts aligned); otherwise the kernels stage w element by element, in j-chunks of 16 or 32
    # only.  The element loads themselves no longer cost what a padded copy of w and b does (timed
    # on 70 shapes with J = 9..237: the copies lose by 2-20 % on large calls and up to 2.5x on small
    # ones), but the chunks do where a chunk of 24 would fit and 32 has to serve: J = 17..23 runs
    # a third more MFMAs unpadded.  So a call with enough work runs on copies padded to the next
    # multiple of 4 (zeros in w, -inf rows in b: terms of weight 0, the result is the same) when
    # that shortens the padded contraction to 0.8 or less (R=64, S=34, I=199, J=17, K=3707:
    # 1493 -> 1195 us; R=32, S=452, I=97, J=21, K=2188: 1653 -> 1318).
    # _pad: True / False force the copies / their absence (tests, timing).
    # (the bf16 paths, whose unaligned builds stage pairs of columns, keep padding from that work on:
    # R=S=I=64, K=4096, J = 33 runs in ~300 us padded against 483 with two pieces)
    if _variant == 0 and J % 4 != 0 and J > 4:
        J4 = J + (-J) % 4
        pad = (K >= _PAD_MIN_K and 2 * R * S * I * _padded(J) * K >= _RESHAPE_MIN_FLOPS
               and (not fp32 or 5 * _padded(J4) <= 4 * _padded_by_element(J))) if _pad is None else _pad
        if pad and _pad is None and fp32 and K > 8 and _rows_first(R, S, I, J, K, w):
            pad = False  # (the same kernel reads rows of any length in place)
        if pad:
            w = torch.nn.functional.pad(w.view(R, S, I, J), (0, J4 - J)).view(R, S, I * J4)
            b = torch.nn.functional.pad(b, (0, 0, 0, J4 - J), value=float("-inf"))
            J = J4
    # Rows of 3, 5, 6 or 7 fill a fifth to a half of a j-chunk; padded to 4 or 8 the fp32 kernel
    # packs them (measured R=86 S=482 I=193 K=145: J = 3 574 -> 244 us, J = 5..7 576-594 -> 453-480;
    # at a tenth of that work the copies cost more than they save).
    if (_variant == 0 and fp32 and J in (3, 5, 6, 7) and I * (4 if J == 3 else 8) >= 32
            and (2 * R * S * I * 16 * K >= _PACK_PAD_MIN_FLOPS if _pad is None else _pad)
            and not (_pad is None and I <= 16 and K > 8 and _rows_first(R, S, I, J, K, w))):
        J4 = 4 if J == 3 else 8
        w = torch.nn.functional.pad(w.view(R, S, I, J), (0, J4 - J)).view(R, S, I * J4)
        b = torch.nn.functional.pad(b, (0, 0, 0, J4 - J), value=float("-inf"))
        J = J4
    sw, sa, sb = w.stride(), a.stride(), b.stride()
    # w is read in place whatever the stride of its flat (i, j) axis (a sliced view: element
    # loads instead of 16-byte ones); only negative strides need a copy
    if min(sw) < 0:
        w = _unit_inner(w)
        sw = w.stride()
    # a and b are read in place whatever their strides, as the reference forwards them
    # (triturus/lt2exp.py:606-620): a lane owns a column, so a trailing stride only scales its offsets
    if min(sa) < 0:
        a = a.contiguous()
        sa = a.stride()
    if min(sb) < 0:
        b = b.contiguous()
        sb = b.stride()
    if _variant == 0 and autotune.is_autotune_enabled() and not _tuning:
        cands = _FP32_CANDIDATES if _precision == "fp32" else _BF16_CANDIDATES
        _variant = autotune.pick(("lt2exp", R, S, I, J, K, mode, _precision), cands,
                                 lambda v: lt2exp(w.view(R, S, I, J), a, b, mode=mode, _variant=v,
                                                  _precision=_precision, _tuning=True))
    pieces = _PIECES.get(_precision, 0)
    key = (R, S, I, J, K, mode_code, pieces)
    ws_bytes = _ws_bytes.get(key)
    if ws_bytes is None:
        ws_bytes = lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, mode_code)
        if pieces:  # the bf16 entry may cut a small grid itself
            ws_bytes = max(ws_bytes, lib.trt_lt2exp_bf16_workspace_bytes(R, S, I, J, K, pieces, mode_code))
        _ws_bytes[key] = ws_bytes
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
        ws_ptr = ws.data_ptr()
    else:
        ws_ptr = None
    dev = a.device
    stride_array = _lib.stride_array
    with _lib.on_device(dev):
        if pieces == 0:
            status = lib.trt_lt2exp_f32(
                w.data_ptr(), a.data_ptr(), b.data_ptr(), c.data_ptr(), R, S, I, J, K,
                stride_array(sw), stride_array(sa), stride_array(sb), stride_array((S * K, K, 1)),
                mode_code, _variant, ws_ptr, ws_bytes, _lib.raw_stream(dev),
            )
        else:
            # bf16 matrix pipe; the library hands grids that are too small for it (those the
            # fp32 path would cut over the contraction) back to the fp32 kernels
            status = lib.trt_lt2exp_bf16(
                w.data_ptr(), a.data_ptr(), b.data_ptr(), c.data_ptr(), R, S, I, J, K,
                stride_array(sw), stride_array(sa), stride_array(sb), stride_array((S * K, K, 1)),
                pieces, mode_code, _variant, ws_ptr, ws_bytes, _lib.raw_stream(dev),
            )
    if status:
        _lib.check(status, "trt_lt2exp_f32" if pieces == 0 else "trt_lt2exp_bf16")
    return c
