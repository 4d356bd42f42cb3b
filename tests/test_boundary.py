"""The drop-in boundary, without a GPU: the C-ABI library loads and exports what
include/triturus_hip.h declares, argument errors are reported as statuses before
anything is enqueued, and the Python wrappers raise what the reference wrappers
raise (triturus/lm2exp.py:168-172, triturus/lt2exp.py:522-541,549,
triturus/max.py:97-99,177-180)."""

import ctypes
import re
from ctypes import c_void_p
from pathlib import Path

import pytest
import torch

from triturus_amd import _lib
from triturus_amd.lm2exp import lm2exp
from triturus_amd.lt2exp import launches_split, lt2exp
from triturus_amd.max import matmax, vamax, vmax
from triturus_amd.utils import ensure_reproducibility, is_triturus_tf32_enabled, set_tf32_enabled

ROOT = Path(__file__).resolve().parents[1]
HEADER = (ROOT / "include" / "triturus_hip.h").read_text()


def declared_functions():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(trt_[a-z0-9_]+)\s*\(", body)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert "trt_lm2exp_f32" in names and "trt_lt2exp_f32" in names and len(names) >= 10
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names:
        assert hasattr(raw, name), f"{name} declared in the header but not exported"
    # the ctypes table binds exactly the declared set
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.trt_version() == _lib.ABI_VERSION
    assert int(re.search(r"#define TRT_ABI_VERSION (\d+)", HEADER).group(1)) == _lib.ABI_VERSION
    assert lib.trt_error_string(0) == b"success"
    for code in (-1, -2, -3, -4):
        assert lib.trt_error_string(code) not in (b"success", b"unknown status")
    assert lib.trt_error_string(-99) == b"unknown status"


def test_header_constants_match_python():
    def const(name):
        return int(re.search(rf"#define {name} \(?(-?\d+)\)?", HEADER).group(1))

    assert (const("TRT_F32"), const("TRT_F64"), const("TRT_F16"), const("TRT_BF16")) == (0, 1, 2, 3)
    assert (const("TRT_MODE_AUTO"), const("TRT_MODE_SPLIT"), const("TRT_MODE_UNSPLIT")) == (
        _lib.MODE_AUTO, _lib.MODE_SPLIT, _lib.MODE_UNSPLIT)


def test_c_abi_argument_errors_are_statuses():
    lib = _lib.load()
    s3 = (ctypes.c_int64 * 3)
    ok = s3(12, 4, 1)
    one = c_void_p(16)  # never dereferenced: every call below is rejected first
    null = c_void_p(None)
    # lm2exp
    tail = (0, 0, null, 0, null)  # variant, splits, workspace, bytes, stream
    assert lib.trt_lm2exp_f32(null, one, one, 1, 1, 1, 1, ok, ok, ok, *tail) == -1
    assert lib.trt_lm2exp_f32(one, one, one, 0, 1, 1, 1, ok, ok, ok, *tail) == -1
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, ok, ok, ok, 99, 0, null, 0, null) == -1
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, ok, ok, ok, 0, -1, null, 0, null) == -1
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, ok, s3(12, 4, -1), ok, *tail) == -2  # b: any stride but a negative one
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, ok, ok, s3(12, 1, 4), *tail) == -2  # c: unit trailing stride
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, s3(12, 4, -1), ok, ok, *tail) == -2
    # a may have any non-negative strides, except under a forced tile that reads rows 16 bytes at a time
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, s3(12, 1, 4), ok, ok, 1, 0, null, 0, null) == -2
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1, 1, 1, ok, s3(-12, 4, 1), ok, *tail) == -2
    assert lib.trt_lm2exp_f32(one, one, one, 1 << 31, 1, 1, 1, ok, ok, ok, *tail) == -4
    assert lib.trt_lm2exp_f32(one, one, one, 1, 2, 2, 8, ok, ok, s3(16, 4, 1), *tail) == -2  # overlapping output rows
    assert lib.trt_lm2exp_f32(one, one, one, 1, 2, 2, 8, ok, s3(1 << 31, 1 << 30, 1), s3(16, 8, 1), *tail) == -4
    big = s3(1024 * 1024, 1024, 1)
    assert lib.trt_lm2exp_f32(one, one, one, 1, 1024, 1024, 1024, big, big, big, 0, 4, null, 0, null) == -3  # split needs a workspace
    # lt2exp
    args = (1, 1, 1, 1, 1, ok, ok, ok, ok)
    assert lib.trt_lt2exp_f32(one, null, one, one, *args, 0, 0, null, 0, null) == -1
    assert lib.trt_lt2exp_f32(one, one, one, one, *args, 7, 0, null, 0, null) == -1
    assert lib.trt_lt2exp_f32(one, one, one, one, 1, 1, 1, 1, 1, ok, ok, s3(1, 1, -2), ok, 0, 0, null, 0, null) == -2  # a, b: any stride but a negative one
    assert lib.trt_lt2exp_f32(one, one, one, one, 1, 1, 1, 1, 1, ok, s3(1, -1, 1), ok, ok, 0, 0, null, 0, null) == -2
    assert lib.trt_lt2exp_f32(one, one, one, one, 1, 1, 1, 1, 1, s3(1, 1, -1), ok, ok, ok, 0, 0, null, 0, null) == -2
    assert lib.trt_lt2exp_f32(one, one, one, one, 1, 1, 1, 1, 1, ok, ok, ok, s3(1, 1, 2), 0, 0, null, 0, null) == -2
    big4 = (64, 64, 16, 16, 4096, s3(16384, 256, 1), s3(65536, 4096, 1), s3(65536, 4096, 1), s3(262144, 4096, 1))
    assert lib.trt_lt2exp_f32(one, one, one, one, *big4, _lib.MODE_SPLIT, 0, null, 0, null) == -3  # split needs a workspace
    assert lib.trt_lt2exp_f32(one, one, one, one, *args, 0, lib.trt_lt2exp_variant_count() + 1, null, 0, null) == -1
    # short rows of w (J = 8) walked packed: a forced split still asks for its workspace
    packed = (64, 64, 256, 8, 64, s3(64 * 2048, 2048, 1), s3(256 * 64, 64, 1), s3(8 * 64, 64, 1), s3(64 * 64, 64, 1))
    assert lib.trt_lt2exp_workspace_bytes(64, 64, 256, 8, 64, _lib.MODE_SPLIT) > 0
    assert lib.trt_lt2exp_f32(one, one, one, one, *packed, _lib.MODE_SPLIT, 0, null, 0, null) == -3
    assert lib.trt_lt2exp_bf16(one, one, one, one, *packed, 3, _lib.MODE_SPLIT, 0, null, 0, null) == -3  # handed to fp32
    # lt2exp on the bf16 matrix pipe: pieces must be 2 or 3, variant 0..4
    btail = (0, 0, null, 0, null)  # mode, variant, workspace, bytes, stream
    assert lib.trt_lt2exp_bf16(one, one, one, one, *args, 4, *btail) == -1
    assert lib.trt_lt2exp_bf16(one, one, one, one, *args, 2, 0, 17, null, 0, null) == -1
    assert lib.trt_lt2exp_bf16(one, one, one, one, *args, 2, 5, 0, null, 0, null) == -1
    assert lib.trt_lt2exp_bf16(null, one, one, one, *args, 2, *btail) == -1
    assert lib.trt_lt2exp_bf16(one, one, one, one, 1, 1, 1, 1, 1, s3(1, 1, -2), ok, ok, ok, 2, *btail) == -2  # any stride but a negative one
    assert lib.trt_lt2exp_bf16(one, one, one, one, 1, 1, 1, 1, 1, ok, ok, ok, s3(1, 1, 2), 2, *btail) == -2  # c: unit trailing stride
    assert lib.trt_lt2exp_bf16(one, one, one, one, 1 << 31, 1, 1, 1, 1, ok, ok, ok, ok, 3, *btail) == -4
    # a grid the fp32 path would split is handed to it, and then needs its workspace
    assert lib.trt_lt2exp_bf16(one, one, one, one, *big4, 2, _lib.MODE_SPLIT, 0, null, 0, null) == -3
    # lm2exp on the bf16 matrix pipe
    mtail = (0, 0, null, 0, null)  # variant, splits, workspace, bytes, stream
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1, 1, 1, ok, ok, ok, 1, *mtail) == -1
    nv = lib.trt_lm2exp_bf16_variant_count()
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1, 1, 1, ok, ok, ok, 2, nv + 1, 0, null, 0, null) == -1
    assert lib.trt_lm2exp_bf16(one, null, one, 1, 1, 1, 1, ok, ok, ok, 3, *mtail) == -1
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1, 1, 1, ok, s3(4, 1, -2), ok, 2, *mtail) == -2  # b: any stride but a negative one
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1, 1, 1, s3(4, 1, -2), ok, ok, 2, *mtail) == -2
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1, 1, 1, ok, ok, s3(4, 1, 2), 2, *mtail) == -2  # c: unit trailing stride
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 2, 2, 8, ok, ok, s3(16, 4, 1), 2, *mtail) == -2
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1 << 30, 1, 1, ok, ok, ok, 2, *mtail) == -4
    assert lib.trt_lm2exp_bf16(one, one, one, 1, 1024, 1024, 1024, big, big, big, 2, 0, 4, null, 0, null) == -3
    # max
    assert lib.trt_vmax(null, 5, 0, one, one, one, 1 << 20, null) == -1
    assert lib.trt_vmax(one, 0, 0, one, one, one, 1 << 20, null) == -1
    assert lib.trt_vmax(one, 5, 9, one, one, one, 1 << 20, null) == -1
    assert lib.trt_vmax(one, 1 << 20, 0, one, one, null, 0, null) == -3
    assert lib.trt_matmax(one, one, 4, 4, 2, 0, null, 0, null) == -1
    assert lib.trt_matmax(one, one, 0, 4, 0, 0, null, 0, null) == -1
    # more workgroups than a 32-bit grid holds: refused, not truncated (2^34 rows along axis 1 are
    # 2^32 workgroups of 4 rows; 2^40 fp16 columns along axis 0 are 2^31 workgroups of 512 columns)
    assert lib.trt_matmax(one, one, 1 << 34, 1, 1, _lib.TRT_F16, null, 0, null) == -4
    assert lib.trt_matmax(one, one, 1 << 33, 2, 1, _lib.TRT_F16, null, 0, null) == -4
    assert lib.trt_matmax(one, one, 1, 1 << 40, 0, _lib.TRT_F16, null, 0, null) == -4
    assert lib.trt_copy_bytes(one, one, 24, null) == -1
    assert lib.trt_max_workspace_init(null, 1 << 20, null) == -3
    assert lib.trt_max_workspace_init(one, 1024, null) == -3  # smaller than the arrival counters
    # mm, vadd
    assert lib.trt_mm_f32(one, null, one, 2, 2, 2, 0, 0, null, 0, null) == -1
    assert lib.trt_mm_f32(one, one, one, 2, 0, 2, 0, 0, null, 0, null) == -1
    assert lib.trt_mm_f32(one, one, one, 2, 2, 2, 5, 0, null, 0, null) == -1
    assert lib.trt_mm_f32(one, one, one, 2, 2, 2, 0, -1, null, 0, null) == -1
    assert lib.trt_mm_f32(one, one, one, 1 << 30, 2, 2, 0, 0, null, 0, null) == -4
    # an explicit cut over k needs its workspace: 2 pieces of a 64 x 64 product
    assert lib.trt_mm_workspace_bytes(64, 64, 64, 0, 2) == 2 * 64 * 64 * 4
    assert lib.trt_mm_workspace_bytes(64, 64, 64, 0, 1) == 0
    assert lib.trt_mm_workspace_bytes(64, 32, 64, 0, 8) == 0  # one chunk of k: nothing to cut
    assert lib.trt_mm_f32(one, one, one, 64, 64, 64, 0, 2, null, 0, null) == -3
    assert lib.trt_mm_bf16(one, one, one, 2, 2, 2, 4, null, 0, null) == -1
    assert lib.trt_mm_bf16(null, one, one, 2, 2, 2, 2, null, 0, null) == -1
    assert lib.trt_mm_bf16(one, one, one, 2, 1 << 30, 2, 3, null, 0, null) == -4
    assert lib.trt_vadd(one, one, null, 5, 0, null) == -1
    assert lib.trt_vadd(one, one, one, 0, 0, null) == -1
    assert lib.trt_vadd(one, one, one, 5, 7, null) == -1
    # batched column maxima
    assert lib.trt_colmax_batched_f32(null, one, 1, 1, 1, ok, 0, null, 0, null) == -1
    assert lib.trt_colmax_batched_f32(one, one, 1, 0, 1, ok, 0, null, 0, null) == -1
    assert lib.trt_colmax_batched_f32(one, one, 1, 1, 1, s3(12, 1, 4), 1, null, 0, null) == -2
    assert lib.trt_colmax_batched_f32(one, one, 1 << 30, 1, 1, ok, 1, null, 0, null) == -4
    assert lib.trt_colmax_batched_f32(one, one, 1, 4096, 256, ok, 1, null, 0, null) == -3  # cut over J: needs workspace
    assert lib.trt_colmax_batched_workspace_bytes(64, 64, 4096) == 0
    assert lib.trt_colmax_batched_workspace_bytes(1, 4096, 256) == 64 * 256 * 4


def test_workspace_queries_are_host_only_and_follow_the_mode_rule():
    lib = _lib.load()
    assert lib.trt_vmax_workspace_bytes(1000, _lib.TRT_F32) == 0  # one workgroup, one launch
    assert lib.trt_vmax_workspace_bytes(1 << 20, _lib.TRT_F32) >= 2048 * 16
    assert lib.trt_vmax_workspace_bytes(1000, 9) == 0
    assert lib.trt_matmax_workspace_bytes(4096, 4096, 1, _lib.TRT_F32) == 0
    assert lib.trt_matmax_workspace_bytes(4096, 4096, 0, _lib.TRT_F32) > 0
    assert lib.trt_matmax_workspace_bytes(2, 1 << 24, 1, _lib.TRT_F32) > 0
    shapes = [(3, 75, 50, 50, 100), (16, 64, 32, 32, 2048), (64, 64, 64, 64, 4096), (1, 16, 16, 16, 16),
              (1, 1024, 32, 32, 1023), (1, 1024, 32, 32, 1024), (4, 8, 2, 256, 100), (4, 8, 23, 23, 100)]
    for R, S, I, J, K in shapes:
        assert lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, _lib.MODE_UNSPLIT) == 0
        assert lib.trt_lt2exp_workspace_bytes(R, S, I, J, K, _lib.MODE_SPLIT) >= 4 * (R * S * K + 2 * R * K)
    # "auto" is a performance decision with thresholds measured on MI355X (the results are
    # the same either way); at the reference's own test shape it splits, as the reference does
    assert lib.trt_lt2exp_workspace_bytes(3, 75, 50, 50, 100, _lib.MODE_AUTO) > 0
    # the large benchmark configurations fill the machine unsplit
    assert lib.trt_lt2exp_workspace_bytes(64, 64, 64, 64, 4096, _lib.MODE_AUTO) == 0
    # lm2exp: splits only for small grids with a long contraction, or on request
    assert lib.trt_lm2exp_workspace_bytes(64, 256, 256, 4096, 0, 0) == 0
    assert lib.trt_lm2exp_workspace_bytes(1, 128, 4096, 128, 0, 1) == 0
    assert lib.trt_lm2exp_workspace_bytes(1, 128, 4096, 128, 0, 0) > 0
    assert lib.trt_lm2exp_workspace_bytes(1, 128, 64, 128, 0, 0) == 0  # two chunks: nothing to share
    assert lib.trt_lm2exp_workspace_bytes(16, 512, 512, 512, 0, 0) == 0  # 256 tiles, 16 chunks: not worth a merge
    assert lib.trt_lm2exp_workspace_bytes(2, 100, 256, 50, 0, 4) == 4 * (4 * 2 * 100 * 50 + 4 * 2 * 50)
    # the bf16 entry's own cut: none on a full grid or when forbidden, sized by the split count
    assert lib.trt_lm2exp_bf16_workspace_bytes(64, 256, 256, 4096, 2, 0) == 0
    assert lib.trt_lm2exp_bf16_workspace_bytes(1, 128, 4096, 128, 2, 1) == 0
    assert lib.trt_lm2exp_bf16_workspace_bytes(1, 128, 4096, 128, 3, 0) > 0
    assert lib.trt_lm2exp_bf16_workspace_bytes(2, 100, 256, 50, 2, 4) == 4 * (4 * 2 * 100 * 50 + 4 * 2 * 50)
    assert lib.trt_lm2exp_bf16_workspace_bytes(2, 100, 20, 50, 2, 4) == 4 * (2 * 2 * 100 * 50 + 2 * 2 * 50)
    assert lib.trt_lm2exp_bf16_workspace_bytes(2, 100, 256, 50, 5, 4) == 0  # pieces must be 2 or 3
    # the reference rule itself, triturus/lt2exp.py:535: at the benchmark configurations it is unsplit
    assert not launches_split(16, 64, 32, 32, 2048, "auto")
    assert not launches_split(64, 64, 64, 64, 4096, "auto")
    assert launches_split(3, 75, 50, 50, 100, "auto")
    assert not launches_split(1, 1024, 32, 32, 1024, "auto")  # 2**20 is not < 2**20
    assert not launches_split(1, 16, 16, 32, 16, "auto")  # I*J = 512 is not > 512


def test_lm2exp_wrapper_validation():
    a, b = torch.rand(2, 3, 4), torch.rand(2, 4, 5)
    with pytest.raises(AssertionError):
        lm2exp(a[0], b)
    with pytest.raises(AssertionError):
        lm2exp(a, b[:1])
    with pytest.raises(AssertionError):
        lm2exp(a, torch.rand(2, 5, 5))
    with pytest.raises(AssertionError):
        lm2exp(a.double(), b)
    with pytest.raises(AssertionError):
        lm2exp(a, b.to("meta"))
    with pytest.raises(RuntimeError, match="GPU only"):
        lm2exp(a, b)


def test_lt2exp_wrapper_validation():
    w, a, b = torch.rand(2, 3, 4, 5), torch.rand(2, 4, 6), torch.rand(2, 5, 6)
    with pytest.raises(AssertionError):
        lt2exp(w[0], a, b)
    with pytest.raises(AssertionError):
        lt2exp(w, a[:1], b)
    with pytest.raises(AssertionError):
        lt2exp(w, b, a)  # I/J swapped
    with pytest.raises(AssertionError):
        lt2exp(w, a, torch.rand(2, 5, 7))
    with pytest.raises(AssertionError):
        lt2exp(w, a.half(), b)
    with pytest.raises(ValueError):
        lt2exp(w, a, b, mode="stream-k")
    with pytest.raises(RuntimeError, match="GPU only"):
        lt2exp(w, a, b, mode="split")


def test_max_wrapper_validation():
    x = torch.randn(10, 12)
    with pytest.raises(AssertionError):
        vmax(x)
    with pytest.raises(AssertionError):
        vamax(torch.arange(5))
    with pytest.raises(AssertionError):
        vmax(x[0, ::2])
    with pytest.raises(AssertionError):
        matmax(x[0])
    with pytest.raises(AssertionError):
        matmax(x.T)
    with pytest.raises(AssertionError):
        matmax(x, axis=2)
    with pytest.raises(RuntimeError, match="GPU only"):
        matmax(x, axis=1, block_size=2)
    with pytest.raises(RuntimeError, match="GPU only"):
        vmax(x[0], block_size=2)
    from triturus_amd.max import bmatmax
    with pytest.raises(AssertionError):
        bmatmax(x)
    with pytest.raises(AssertionError):
        bmatmax(torch.zeros(2, 3, 4, dtype=torch.float64))
    with pytest.raises(RuntimeError, match="GPU only"):
        bmatmax(torch.zeros(2, 3, 4))


def test_flags():
    set_tf32_enabled(True)
    assert is_triturus_tf32_enabled()
    set_tf32_enabled(False)
    assert not is_triturus_tf32_enabled()
    # the arithmetic follows the flag unless it is pinned explicitly
    from triturus_amd.utils import matrix_precision, set_matrix_precision
    assert matrix_precision() == "fp32"
    set_tf32_enabled(True)
    assert matrix_precision() == "bf16x3"
    set_matrix_precision("bf16x6")
    assert matrix_precision() == "bf16x6"
    set_tf32_enabled(False)
    assert matrix_precision() == "bf16x6"
    set_matrix_precision(None)
    assert matrix_precision() == "fp32"
    with pytest.raises(ValueError):
        set_matrix_precision("tf32")
    ensure_reproducibility(seed=7, device="cpu")
    x = torch.rand(3)
    ensure_reproducibility(seed=7, device="cpu")
    assert torch.equal(x, torch.rand(3))


def test_flags_write_the_torch_settings_the_reference_writes():
    """triturus/utils.py:26-30,33-48: the flag functions also set torch's own matmul precision,
    its two allow_tf32 backends, and (with determinism) cudnn benchmarking, the BLAS workspace
    variable and the dynamo recompile limit."""
    import os

    from triturus.utils import is_torch_tf32_enabled as shim_fn
    from triturus_amd.utils import is_torch_tf32_enabled

    assert shim_fn is is_torch_tf32_enabled
    before = (torch.get_float32_matmul_precision(), torch.backends.cuda.matmul.allow_tf32,
              torch.backends.cudnn.allow_tf32, torch.backends.cudnn.benchmark,
              torch.are_deterministic_algorithms_enabled(), torch.is_deterministic_algorithms_warn_only_enabled(),
              os.environ.get("CUBLAS_WORKSPACE_CONFIG"))
    try:
        set_tf32_enabled(True)
        assert torch.get_float32_matmul_precision() == "high"
        assert torch.backends.cuda.matmul.allow_tf32 is True and torch.backends.cudnn.allow_tf32 is True
        assert is_torch_tf32_enabled() is True and is_triturus_tf32_enabled()
        set_tf32_enabled(False)
        assert torch.get_float32_matmul_precision() == "highest"
        assert torch.backends.cuda.matmul.allow_tf32 is False and torch.backends.cudnn.allow_tf32 is False
        assert is_torch_tf32_enabled() is False and not is_triturus_tf32_enabled()
        torch.backends.cudnn.benchmark = True
        ensure_reproducibility(seed=3, determinism=True, device="cpu")
        assert torch.are_deterministic_algorithms_enabled()
        assert torch.backends.cudnn.benchmark is False
        assert os.environ["CUBLAS_WORKSPACE_CONFIG"] == ":16:8"
        assert torch._dynamo.config.recompile_limit == 64
    finally:
        torch.set_float32_matmul_precision(before[0])
        torch.backends.cuda.matmul.allow_tf32 = before[1]
        torch.backends.cudnn.allow_tf32 = before[2]
        torch.backends.cudnn.benchmark = before[3]
        torch.use_deterministic_algorithms(before[4], warn_only=before[5])
        if before[6] is None:
            os.environ.pop("CUBLAS_WORKSPACE_CONFIG", None)
        else:
            os.environ["CUBLAS_WORKSPACE_CONFIG"] = before[6]
        set_tf32_enabled(False)


def test_tile_tuning_is_off_by_default():
    from triturus_amd import autotune

    assert not autotune.is_autotune_enabled()
    calls = []
    assert autotune.pick(("k",), (0, 1, 2), calls.append) == 0
    assert calls == [] and autotune.chosen() == {}


def test_reference_import_paths_exist():
    from triturus.lm2exp import lm2exp as f1
    from triturus.lt2exp import lt2exp as f2
    from triturus.max import matmax as f3, vamax as f4, vmax as f5
    from triturus.utils import ensure_reproducibility as f6, set_tf32_enabled as f7
    from triturus.mm import mm as f8
    from triturus.add import vadd as f9

    assert f1 is lm2exp and f2 is lt2exp and (f3, f4, f5) == (matmax, vamax, vmax)
    assert callable(f6) and callable(f7)
    import triturus

    assert not hasattr(triturus, "__all__")  # the reference's __init__ is empty


def test_product_never_imports_the_oracle():
    for pkg in ("triturus_amd", "triturus"):
        for f in (ROOT / pkg).rglob("*"):
            if f.suffix in {".py", ".hip", ".hpp", ".h"}:
                text = f.read_text()
                assert "oracle" not in text.replace("the oracle the reference tests use", ""), f


def test_short_row_rule_of_the_lt2exp_wrapper():
    """Rows of w that the fp32 kernel packs: 2, 4 or 8 values, a whole number of 16-byte pieces in
    all, more than one chunk of 16."""
    from triturus_amd.lt2exp import _packs

    assert _packs(193, 8) and _packs(64, 4) and _packs(50, 2)
    assert not _packs(3, 2)        # 6 floats: not a multiple of 4
    assert not _packs(2, 8)        # a single chunk
    assert not _packs(64, 16) and not _packs(64, 3) and not _packs(64, 1)


def test_small_lm2exp_grids_get_tile_and_cut_chosen_together():
    """Host-side plan of lm2exp (no GPU needed: trt_lm2exp_kernel_name reports the tile,
    trt_lm2exp_workspace_bytes the cut: splits * (R*I*K partial sums + R*K shifts) floats)."""
    lib = _lib.load()
    name = lambda R, I, J, K: _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1)
    cut = lambda R, I, J, K: lib.trt_lm2exp_workspace_bytes(R, I, J, K, 0, 0) // (4 * (R * I * K + R * K))
    # a batch-1 square of 1536: 96-row tiles cut four ways are 768 workgroups, three per CU
    assert name(1, 1536, 1536, 1536) == "trt::lm2exp_kernel<3, 1, 1, 4, 4, true, 1>" and cut(1, 1536, 1536, 1536) == 4
    assert name(2, 1536, 1536, 1536) == "trt::lm2exp_kernel<3, 1, 1, 4, 4, true, 1>" and cut(2, 1536, 1536, 1536) == 2
    # 256 tiles of 64 rows under 16 chunks: one workgroup per tile (a cut would cost more than it hides)
    assert name(16, 512, 512, 512) == "trt::lm2exp_kernel<2, 1, 1, 4, 4, true, 1>" and cut(16, 512, 512, 512) == 0
    # a forced cut keeps its count; the tile follows it
    assert lib.trt_lm2exp_workspace_bytes(1, 1536, 1536, 1536, 0, 3) == 3 * 4 * (1536 * 1536 + 1536)
    # outside the region (a short contraction, a large grid, a contraction that wants chunks of 16)
    # the tile rules decide as before
    assert name(64, 256, 256, 4096) == "trt::lm2exp_pair_kernel<4, 4, 2, 0>"
    assert name(6, 325, 464, 1266) == "trt::lm2exp_kernel<3, 1, 1, 4, 2, true, 1>"
    assert cut(1, 128, 64, 128) == 0


def test_lm2exp_takes_64_column_pair_tiles_where_128_column_tiles_would_stand_partly_empty():
    """Host-side tile rule of lm2exp on large grids (lm2exp_pair_kernel<rows / 64, wavefront
    columns, ...>: two wavefront columns are a 64-column tile)."""
    name = lambda R, I, J, K: _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1)
    assert name(384, 2039, 420, 180) == "trt::lm2exp_pair_kernel<2, 2, 2, 0>"   # 128 rows pad 2039 less than 192
    assert name(64, 2085, 772, 268) == "trt::lm2exp_pair_kernel<3, 2, 2, 0>"
    assert name(16, 1755, 268, 652) == "trt::lm2exp_pair_kernel<2, 2, 2, 0>"    # 0.92 of the columns, long and tall
    assert name(64, 256, 256, 4096) == "trt::lm2exp_pair_kernel<4, 4, 2, 0>"    # whole 128-column tiles
    assert name(32, 2496, 112, 276).startswith("trt::lm2exp_kernel<")           # a short contraction
    assert name(384, 654, 96, 564).startswith("trt::lm2exp_kernel<")            # 0.9 of the columns, short
    # rows of a that are not 16-byte aligned take the same tiles (last argument: how a is loaded)
    assert _lib.kernel_name("lm2exp", 384, 2039, 421, 180, 0, 0, 0) == "trt::lm2exp_pair_kernel<2, 2, 2, 1>"
    # smaller grids whose K leaves a quarter of the 128-column tiling empty: 64 x 64 tiles from 100 on
    assert name(6, 1159, 2880, 159) == "trt::lm2exp_pair_kernel<1, 2, 2, 0>"
    assert _lib.kernel_name("lm2exp", 3, 2878, 587, 158, 0, 0, 0) == "trt::lm2exp_pair_kernel<1, 2, 2, 1>"
    assert name(3, 2878, 100, 158).startswith("trt::lm2exp_kernel<")            # a short contraction
    assert name(1, 1159, 2880, 159).startswith("trt::lm2exp_kernel<")           # 57 tiles
    assert name(6, 1159, 2880, 300).startswith("trt::lm2exp_kernel<")           # 320 of 384 columns


def test_lm2exp_outputs_of_at_most_64_columns_take_the_narrow_tiles():
    """Host-side tile rule of lm2exp for K <= 64 (lm2exp_kernel<rows / 32, column blocks, wavefronts
    over rows, wavefronts over columns, ...>): the wavefronts are stacked over rows whatever the
    number of tiles; large grids of 33..64 columns take the paired kernel's 128 x 64 tile."""
    name = lambda R, I, J, K: _lib.kernel_name("lm2exp", R, I, J, K, 0, 0, 1)
    assert name(30, 283, 2788, 10) == "trt::lm2exp_kernel<1, 1, 4, 1, 4, true, 1>"    # 128 x 32, 90 tiles
    assert name(10, 162, 1324, 39) == "trt::lm2exp_kernel<1, 1, 2, 2, 4, true, 1>"    # 64 x 64, 30 tiles
    assert name(101, 1510, 48, 48) == "trt::lm2exp_pair_kernel<2, 2, 2, 0>"           # 2424 tiles of 64 rows
    assert name(14, 2464, 2688, 48) == "trt::lm2exp_pair_kernel<2, 2, 2, 0>"          # 546, a long contraction
    assert name(203, 267, 2788, 63) == "trt::lm2exp_kernel<1, 1, 2, 2, 4, true, 1>"   # 128 rows would pad 267 to 384
    # I <= 32: the 32 x 128 tile (here with rows of a that are not 16-byte aligned; aligned ones: the next test)
    assert _lib.kernel_name("lm2exp", 40, 30, 500, 20, 0, 0, 0) == "trt::lm2exp_kernel<1, 1, 1, 4, 4, false, 1>"


def test_paired_wavefront_groups_take_grids_of_at_most_two_tiles_per_cu():
    """Host-side tile rule of lt2exp (no GPU needed: trt_lt2exp_kernel_name reports what a call
    would launch).  The last template argument is the number of wavefront groups that share a
    tile's contraction inside a workgroup."""
    name = lambda *sh, mode=_lib.MODE_AUTO, aligned=1: _lib.kernel_name("lt2exp", *sh, mode, 0, aligned)
    # R=16, S=64, I=J=32, K=2048: 256 tiles of 64 rows, a short contraction: 64 rows, two groups
    assert name(16, 64, 32, 32, 2048) == "trt::lt2exp_kernel<2, 1, 4, 4, true, false, 1, 0, 2>"
    # one 32-row tile per CU, or a long contraction: 32 rows, two groups
    assert name(16, 32, 32, 32, 2048) == "trt::lt2exp_kernel<1, 1, 4, 4, true, false, 1, 0, 2>"
    assert name(16, 64, 64, 64, 2048).endswith("4, 4, true, false, 1, 0, 2>")
    # the large configuration fills the machine many times over: one group per tile
    assert name(64, 64, 64, 64, 4096) == "trt::lt2exp_kernel<2, 1, 8, 4, true, false, 1, 0, 1>"  # (j-chunks of 64)
    # never under a forced cut over workgroups, for rows of w that are not 16-byte aligned, or
    # where another j-chunk than 32 fits J better
    assert name(16, 64, 32, 32, 2048, mode=_lib.MODE_SPLIT).endswith("true, true, 1, 0, 1>")
    assert name(16, 64, 32, 32, 2048, aligned=0).endswith("false, false, 1, 0, 1>")
    assert name(16, 64, 32, 16, 2048).endswith(", 1>") and ", 2, 4, " in name(16, 64, 32, 16, 2048)


def test_lt2exp_takes_64_column_tiles_where_128_column_tiles_would_stand_half_empty():
    """Host-side tile rule (seventh template argument: wavefronts stacked over rows; 2 is the
    64 x 64 tile).  K = 192 is three tiles of 64 columns or two of 128."""
    name = lambda *sh, aligned=1: _lib.kernel_name("lt2exp", *sh, _lib.MODE_AUTO, 0, aligned)
    wm = lambda n: int(n.split(", ")[6])
    assert wm(name(1, 192, 192, 192, 192)) == 2      # one of the reference's benchmark shapes
    assert wm(name(4, 535, 26, 64, 136)) == 2
    assert wm(name(1, 192, 192, 192, 256)) == 1      # whole 128-column tiles
    assert wm(name(1, 192, 192, 192, 448)) == 1      # 7 tiles of 64 against 4 of 128: 0.875 of the area
    assert wm(name(4, 535, 26, 64, 136, aligned=0)) == 1 and wm(name(4, 535, 26, 24, 136)) == 1  # aligned rows, chunks of 32 only
    assert name(16, 382, 10, 32, 184).endswith(", 2>")  # paired groups keep their grids


def test_lt2exp_cuts_64_row_tiles_where_the_contraction_is_cut_anyway():
    """Host-side tile rule (first template argument: rows of S in units of 32; sixth: the
    contraction is cut over workgroups)."""
    name = lambda *sh, mode=_lib.MODE_AUTO: _lib.kernel_name("lt2exp", *sh, mode, 0, 1)
    # R=32, S=I=J=64, K=256 (one of the reference's benchmark shapes): 64 tiles of 64 rows, cut
    assert name(32, 64, 64, 64, 256) == "trt::lt2exp_kernel<2, 1, 4, 4, true, true, 1, 0, 1>"
    assert name(4, 170, 90, 128, 245).startswith("trt::lt2exp_kernel<2, 1, 4, 4, true, true")
    # fewer than twelve 64-row tiles, rows that 64 pads further than 32, or no cut: 32 rows
    assert name(1, 128, 128, 128, 512).startswith("trt::lt2exp_kernel<1, 1, 4, 4, true, true")
    assert name(32, 82, 131, 64, 184).startswith("trt::lt2exp_kernel<1, 1, 4, 4, true, true")
    assert name(32, 64, 64, 64, 256, mode=_lib.MODE_UNSPLIT).startswith("trt::lt2exp_kernel<1, 1, 4, 4, true, false")


def test_lt2exp_few_s_per_batch_contract_j_first():
    """Host-side rule of lt2exp for few s per batch: lt2exp_rows_kernel<column blocks of 32 that a
    wavefront contracts at once, groups of them in the workgroup's tile, 16-byte loads of w> puts the
    rows (s, i) of w on the rows of the MFMA where padding s to 32 costs more than padding i to 32,
    K is moderate and J is not too short.  Never for forced tiles or at most 8 columns (the sweep's)."""
    name = lambda *sh, variant=0, aligned=1: _lib.kernel_name("lt2exp", *sh, 0, variant, aligned)
    assert name(2048, 1, 64, 64, 64) == "trt::lt2exp_rows_kernel<1, 2, true>"      # two tiles: their column blocks on four wavefronts
    assert name(2048, 1, 64, 64, 12) == "trt::lt2exp_rows_kernel<1, 1, true>"
    assert name(4096, 1, 32, 32, 100) == "trt::lt2exp_rows_kernel<1, 4, true>"     # one tile of four column blocks
    assert name(5, 3, 33, 20, 70) == "trt::lt2exp_rows_kernel<4, 1, true>"
    assert name(1520, 1, 245, 256, 256) == "trt::lt2exp_rows_kernel<1, 1, true>"      # the factors of 32 columns fill LDS
    assert name(64, 4, 128, 128, 4096) == "trt::lt2exp_rows_kernel<1, 1, true>"       # S = 4: 8 times the padding
    assert name(64, 64, 64, 64, 4096).startswith("trt::lt2exp_kernel<")      # the large configuration: s-row tiles
    assert name(64, 16, 64, 64, 4096).startswith("trt::lt2exp_kernel<")
    # from 13 values of s on: calls of less than about a GFLOP, whatever S is
    assert name(1, 128, 128, 128, 128) == "trt::lt2exp_rows_kernel<1, 1, true>"
    assert name(16, 128, 128, 128, 128).startswith("trt::lt2exp_kernel<")
    assert name(16, 192, 192, 192, 192).startswith("trt::lt2exp_kernel<")
    assert name(6755, 9, 5, 20, 783).startswith("trt::lt2exp_kernel<")       # I = 5 would pad to 32
    assert name(2048, 1, 64, 64, 8).startswith("trt::lt2exp_smallk_kernel<")
    assert name(2048, 1, 64, 64, 64, variant=3).startswith("trt::lt2exp_kernel<")
    # rows of w that cannot be read 16 bytes at a time: the same kernel, loading float by float
    assert name(2048, 1, 64, 64, 64, aligned=0) == "trt::lt2exp_rows_kernel<1, 2, false>"
    assert name(2048, 1, 64, 66, 64) == "trt::lt2exp_rows_kernel<1, 2, false>"  # J not a multiple of 4
    assert name(4, 1, 5000, 5000, 64).startswith("trt::lt2exp_kernel<")      # the factors do not fit LDS


def test_lt2exp_few_units_over_many_batches_take_a_lane_per_column():
    """Host-side rule of lt2exp for I and J of at most 16: lt2exp_cols_kernel<I and J padded to 4, 8
    or 16, exact sizes on a dense w> where a lane's S I J FMAs stay few enough and the call is large
    enough.  Never for forced tiles or at most 8 columns."""
    name = lambda *sh, variant=0: _lib.kernel_name("lt2exp", *sh, 0, variant, 1)
    assert name(8192, 8, 8, 8, 256) == "trt::lt2exp_cols_kernel<8, 8, true>"
    assert name(8192, 4, 4, 4, 64) == "trt::lt2exp_cols_kernel<4, 4, true>"
    assert name(4096, 4, 16, 16, 256) == "trt::lt2exp_cols_kernel<16, 16, true>"
    assert name(1500, 3, 5, 7, 64) == "trt::lt2exp_cols_kernel<8, 8, false>"
    assert name(2500, 7, 16, 1, 90) == "trt::lt2exp_cols_kernel<1, 16, true>"      # J = 1: i and j exchanged first
    assert name(8192, 16, 16, 16, 256).startswith("trt::lt2exp_kernel<")            # 4096 FMAs per lane: the MFMA tiles
    assert name(16, 8, 8, 8, 64).startswith("trt::lt2exp_kernel<")                  # a call of a few microseconds either way
    assert name(8192, 8, 8, 17, 256).startswith("trt::lt2exp_kernel<")              # J beyond 16
    assert name(8192, 8, 8, 8, 8).startswith("trt::lt2exp_rows_kernel<")            # 8 columns: not asked
    assert name(8192, 8, 8, 8, 256, variant=3).startswith("trt::lt2exp_kernel<")


def test_lm2exp_contractions_of_at_most_16_terms_take_a_lane_per_column():
    """Host-side rule of lm2exp for J <= 16 over many batches: the lane-per-column kernel of lt2exp
    (lt2exp_cols_kernel<1, J padded to 4, 8 or 16, rows of exactly that many dense values>)."""
    name = lambda *sh, variant=0, splits=0: _lib.kernel_name("lm2exp", *sh, variant, splits, 1)
    assert name(8192, 4, 4, 1024) == "trt::lt2exp_cols_kernel<1, 4, true>"
    assert name(8192, 8, 8, 1024) == "trt::lt2exp_cols_kernel<1, 8, true>"
    assert name(4096, 64, 8, 256) == "trt::lt2exp_cols_kernel<1, 8, true>"
    assert name(3000, 5, 7, 100) == "trt::lt2exp_cols_kernel<1, 8, false>"
    assert name(64, 8, 8, 64).startswith("trt::lm2exp_kernel<")            # a call of a few microseconds either way
    assert name(8192, 8, 17, 1024).startswith("trt::lm2exp_kernel<")       # J beyond 16
    assert name(8192, 8, 8, 8).startswith("trt::lm2exp_kernel<")           # 8 columns: not asked
    assert name(8192, 8, 8, 1024, variant=3).startswith("trt::lm2exp")     # forced tiles
    assert name(8192, 8, 8, 1024, splits=2).startswith("trt::lm2exp")      # a forced cut


def test_lm2exp_narrow_outputs_of_few_rows_cut_the_contraction_over_the_wavefronts():
    """Host-side rule of lm2exp for at most 64 columns under few rows per batch: lm2exp_jsplit_kernel<column
    blocks of 32> gives a workgroup one tile and each wavefront a quarter of J."""
    name = lambda *sh, variant=0, splits=0, aligned=1: _lib.kernel_name("lm2exp", *sh, variant, splits, aligned)
    assert name(8192, 20, 256, 16) == "trt::lm2exp_jsplit_kernel<1>"
    assert name(2000, 40, 128, 48) == "trt::lm2exp_jsplit_kernel<2>"
    assert name(40, 30, 500, 20) == "trt::lm2exp_jsplit_kernel<1>"
    assert name(508, 16, 256, 256).startswith("trt::lm2exp_kernel<")        # more than 64 columns
    assert name(4000, 24, 66, 20).startswith("trt::lm2exp_kernel<")         # J not a multiple of 4
    assert name(8192, 20, 256, 16, aligned=0).startswith("trt::lm2exp_kernel<")
    # at most 16 rows and 32 columns: the 16 x 16 x 4 MFMA's tile, <column blocks of 16>, any J and layout of a
    # (second argument: the units of 4 values of j that a wavefront keeps in registers between the maxima
    # and the exponentials, 0 where its quarter of J is longer than 32 units)
    assert name(8192, 1, 256, 16) == "trt::lm2exp_jsplit16_kernel<1, 16, false>"
    assert name(4000, 8, 66, 20) == "trt::lm2exp_jsplit16_kernel<2, 6, false>"
    assert name(8192, 1, 255, 16, aligned=0) == "trt::lm2exp_jsplit16_kernel<1, 16, false>"
    assert name(8192, 1, 32, 16) == "trt::lm2exp_jsplit16_kernel<1, 2, false>"
    assert name(4000, 8, 512, 32) == "trt::lm2exp_jsplit16_kernel<2, 32, false>"
    assert name(4000, 8, 513, 32) == "trt::lm2exp_jsplit16_kernel<2, 0, false>"
    # (third argument: from 12 rows on, dense aligned rows of a and whole groups of four units are read
    # 16 bytes at a time and transposed among the four lanes of a row)
    assert name(4438, 16, 256, 16) == "trt::lm2exp_jsplit16_kernel<1, 16, true>"
    assert name(4438, 16, 256, 16, aligned=0) == "trt::lm2exp_jsplit16_kernel<1, 16, false>"
    assert name(4000, 12, 512, 32) == "trt::lm2exp_jsplit16_kernel<2, 32, true>"
    assert name(4000, 12, 96, 32) == "trt::lm2exp_jsplit16_kernel<2, 6, false>"
    assert name(4000, 11, 512, 32) == "trt::lm2exp_jsplit16_kernel<2, 32, false>"
    assert name(8, 2, 3848, 24).startswith("trt::lm2exp_kernel<")           # a few batches under a long contraction: tiles cut over J
    assert name(30, 283, 2788, 10).startswith("trt::lm2exp_kernel<")        # nine row tiles per batch on a small grid
    assert name(8192, 1, 256, 16, variant=3).startswith("trt::lm2exp")      # forced tiles
    assert name(8192, 1, 256, 16, splits=2).startswith("trt::lm2exp_")      # a forced cut over workgroups
    assert "jsplit" not in name(8192, 1, 256, 16, splits=2)
    assert name(8192, 8, 8, 16).startswith("trt::lt2exp_cols_kernel<")      # short contractions: a lane per column
