"""The C-ABI library loads without a GPU and exports every function the header declares."""
import ctypes
import os
import re

from tritonbench_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355x_fp8_rowwise.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355x_fp8_[a-z]\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    assert _declared_functions() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.library_path())
    for name in _declared_functions():
        assert hasattr(lib, name), name


def test_abi_version_and_status_constants_match_header():
    text = open(HEADER).read()
    consts = dict(re.findall(r"#define\s+(MI355X_FP8_\w+)\s+\(?(-?\d+)\)?", text))
    assert int(consts["MI355X_FP8_ABI_VERSION"]) == _lib.ABI_VERSION == _lib.load().mi355x_fp8_rowwise_abi_version()
    assert int(consts["MI355X_FP8_EINVAL"]) == _lib.EINVAL
    assert int(consts["MI355X_FP8_ENOTSUP"]) == _lib.ENOTSUP
    assert int(consts["MI355X_FP8_ELAUNCH"]) == _lib.ELAUNCH
    assert int(consts["MI355X_FP8_VARIANT_TILED"]) == _lib.VARIANT_TILED
    assert int(consts["MI355X_FP8_VARIANT_SKINNY"]) == _lib.VARIANT_SKINNY
    assert int(consts["MI355X_FP8_VARIANT_GENERIC"]) == _lib.VARIANT_GENERIC
    assert int(consts["MI355X_FP8_SRC_BF16"]) == _lib.SRC_BF16


def test_host_side_argument_checks_need_no_gpu():
    lib = _lib.load()
    # shape checks happen before anything touches a device
    assert lib.mi355x_fp8_rowwise_select_variant(16, 8192, 8192) == _lib.VARIANT_SKINNY
    assert lib.mi355x_fp8_rowwise_select_variant(8192, 8192, 8192) == _lib.VARIANT_TILED
    assert lib.mi355x_fp8_rowwise_select_variant(32, 2048, 2048) == _lib.VARIANT_SKINNY
    assert lib.mi355x_fp8_rowwise_select_variant(64, 8192, 8192) == _lib.VARIANT_SKINNY  # (its narrow-tile form)
    assert lib.mi355x_fp8_rowwise_select_variant(64, 28672, 8192) == _lib.VARIANT_TILED
    # (65 .. 256 rows: the narrow-tile form in row blocks where it fits the chip in one round)
    assert lib.mi355x_fp8_rowwise_select_variant(128, 8192, 8192) == _lib.VARIANT_SKINNY
    assert lib.mi355x_fp8_rowwise_select_variant(128, 10240, 8192) == _lib.VARIANT_TILED
    assert lib.mi355x_fp8_rowwise_workspace_bytes(128, 8192, 8192, _lib.VARIANT_AUTO) == 0
    # the Python mirror of the family's shape rule agrees with the library's choice being possible at all
    for m, n in ((64, 99999), (65, 16320), (65, 16384), (128, 8192), (128, 8200), (256, 4096), (256, 4160), (257, 64)):
        if not _lib.skinny_family_takes(m, n):
            assert lib.mi355x_fp8_rowwise_select_variant(m, n, 1024) == _lib.VARIANT_TILED
    assert lib.mi355x_fp8_rowwise_select_variant(64, 57344, 8192) == _lib.VARIANT_TILED
    # up to 8 rows the streaming family keeps the shape unless split tiles are expected a tenth ahead
    # (few columns, very long rows: a handful of workgroups each streaming a long tile)
    assert lib.mi355x_fp8_rowwise_select_variant(8, 8192, 8192) == _lib.VARIANT_SKINNY
    assert lib.mi355x_fp8_rowwise_select_variant(1, 2048, 28672) == _lib.VARIANT_SKINNY
    assert lib.mi355x_fp8_rowwise_select_variant(8, 1024, 28672) == _lib.VARIANT_TILED
    assert lib.mi355x_fp8_rowwise_select_variant(0, 8, 16) == _lib.EINVAL
    assert lib.mi355x_fp8_rowwise_select_variant(8, 8, 24) == _lib.VARIANT_GENERIC  # K not a multiple of 16
    assert lib.mi355x_fp8_rowwise_workspace_bytes(128, 8192, 8200, _lib.VARIANT_AUTO) == 0
    assert lib.mi355x_fp8_rowwise_select_variant(2 ** 31, 8, 16) == _lib.ENOTSUP
    assert "2^31" in _lib.last_error()
    st = lib.mi355x_fp8_rowwise_gemm(None, None, None, None, None, None, 16, 16, 16, 16, 16, 16, None, 0, 0, None)
    assert st == _lib.EINVAL and "null" in _lib.last_error()
    st = lib.mi355x_fp8_rowwise_gemm(None, None, None, None, None, None, 16, 16, 20, 32, 32, 16, None, 0, 0, None)
    assert st == _lib.EINVAL  # (null pointers; K = 20 alone is the generic family's business)


def test_status_to_exception_mapping():
    import pytest

    lib = _lib.load()
    with pytest.raises(NotImplementedError):
        _lib.check(lib.mi355x_fp8_rowwise_select_variant(8, 2 ** 31, 16), "select")
    with pytest.raises(ValueError):
        _lib.check(lib.mi355x_fp8_rowwise_select_variant(-1, 8, 16), "select")
    _lib.check(0, "fine")


def test_workspace_size_follows_the_plan_without_a_gpu():
    lib = _lib.load()
    ws = lib.mi355x_fp8_rowwise_workspace_bytes
    text = open(HEADER).read()
    assert int(re.search(r"#define\s+MI355X_FP8_NUM_TILE_CONFIGS\s+(\d+)", text).group(1)) == _lib.NUM_TILE_CONFIGS
    assert int(re.search(r"#define\s+MI355X_FP8_NUM_GROUPED_TILE_CONFIGS\s+(\d+)", text).group(1)) == _lib.NUM_GROUPED_TILE_CONFIGS
    # enough tiles to fill the chip, or the on-chip reduction of the skinny kernel: no workspace
    assert ws(8192, 8192, 8192, _lib.VARIANT_AUTO) == 0
    assert ws(16, 8192, 8192, _lib.VARIANT_AUTO) == 0
    assert ws(16, 8192, 8192, _lib.VARIANT_SKINNY) == 0
    # few tiles and a long K: split, S * M * N fp32 partial sums
    auto = ws(128, 10240, 8192, _lib.VARIANT_AUTO)
    assert auto > 0 and auto % (128 * 10240 * 4) == 0
    # a pinned split factor is honoured, clipped to the number of 128-byte K steps
    assert ws(256, 256, 1024, _lib.tiled_variant(0, 4)) == 4 * 256 * 256 * 4
    assert ws(256, 256, 1024, _lib.tiled_variant(1, 1)) == 0
    assert ws(256, 256, 256, _lib.tiled_variant(0, 16)) == 2 * 256 * 256 * 4
    assert ws(256, 256, 128, _lib.tiled_variant(0, 16)) == 0
    # 9 steps in 4 parts of 3: only 3 parts are non-empty
    assert ws(256, 256, 9 * 128, _lib.tiled_variant(0, 4)) == 3 * 256 * 256 * 4
    # unsupported shapes need nothing (the GEMM call itself reports the error)
    assert ws(8, 8, 24, _lib.VARIANT_AUTO) == 0


def test_grouped_and_blockwise_argument_checks_need_no_gpu():
    lib = _lib.load()
    grouped = lib.mi355x_fp8_rowwise_grouped_gemm
    blockwise = lib.mi355x_fp8_blockwise_gemm
    # shape and range checks come before anything touches a pointer or a device
    assert grouped(None, None, None, None, None, None, 0, 64, 64, 64, 64, 64, 64, -1, None) == _lib.EINVAL
    assert "G must be" in _lib.last_error()
    assert grouped(None, None, None, None, None, None, 2, 64, 64, 24, 32, 32, 64, -1, None) == _lib.ENOTSUP
    assert grouped(None, None, None, None, None, None, 2, 64, 64, 64, 64, 64, 64, -1, None) == _lib.EINVAL
    assert "null" in _lib.last_error()
    assert blockwise(None, None, None, None, None, 64, 64, 32768 + 128, 40000, 40000, 64, None) == _lib.ENOTSUP
    assert "K <=" in _lib.last_error()
    assert blockwise(None, None, None, None, None, 64, 64, 256, 256, 256, 64, None) == _lib.EINVAL


def test_leading_dimension_limits_are_checked_on_the_host():
    """A tile's rows are addressed with 32-bit byte offsets: 256 rows of A or B and 256 rows of
    16-bit output must stay below 2^31 bytes for the MFMA families (pinned here: the automatic
    choice would hand such operands to the generic family). The check comes before any device
    call, so host buffers (never dereferenced) can stand in for the operands."""
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096 + 64)
    base = (ctypes.addressof(buf) + 63) & ~63  # 64-byte aligned stand-in for every operand
    m, n, k = 16, 16, 16
    limit_ab = (2 ** 31 - 1) // 256  # largest lda/ldb that passes, rounded down to a multiple of 16 below
    limit_c = (2 ** 31 - 1) // 512

    def call(lda, ldb, ldc):
        return lib.mi355x_fp8_rowwise_gemm(base, base, base, base, None, base, m, n, k, lda, ldb, ldc, None, 0,
                                           _lib.VARIANT_TILED, None)

    too_wide = (limit_ab // 16 + 1) * 16
    assert call(too_wide, 16, 16) == _lib.ENOTSUP and "leading dimension too large" in _lib.last_error()
    assert call(16, too_wide, 16) == _lib.ENOTSUP and "leading dimension too large" in _lib.last_error()
    assert call(16, 16, limit_c + 1) == _lib.ENOTSUP and "leading dimension too large" in _lib.last_error()
    # smaller than the row is a different complaint
    assert call(8, 16, 16) == _lib.EINVAL and "smaller than the row" in _lib.last_error()


def test_init_reports_a_missing_device_instead_of_crashing():
    import pytest
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is visible: the set-up itself is exercised by the gpu tests")
    lib = _lib.load()
    assert lib.mi355x_fp8_rowwise_init() == _lib.ELAUNCH
    assert "hipGetDevice" in _lib.last_error()
