"""ctypes binding of the C ABI declared in include/mi355x_fp8_rowwise.h.

The shared library is loaded from tritonbench_amd/lib/ (built in-tree by
tritonbench_amd.build). There is no fallback: if the library is missing or does not
load, every entry point raises.
"""
import ctypes
import os
import threading
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p

from .build import LIB_PATH

ABI_VERSION = 2

OK = 0
EINVAL = -1
ENOTSUP = -2
ELAUNCH = -3

VARIANT_AUTO = 0
VARIANT_TILED = 1
VARIANT_SKINNY = 2
VARIANT_GENERIC = 3  # byte loads + f32 multiply-adds: any K, leading dimension and alignment
SKINNY_ONE_TILE = 1 << 8  # skinny family: pins the one-tile-per-workgroup kernel
SKINNY_NARROW = 2 << 8  # skinny family: pins the narrow-tile kernel (the shapes `skinny_family_takes`)
SKINNY_RESIDENT = 4 << 8  # skinny family: pins the forms that keep A on chip (pair / persistent kernel)


def skinny_family_takes(m: int, n: int) -> bool:
    """Whether VARIANT_SKINNY accepts an M x N output (it answers "not supported" otherwise): up to
    64 rows always; up to 256 rows where 64x64 tiles in row blocks of 64, the tile count rounded up to
    a multiple of 8, are at most one workgroup per CU."""
    if m <= 64:
        return True
    return m <= 256 and -(-m // 64) * ((-(-n // 64) + 7) // 8 * 8) <= 256

NUM_TILE_CONFIGS = 7
NOALLOC_SCRATCH_BYTES = 64 << 20
STAMP_ENTRIES = 2048
NUM_GROUPED_TILE_CONFIGS = 3


def tiled_variant(config=None, splits=0) -> int:
    """Variant word of the tiled family with the tile configuration and/or split-K factor
    pinned (MI355X_FP8_TILED_CONFIG / MI355X_FP8_TILED_SPLITS of the header)."""
    word = VARIANT_TILED
    if config is not None:
        word |= ((config + 1) & 0xFF) << 8
    return word | ((splits & 0xFF) << 16)


OUT_BF16 = 0
OUT_F16 = 1

SRC_F32 = 0
SRC_BF16 = 1

# symbol -> (restype, argtypes); must list every function the header declares
SIGNATURES = {
    "mi355x_fp8_rowwise_abi_version": (c_int, []),
    "mi355x_fp8_rowwise_init": (c_int, []),
    "mi355x_fp8_rowwise_last_error": (c_char_p, []),
    "mi355x_fp8_rowwise_select_variant": (c_int, [c_int64, c_int64, c_int64]),
    "mi355x_fp8_rowwise_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int]),
    "mi355x_fp8_rowwise_gemm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_size_t, c_int, c_void_p],
    ),
    "mi355x_fp8_rowwise_gemm_ex": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_size_t, c_int, c_void_p],
    ),
    "mi355x_fp8_rowwise_gemm_stamped": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_void_p, c_size_t, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "mi355x_fp8_rowwise_gemm_noalloc": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p],
    ),
    "mi355x_fp8_rowwise_grouped_gemm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
         c_int, c_void_p],
    ),
    "mi355x_fp8_blockwise_gemm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "mi355x_fp8_blockwise_quantize": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "mi355x_fp8_rowwise_quantize": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "mi355x_fp8_rmsnorm_rowwise_quantize": (
        c_int,
        [c_void_p, c_void_p, ctypes.c_float, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "mi355x_fp8_silu_mul_rowwise_quantize": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
}

_lock = threading.Lock()
_lib = None


class LibraryNotBuilt(RuntimeError):
    pass


def library_path() -> str:
    return LIB_PATH


def load() -> ctypes.CDLL:
    """Loads the library once and checks its ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise LibraryNotBuilt(
                f"{LIB_PATH} does not exist; build it with `python -m tritonbench_amd.build` "
                "(needs hipcc). There is no CPU or PyTorch fallback for this operator."
            )
        # The library needs libamdhip64 by soname only. PyTorch-ROCm ships its own copy of the
        # HIP runtime; whichever copy is mapped first serves the whole process, and two
        # different copies cannot share a device. Importing torch first makes its runtime
        # the one this library binds to, so torch streams and pointers are valid here.
        import torch  # noqa: F401

        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is missing
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.mi355x_fp8_rowwise_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH}: ABI version {got}, this binding expects {ABI_VERSION}")
        _lib = lib
    return _lib


_initialised = set()


def init_device(index: int) -> None:
    """Sets device `index` up for the library (mi355x_fp8_rowwise_init: device check, LDS limits of
    every kernel, scratch address), once per process and device. After it every entry point only
    enqueues work there, so any call may be the first of its kind under graph capture."""
    if index in _initialised:
        return
    import torch

    with torch.cuda.device(index):
        check(load().mi355x_fp8_rowwise_init(), "mi355x_fp8_rowwise_init")
    _initialised.add(index)


def last_error() -> str:
    msg = load().mi355x_fp8_rowwise_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(status: int, what: str) -> None:
    """Maps a C status to the exception the benchmark harness understands:
    NotImplementedError becomes a "not supported" cell, anything else propagates."""
    if status == OK:
        return
    msg = f"{what}: {last_error()} (status {status})"
    if status == ENOTSUP:
        raise NotImplementedError(msg)
    if status == EINVAL:
        raise ValueError(msg)
    raise RuntimeError(msg)
