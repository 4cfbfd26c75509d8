"""ctypes loader for oracle/fp8_rowwise_ref.c. TEST INFRASTRUCTURE ONLY (see oracle/__init__.py)."""
import ctypes
import os
import subprocess
from typing import Optional

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "_build", "liboracle_fp8_rowwise.so")
_lib = None


def build() -> str:
    """Compiles the C oracle with the Makefile beside it (gcc only)."""
    subprocess.run(["make", "-C", _DIR, "-B"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = ctypes.CDLL(LIB_PATH)
        lib.oracle_e4m3_decode.restype = ctypes.c_float
        lib.oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
        lib.oracle_e4m3_encode.restype = ctypes.c_uint8
        lib.oracle_e4m3_encode.argtypes = [ctypes.c_float]
        lib.oracle_quantize_rows.restype = None
        lib.oracle_quantize_rows.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        lib.oracle_gemm.restype = None
        lib.oracle_gemm.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 3
        _lib = lib
    return _lib


def quantize_rows(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    r, k = x.shape
    xq = np.empty((r, k), dtype=np.uint8)
    inv = np.empty((r,), dtype=np.float32)
    load().oracle_quantize_rows(x.ctypes.data, r, k, xq.ctypes.data, inv.ctypes.data)
    return xq, inv


def gemm(a: np.ndarray, b: np.ndarray, a_scale: np.ndarray, b_scale: np.ndarray,
         bias_bits: Optional[np.ndarray] = None) -> np.ndarray:
    """uint8 codes in, bf16 bit patterns (uint16 [M,N]) out; double accumulation."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    a_scale = np.ascontiguousarray(a_scale, dtype=np.float32)
    b_scale = np.ascontiguousarray(b_scale, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0]
    assert b.shape[1] == k and a_scale.shape == (m,) and b_scale.shape == (n,)
    c = np.empty((m, n), dtype=np.uint16)
    bias_ptr = None
    if bias_bits is not None:
        bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
        assert bias_bits.shape == (n,)
        bias_ptr = bias_bits.ctypes.data
    load().oracle_gemm(a.ctypes.data, b.ctypes.data, a_scale.ctypes.data, b_scale.ctypes.data,
                       bias_ptr, c.ctypes.data, m, n, k)
    return c
