"""Builds the gfx950 shared library from the HIP sources next to this file.

The library has no dependency on PyTorch headers: it is plain HIP behind a C ABI
(include/mi355x_fp8_rowwise.h), compiled with hipcc for gfx950 only.
"""
import os
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(_PKG, "csrc", "fp8_rowwise_gemm.hip")]
LIB_DIR = os.path.join(_PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmi355x_fp8_rowwise.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU forms stay off for every device function in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    cand = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(cand):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return cand


def build_library(verbose: bool = False) -> str:
    """Compiles the library unconditionally and returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-o", tmp, *SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
