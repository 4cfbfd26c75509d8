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


NUM_TILED_PARTS = 7  # mi355x_shared::kNumTiledParts in the source
BUILD_DIR = os.path.join(_PKG, "lib", "obj")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + proc.stdout)


def build_library(verbose: bool = False, jobs: int = 0) -> str:
    """Compiles the library unconditionally and returns its path.

    The one source file is compiled as several translation units side by side (the main unit and
    one per tile configuration of the tiled kernel, selected by -DMI355X_SPLIT_MAIN and
    -DMI355X_TILED_PART=<k>) and linked into one shared object; `jobs` = 1 compiles it as a single
    unit instead (same library, about four times the wall time)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = find_hipcc()
    tmp = LIB_PATH + ".tmp"
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    if jobs == 1:
        _run([hipcc, *HIPCC_FLAGS, "-o", tmp, *SOURCES], verbose)
        os.replace(tmp, LIB_PATH)
        return LIB_PATH
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(BUILD_DIR, exist_ok=True)
    units = [("main", ["-DMI355X_SPLIT_MAIN"])] + [(f"tiled{k}", [f"-DMI355X_TILED_PART={k}"]) for k in range(NUM_TILED_PARTS)]
    objects = [os.path.join(BUILD_DIR, name + ".o") for name, _ in units]
    workers = jobs if jobs > 0 else min(len(units), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        futures = [pool.submit(_run, [hipcc, *flags, *defs, "-c", SOURCES[0], "-o", obj], verbose)
                   for (name, defs), obj in zip(units, objects)]
        for f in futures:
            f.result()
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", tmp, *objects], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
