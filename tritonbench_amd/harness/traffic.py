"""Turns two rocprofv3 counter passes over `bench.py --profile-kernel <which>` into the small
JSON summary bench.py reports as `roofline.traffic`.

    rocprofv3 --pmc FETCH_SIZE -f csv -d <dir>/fetch -o run -- python3 bench.py --profile-kernel tiled > <dir>/fetch.json
    rocprofv3 --pmc WRITE_SIZE -f csv -d <dir>/write -o run -- python3 bench.py --profile-kernel tiled > <dir>/write.json
    python -m tritonbench_amd.harness.traffic --dir <dir> --kernel "gemm_tiled_kernel<256, 256" --out profiles/tiled_8192cubed_traffic.json

Both counters read KiB per dispatch; each is scaled by what it reads for the copy kernel of
known size that bench.py launches in the same run (an elementwise negation of a 256 MiB tensor).
The summary records the hash of the kernel source it was measured on; bench.py marks a summary
whose hash differs from the present source as stale.
"""
import argparse
import json
import os
import sys

from . import rocprof


def _bench_line(path: str) -> dict:
    with open(path) as f:
        for line in f:
            line = line.strip()
            if line.startswith("{") and "profile_kernel" in line:
                return json.loads(line)
    raise ValueError(f"{path} holds no bench.py --profile-kernel line")


def summarise(directory: str, kernel: str) -> dict:
    meta = _bench_line(os.path.join(directory, "fetch.json"))
    meta_w = _bench_line(os.path.join(directory, "write.json"))
    if meta["source_sha"] != meta_w["source_sha"] or meta["profile_kernel"] != meta_w["profile_kernel"]:
        raise ValueError("the two passes ran different kernels or kernel sources")
    cal = meta["calibration"]
    out = rocprof.traffic_summary(
        rocprof._find(os.path.join(directory, "fetch"), "_counter_collection.csv"),
        rocprof._find(os.path.join(directory, "write"), "_counter_collection.csv"),
        kernel, cal["kernel"], cal["read_bytes"], cal["write_bytes"])
    out["workload"] = meta["profile_kernel"]
    out["source_sha"] = meta["source_sha"]
    out["counters"] = "rocprofv3 --pmc FETCH_SIZE / --pmc WRITE_SIZE (KiB per dispatch), one pass each"
    out["calibration"] = f"{cal['kernel']} elementwise kernel reading {cal['read_bytes']} and writing {cal['write_bytes']} bytes"
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--dir", required=True, help="directory holding fetch/, write/, fetch.json and write.json")
    ap.add_argument("--kernel", required=True, help="substring of the kernel's name")
    ap.add_argument("--out", required=True)
    a = ap.parse_args(argv)
    out = summarise(a.dir, a.kernel)
    with open(a.out, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
