"""Writes the golden fixtures in this directory from the repository's own CPU oracle.

The tritonbench checkout holds no golden vectors or known-answer tests for
fp8_gemm_rowwise (the operator is skipped by its CI), so the vectors are produced here:
seeded inputs, quantised by oracle.fp8_rowwise.fp8_row_quantize, outputs from
oracle.fp8_rowwise.dequant_matmul (grouped_dequant_matmul / blockwise_dequant_matmul for the grouped and block-scaled cases). Each .npz holds raw arrays only (uint8 e4m3fn codes,
float32 scales, uint16 bf16 bit patterns); load with allow_pickle=False.

    python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import fp8_rowwise as orc  # noqa: E402

CASES = [
    # name, m, n, k, sigma, bias
    ("c1_plumbing_128x256x512", 128, 256, 512, 1.0, False),
    ("ragged_33x65x272_bias", 33, 65, 272, 1.0, True),
    ("ragged_17x300x144", 17, 300, 144, 1.0, False),
    ("decode_1x512x1024_sigma002", 1, 512, 1024, 0.02, False),
    ("edge_257x259x400_bias", 257, 259, 400, 1.0, True),
]


GROUPED_CASES = [
    # name, g, m, n, k, sizes
    ("grouped_g3_300x72x144", 3, 300, 72, 144, [130, 0, 150]),  # an empty group; 20 rows owned by no group
    ("grouped_g2_64x33x272", 2, 64, 33, 272, None),              # equal split, N not a multiple of 4
]


BLOCKWISE_CASES = [
    # name, m, n, k  (128x128 block scales)
    ("blockwise_130x72x272", 130, 72, 272),
]


def main():
    manifest = {"generator": "tests/golden/make_golden.py", "seed": orc.MAIN_RANDOM_SEED, "cases": []}
    for name, m, n, k, sigma, bias in CASES:
        xq, wq, xs, ws, b = orc.make_inputs(m, n, k, sigma, bias)
        out = orc.dequant_matmul(xq, wq, xs, ws, b)
        arrays = dict(
            a=xq.view(torch.uint8).numpy(),
            b=wq.view(torch.uint8).numpy(),
            a_scale=xs.numpy(),
            b_scale=ws.numpy(),
            c=out.view(torch.int16).numpy().view(np.uint16),
        )
        if bias:
            arrays["bias"] = b.view(torch.int16).numpy().view(np.uint16)
        fname = name + ".npz"
        np.savez_compressed(os.path.join(HERE, fname), **arrays)
        digest = hashlib.sha256(b"".join(np.ascontiguousarray(v).tobytes() for _, v in sorted(arrays.items()))).hexdigest()
        manifest["cases"].append(dict(name=name, file=fname, m=m, n=n, k=k, sigma=sigma, bias=bias, sha256=digest))
    manifest["grouped_cases"] = []
    for name, g, m, n, k, sizes in GROUPED_CASES:
        xq, wq, ms, xs, ws = orc.make_grouped_inputs(g, m, n, k, sizes=sizes)
        out = orc.grouped_dequant_matmul(xq, wq, ms, xs, ws)
        arrays = dict(
            a=xq.view(torch.uint8).numpy(),
            b=wq.view(torch.uint8).numpy(),
            m_sizes=ms.numpy(),
            a_scale=xs.numpy(),
            b_scale=ws.numpy(),
            c=out.view(torch.int16).numpy().view(np.uint16),
        )
        fname = name + ".npz"
        np.savez_compressed(os.path.join(HERE, fname), **arrays)
        digest = hashlib.sha256(b"".join(np.ascontiguousarray(v).tobytes() for _, v in sorted(arrays.items()))).hexdigest()
        manifest["grouped_cases"].append(dict(name=name, file=fname, g=g, m=m, n=n, k=k, sha256=digest))
    manifest["blockwise_cases"] = []
    for name, m, n, k in BLOCKWISE_CASES:
        xq, wq, xs, ws = orc.make_blockwise_inputs(m, n, k)
        out = orc.blockwise_dequant_matmul(xq, wq, xs, ws)
        arrays = dict(
            a=xq.view(torch.uint8).numpy(),
            b=wq.view(torch.uint8).numpy(),
            a_scale=xs.numpy(),
            b_scale=ws.numpy(),
            c=out.view(torch.int16).numpy().view(np.uint16),
        )
        fname = name + ".npz"
        np.savez_compressed(os.path.join(HERE, fname), **arrays)
        digest = hashlib.sha256(b"".join(np.ascontiguousarray(v).tobytes() for _, v in sorted(arrays.items()))).hexdigest()
        manifest["blockwise_cases"].append(dict(name=name, file=fname, m=m, n=n, k=k, sha256=digest))
    with open(os.path.join(HERE, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    print(f"wrote {len(CASES)} + {len(GROUPED_CASES)} + {len(BLOCKWISE_CASES)} cases")


if __name__ == "__main__":
    main()
