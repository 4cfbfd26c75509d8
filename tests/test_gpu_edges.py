"""Edges of the output and of the split-K workspace, and first use under graph capture. Needs an MI355X.

The tiled and narrow-tile kernels mask the rows past a matrix edge with the extent of a buffer
descriptor: the row part of such an access sits in the instruction's scalar offset, the lane part
in its vector offset, and the hardware compares their sum with the extent (loads past it return
zeros, stores past it are dropped). Nothing but that comparison keeps a 256-row tile of a 257-row
problem from writing 255 rows past C. These tests put C and the workspace in front of guard
regions larger than any tile and require every guard byte to survive, on the store paths that
write 16 bytes per lane (N and the row pitch multiples of 8, 16-byte aligned base).
"""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUARD_ROWS = 320          # more than the tallest tile (256 rows)
CANARY = -77.0


def _guarded_output(dev, m, n, pitch):
    buf = torch.full((m + GUARD_ROWS, pitch), CANARY, dtype=torch.bfloat16, device=dev)
    assert buf.data_ptr() % 16 == 0 and pitch % 8 == 0 and n % 8 == 0
    return buf, buf[:m, :n]


def _guard_intact(buf, m, n):
    mask = torch.ones_like(buf, dtype=torch.bool)
    mask[:m, :n] = False
    return bool(torch.all(buf[mask] == CANARY))


# ragged M against every tile height: one row into a new tile row (the other waves of that tile lie
# wholly past the edge), a few rows, and a row count no tile divides; N a multiple of 8 that no tile
# width divides (the last tile column has 8 valid columns); K with a partial last step
EDGE_SHAPES = [(1, 264, 272), (65, 264, 272), (129, 520, 400), (193, 264, 272), (257, 264, 272), (300, 1032, 528)]


@pytest.mark.parametrize("m,n,k", EDGE_SHAPES)
@pytest.mark.parametrize("config", range(_lib.NUM_TILE_CONFIGS))
@pytest.mark.parametrize("splits", [1, 3])
def test_tiled_stores_stay_inside_c_and_workspace(gpu_device, m, n, k, config, splits):
    print(f"case m={m} n={n} k={k} config={config} splits={splits}", flush=True)
    dev = gpu_device
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    variant = _lib.tiled_variant(config, splits)
    need = _lib.load().mi355x_fp8_rowwise_workspace_bytes(m, n, k, variant)
    guard_bytes = GUARD_ROWS * n * 4
    space = torch.full((need + guard_bytes,), 0xA5, dtype=torch.uint8, device=dev)
    buf, c_view = _guarded_output(dev, m, n, n + 8)
    ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), bias=b.to(dev), out=c_view, variant=variant,
                         workspace=space[:need] if need else None)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=1e-2, atol=1e-2)
    assert _guard_intact(buf, m, n), "a store landed outside C"
    assert bool(torch.all(space[need:] == 0xA5)), "a partial-sum store landed past the workspace"


# the narrow-tile forms: all rows in one workgroup (32- and 64-column tiles), and row blocks of every tile size
NARROW_EDGE_SHAPES = [(1, 264, 528), (33, 264, 528), (63, 1032, 272), (47, 8200, 512), (65, 520, 528), (100, 2056, 528),
                      (129, 1032, 272), (200, 4104, 528), (255, 264, 1040)]


@pytest.mark.parametrize("m,n,k", NARROW_EDGE_SHAPES)
def test_narrow_tile_stores_stay_inside_c(gpu_device, m, n, k):
    if not _lib.skinny_family_takes(m, n):
        pytest.skip("the narrow-tile form does not take this shape")
    print(f"case m={m} n={n} k={k}", flush=True)
    dev = gpu_device
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    buf, c_view = _guarded_output(dev, m, n, n + 8)
    ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), bias=b.to(dev), out=c_view,
                         variant=_lib.VARIANT_SKINNY | _lib.SKINNY_NARROW)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=1e-2, atol=1e-2)
    assert _guard_intact(buf, m, n), "a store landed outside C"


def test_grouped_and_blockwise_stores_stay_inside_c(gpu_device):
    dev = gpu_device
    gq, gw, gm, gs, gws = orc.make_grouped_inputs(3, 300, 264, 272, sizes=[130, 0, 150])
    want = orc.grouped_dequant_matmul(gq, gw, gm, gs, gws)
    for config in range(_lib.NUM_GROUPED_TILE_CONFIGS):
        print(f"grouped config={config}", flush=True)
        # (rows 280..299 belong to no group and are left untouched: they start as canaries too)
        buf, c_view = _guarded_output(dev, 300, 264, 272)
        ops.fp8_gemm_rowwise_grouped(gq.to(dev), gw.to(dev), gm.to(dev), gs.to(dev), gws.to(dev), out=c_view, tile_config=config)
        torch.cuda.synchronize()
        torch.testing.assert_close(c_view[:280].cpu(), want[:280], rtol=1e-2, atol=1e-2)
        assert bool(torch.all(c_view[280:] == CANARY))
        assert _guard_intact(buf, 300, 264)
    bq, bw, bs, bws = orc.make_blockwise_inputs(130, 264, 272)
    want = orc.blockwise_dequant_matmul(bq, bw, bs, bws)
    buf, c_view = _guarded_output(dev, 130, 264, 272)
    ops.fp8_gemm_blockwise(bq.to(dev), bw.to(dev), bs.to(dev), bws.to(dev), out=c_view)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=1e-2, atol=1e-2)
    assert _guard_intact(buf, 130, 264)


_FIRST_USE_UNDER_CAPTURE = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops
dev = torch.device("cuda:0")
# (the quantiser and the device set-up run eagerly; no GEMM kernel of the library has run in this process)
cases = []
for (m, n, k, bias, variant) in [(320, 1536, 8192, True, _lib.VARIANT_AUTO), (16, 512, 2048, False, _lib.VARIANT_AUTO),
                                 (100, 264, 528, True, _lib.VARIANT_SKINNY | _lib.SKINNY_NARROW), (700, 520, 272, False, _lib.tiled_variant(5, 0))]:
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    d = lambda t: None if t is None else t.to(dev)
    cases.append((d(xq), d(wq), d(xs), d(ws), d(b), torch.zeros((m, n), dtype=torch.bfloat16, device=dev),
                  ops.gemm_workspace(m, n, k, dev, variant), variant, orc.dequant_matmul(xq, wq, xs, ws, b)))
torch.cuda.synchronize()
side = torch.cuda.Stream()
g = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(g, stream=side):
        for (xq, wq, xs, ws, b, out, space, variant, _) in cases:
            ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=space, variant=variant)
torch.cuda.synchronize()
for replay in range(3):
    for c in cases:
        c[5].zero_()
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    for (xq, wq, xs, ws, b, out, space, variant, want) in cases:
        torch.testing.assert_close(out.cpu(), want, rtol=1e-2, atol=1e-2)
print("FIRST-USE-UNDER-CAPTURE OK")
"""


def test_first_use_of_every_kernel_family_may_be_under_graph_capture(gpu_device):
    """A fresh process whose very first GEMM calls (split-K tiled plan + finalize, persistent skinny,
    narrow tiles, a pinned tile configuration) are recorded into a graph: after the device set-up no
    launch path makes anything but launches, so the capture succeeds and every replay is right."""
    proc = subprocess.run([sys.executable, "-c", _FIRST_USE_UNDER_CAPTURE, ROOT], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=300)
    print(proc.stdout[-2000:], flush=True)
    assert proc.returncode == 0 and "FIRST-USE-UNDER-CAPTURE OK" in proc.stdout
