"""Seeded random shapes through every kernel family, tile configuration and split factor,
against the CPU oracle. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to
ATOL = 1e-2


def _shapes(seed, count, max_m, max_n, max_k):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m = int(rng.integers(1, max_m + 1))
        n = int(rng.integers(1, max_n + 1))
        k = 16 * int(rng.integers(1, max_k // 16 + 1))
        out.append((m, n, k, bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("m,n,k,bias", _shapes(101, 24, 700, 900, 3000))
def test_random_shapes_every_plan(gpu_device, m, n, k, bias):
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    d = [None if t is None else t.to(dev) for t in (xq, wq, xs, ws, b)]
    variants = [_lib.VARIANT_AUTO]
    if _lib.skinny_family_takes(m, n):
        variants.append(_lib.VARIANT_SKINNY)
    rng = np.random.default_rng(m * 7919 + n * 31 + k)
    for cfg in range(_lib.NUM_TILE_CONFIGS):
        variants.append(_lib.tiled_variant(cfg, int(rng.integers(1, 7))))
    for variant in variants:
        print(f"case m={m} n={n} k={k} bias={bias} variant={variant:#x}", flush=True)
        out = ops.fp8_gemm_rowwise(d[0], d[1], d[2], d[3], bias=d[4], variant=variant)
        torch.cuda.synchronize()
        torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(8))
def test_random_group_sizes(gpu_device, seed):
    rng = np.random.default_rng(500 + seed)
    g = int(rng.integers(1, 12))
    n = int(rng.integers(1, 400))
    k = 16 * int(rng.integers(1, 80))
    sizes = [int(v) for v in rng.integers(0, 300, size=g)]
    if seed % 3 == 0:
        sizes[int(rng.integers(0, g))] = 0
    m = max(1, sum(sizes) + int(rng.integers(0, 40)) - (20 if seed % 4 == 1 else 0))  # sometimes short of the sum
    xq, wq, ms, xs, ws = orc.make_grouped_inputs(g, m, n, k, sizes=sizes, seed_tag=seed)
    want = orc.grouped_dequant_matmul(xq, wq, ms, xs, ws)
    covered = min(sum(sizes), m)
    dev = gpu_device
    for cfg in [-1] + list(range(_lib.NUM_GROUPED_TILE_CONFIGS)):
        print(f"case g={g} m={m} n={n} k={k} sizes={sizes} tile_config={cfg}", flush=True)
        canvas = torch.full((m, n), -77.0, dtype=torch.bfloat16, device=dev)
        ops.fp8_gemm_rowwise_grouped(xq.to(dev), wq.to(dev), ms.to(dev), xs.to(dev), ws.to(dev), out=canvas, tile_config=cfg)
        torch.cuda.synchronize()
        torch.testing.assert_close(canvas[:covered].cpu(), want[:covered], rtol=RTOL, atol=ATOL)
        assert torch.all(canvas[covered:] == -77.0)


@pytest.mark.parametrize("m,n,k,_", _shapes(303, 10, 600, 700, 2500))
def test_random_shapes_blockwise(gpu_device, m, n, k, _):
    print(f"case m={m} n={n} k={k}", flush=True)
    xq, wq, xs, ws = orc.make_blockwise_inputs(m, n, k)
    want = orc.blockwise_dequant_matmul(xq, wq, xs, ws)
    dev = gpu_device
    out = ops.fp8_gemm_blockwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev))
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(6))
def test_random_quantiser_shapes(gpu_device, seed):
    rng = np.random.default_rng(900 + seed)
    rows = int(rng.integers(1, 300))
    cols = int(rng.integers(1, 5000))
    dtype = torch.float32 if seed % 2 == 0 else torch.bfloat16
    x = orc.randn_f32(rows, cols, float(rng.choice([0.02, 1.0, 30.0])), seed=seed).to(dtype)
    want_q, want_inv = orc.fp8_row_quantize(x)
    got_q, got_inv = ops.fp8_row_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(got_q.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(got_inv.cpu().view(torch.int32), want_inv.view(torch.int32))
