"""Pins the oracle's block-scaled functions (quantiser and product) without a GPU."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc


def _codes(t):
    return t.view(torch.uint8).numpy()


@pytest.mark.parametrize("m,k,sigma", [(128, 128, 1.0), (130, 272, 1.0), (1, 16, 0.02), (300, 640, 3.0), (257, 129, 1.0)])
def test_block_quantiser_against_independent_numpy_restatement(m, k, sigma):
    x = orc.randn_f32(m, k, sigma, seed=m * 7 + k)
    xq, inv = orc.fp8_block_quantize(x)
    gm, gk = -(-m // 128), -(-k // 128)
    assert xq.shape == (m, k) and inv.shape == (gm, gk) and inv.dtype == torch.float32
    xn = x.numpy()
    want_codes = np.zeros((m, k), np.uint8)
    for bi in range(gm):
        for bj in range(gk):
            blk = xn[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128]
            amax = np.float32(max(np.abs(blk).max(), np.float32(1e-12)))
            scale = np.float32(np.float32(1.0) / amax) * np.float32(448.0)  # how PyTorch evaluates 448 / t
            assert np.float32(1.0) / scale == inv[bi, bj].item()
            want_codes[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128] = e4m3.encode_rne(blk * scale)
    assert np.array_equal(_codes(xq), want_codes)
    # invariants: the block maximum lands on +-448, and dequantising is within half an e4m3 step
    back = e4m3.decode(_codes(xq)).astype(np.float64)
    for bi in range(gm):
        for bj in range(gk):
            sl = (slice(bi * 128, (bi + 1) * 128), slice(bj * 128, (bj + 1) * 128))
            assert np.abs(back[sl]).max() == 448.0
            err = np.abs(back[sl] * inv[bi, bj].item() - xn[sl])
            step = np.maximum(np.abs(back[sl]), 2.0 ** -6) * 2.0 ** -3 * inv[bi, bj].item()
            assert np.all(err <= 0.5001 * step + 1e-30)


def test_block_quantiser_zero_block_and_padding():
    x = torch.zeros(140, 200)
    x[130:, 150:] = 2.0  # only the last (partial) block is non-zero
    xq, inv = orc.fp8_block_quantize(x)
    assert inv.shape == (2, 2)
    assert torch.all(xq[:128].float() == 0) and torch.all(xq[128:, :128].float() == 0)
    assert inv[0, 0].item() == np.float32(1.0) / (np.float32(np.float32(1.0) / np.float32(1e-12)) * np.float32(448.0))
    assert torch.all(xq[130:, 150:].float() == 448.0) and inv[1, 1].item() == pytest.approx(2.0 / 448.0, rel=1e-6)


def _blockwise_bruteforce(xq, wq, xs, ws):
    a = e4m3.decode(_codes(xq)).astype(np.float64)
    b = e4m3.decode(_codes(wq)).astype(np.float64)
    m, k = a.shape
    n = b.shape[0]
    out, mag = np.zeros((m, n)), np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            for kb in range(-(-k // 128)):
                ks = slice(kb * 128, min((kb + 1) * 128, k))
                s = float(xs[i // 128, kb]) * float(ws[j // 128, kb])
                out[i, j] += np.dot(a[i, ks], b[j, ks]) * s
                mag[i, j] += np.dot(np.abs(a[i, ks]), np.abs(b[j, ks])) * s
    return out, mag * k * 2.0 ** -24


@pytest.mark.parametrize("m,n,k", [(5, 7, 128), (9, 6, 272), (130, 3, 384), (4, 131, 144)])
def test_blockwise_product_against_float64_bruteforce(m, n, k):
    xq, wq, xs, ws = orc.make_blockwise_inputs(m, n, k)
    got = orc.blockwise_dequant_matmul(xq, wq, xs, ws).float().numpy().astype(np.float64)
    want, slack = _blockwise_bruteforce(xq, wq, xs, ws)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + slack)


def test_blockwise_with_uniform_scales_is_the_rowwise_product():
    # one scale value for all of A and one for all of B: the block-scaled product must equal the
    # row-wise one with constant scale vectors (same fp32 operations in the same order)
    m, n, k = 40, 24, 256
    xq, wq, _, _ = orc.make_blockwise_inputs(m, n, k)
    xs = torch.full((1, 2), 0.25)
    ws = torch.full((1, 2), 3.0)
    assert torch.equal(orc.blockwise_dequant_matmul(xq, wq, xs, ws),
                       orc.dequant_matmul(xq, wq, torch.full((m,), 0.25), torch.full((n,), 3.0)))


def test_blockwise_scales_pick_their_own_k_block():
    # A = ones, B = ones, K = 256: C = 128 * (xs[0,0]*ws[0,0] + xs[0,1]*ws[0,1])
    xq = torch.ones(3, 256).to(torch.float8_e4m3fn)
    wq = torch.ones(2, 256).to(torch.float8_e4m3fn)
    xs = torch.tensor([[0.5, 2.0]])
    ws = torch.tensor([[4.0, 0.25]])
    out = orc.blockwise_dequant_matmul(xq, wq, xs, ws).float()
    assert torch.all(out == 128 * (0.5 * 4.0 + 2.0 * 0.25))


def test_blockwise_golden_fixture_matches_oracle_and_bruteforce():
    import json
    import os

    golden = os.path.join(os.path.dirname(__file__), "golden")
    with open(os.path.join(golden, "manifest.json")) as f:
        manifest = json.load(f)
    assert manifest["blockwise_cases"]
    for case in manifest["blockwise_cases"]:
        z = np.load(os.path.join(golden, case["file"]), allow_pickle=False)
        m, n, k = case["m"], case["n"], case["k"]
        assert z["a"].shape == (m, k) and z["b"].shape == (n, k) and z["c"].shape == (m, n)
        assert z["a_scale"].shape == (-(-m // 128), -(-k // 128)) and z["b_scale"].shape == (-(-n // 128), -(-k // 128))
        xq = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
        wq = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn)
        xs, ws = torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"])
        out = orc.blockwise_dequant_matmul(xq, wq, xs, ws)
        got_bits = out.view(torch.int16).numpy().view(np.uint16)
        assert np.mean(got_bits == z["c"]) > 0.99, case["name"]
        want = orc.bf16_bits_to_f32(z["c"]).astype(np.float64)
        exact, slack = _blockwise_bruteforce(xq, wq, xs, ws)
        assert np.all(np.abs(want - exact) <= np.abs(exact) * 2.0 ** -8 + slack), case["name"]
