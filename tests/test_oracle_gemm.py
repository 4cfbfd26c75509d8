"""Pins the oracle's GEMM (fp32 dequantise + torch.matmul) against float64 brute force,
exact-integer cases, structured operands and the C restatement, then pins the committed
golden fixtures to the oracle."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import cref, e4m3
from oracle import fp8_rowwise as orc

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _codes(t):
    return t.view(torch.uint8).numpy()


def _bits(t):
    return t.view(torch.int16).numpy().view(np.uint16)


def _ulp_bf16(x):
    x = np.maximum(np.abs(x), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(x)) - 7)


def _fp32_sum_slack(a_codes, b_codes, a_scale, b_scale):
    """Bound on how far an fp32 accumulation in any order can sit from the exact sum:
    k * eps32 * sum_k |a||b| (scaled). Matters only where the sum cancels to near zero."""
    a = np.abs(e4m3.decode(a_codes).astype(np.float64))
    b = np.abs(e4m3.decode(b_codes).astype(np.float64))
    k = a.shape[1]
    return (a @ b.T) * a_scale.astype(np.float64)[:, None] * b_scale.astype(np.float64)[None, :] * k * 2.0 ** -24


@pytest.mark.parametrize("m,n,k,bias", [(1, 1, 16, False), (3, 5, 16, True), (17, 33, 272, True), (33, 17, 144, False), (16, 16, 128, False)])
def test_against_float64_bruteforce(m, n, k, bias):
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    got = orc.dequant_matmul(xq, wq, xs, ws, b).float().numpy().astype(np.float64)
    exact = orc.gemm_f64(_codes(xq), _codes(wq), xs.numpy(), ws.numpy(), _bits(b) if bias else None)
    # one bf16 rounding (half ulp) plus fp32 accumulation noise
    slack = _fp32_sum_slack(_codes(xq), _codes(wq), xs.numpy(), ws.numpy())
    assert np.all(np.abs(got - exact) <= 0.5 * _ulp_bf16(exact) * 1.001 + slack)


def test_exact_integer_case_is_bit_exact():
    # codes of small integers, unit scales: every partial sum < 2^24, so fp32 is exact and the
    # only rounding is the final bf16 one, which a float64 computation reproduces bit for bit
    rng = np.random.default_rng(7)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4], dtype=np.float32)
    m, n, k = 24, 40, 256
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    xq = torch.from_numpy(a).to(torch.float8_e4m3fn)
    wq = torch.from_numpy(b).to(torch.float8_e4m3fn)
    assert np.array_equal(e4m3.decode(_codes(xq)), a)
    ones_m, ones_n = torch.ones(m), torch.ones(n)
    got = _bits(orc.dequant_matmul(xq, wq, ones_m, ones_n))
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(got, want)
    assert np.array_equal(cref.gemm(_codes(xq), _codes(wq), np.ones(m, np.float32), np.ones(n, np.float32)), want)


def test_identity_weight_returns_scaled_activation():
    k = 64
    xq, _, xs, _, _ = orc.make_inputs(9, k, k, 1.0, False)
    eye = torch.eye(k).to(torch.float8_e4m3fn)
    ws = torch.linspace(0.5, 2.0, k)
    got = orc.dequant_matmul(xq, eye, xs, ws).float()
    want = (xq.float() * xs[:, None] * ws[None, :]).to(torch.bfloat16).float()
    assert torch.equal(got, want)


def test_one_hot_operands_catch_transposition():
    m, n, k = 5, 7, 32
    a = torch.zeros(m, k)
    b = torch.zeros(n, k)
    a[2, 9] = 3.0
    b[4, 9] = 2.0
    b[6, 10] = 5.0  # different k: must not contribute
    out = orc.dequant_matmul(a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn), torch.ones(m), torch.ones(n)).float()
    want = torch.zeros(m, n)
    want[2, 4] = 6.0
    assert torch.equal(out, want)


def test_scales_are_row_of_a_and_row_of_b():
    m, n, k = 4, 6, 16
    a = torch.ones(m, k).to(torch.float8_e4m3fn)
    b = torch.ones(n, k).to(torch.float8_e4m3fn)
    xs = torch.tensor([1.0, 2.0, 4.0, 8.0])
    ws = torch.tensor([1.0, 0.5, 0.25, 3.0, 5.0, 7.0])
    out = orc.dequant_matmul(a, b, xs, ws).float()
    assert torch.equal(out, (k * xs[:, None] * ws[None, :]))


def test_bias_added_before_single_rounding():
    # 256 + 1 is not representable in bf16 (8 significant bits): adding the bias in fp32
    # before rounding gives bf16(257.0) = 256 or 258 by RNE -> 256; rounding first and then
    # adding in bf16 would give the same here, so use a case that separates them:
    # acc = 1.00390625 (1 + 2^-8, rounds to 1.0 in bf16), bias = 2^-8 -> fused: bf16(1.0078125) = 1.0078125
    a = torch.tensor([[1.0] + [0.0] * 15]).to(torch.float8_e4m3fn)
    b = torch.tensor([[1.0] + [0.0] * 15]).to(torch.float8_e4m3fn)
    xs = torch.tensor([1.00390625])
    ws = torch.tensor([1.0])
    bias = torch.tensor([2.0 ** -8]).to(torch.bfloat16)
    fused = orc.dequant_matmul(a, b, xs, ws, bias).float().item()
    assert fused == 1.0078125
    two_step = (orc.dequant_matmul(a, b, xs, ws) + bias).float().item()
    assert two_step == 1.0  # what the CK/cuBLAS style callables of operator.py:207-213 produce
    assert fused != two_step


@pytest.mark.parametrize("m,n,k,bias", [(33, 65, 272, True), (128, 256, 512, False)])
def test_c_restatement_agrees_within_one_ulp(m, n, k, bias):
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    got = orc.dequant_matmul(xq, wq, xs, ws, b)
    c = cref.gemm(_codes(xq), _codes(wq), xs.numpy(), ws.numpy(), _bits(b) if bias else None)
    a_f = orc.bf16_bits_to_f32(_bits(got)).astype(np.float64)
    c_f = orc.bf16_bits_to_f32(c).astype(np.float64)
    slack = _fp32_sum_slack(_codes(xq), _codes(wq), xs.numpy(), ws.numpy())
    assert np.all(np.abs(a_f - c_f) <= _ulp_bf16(c_f) + slack)
    assert np.mean(_bits(got) == c) > 0.98


def test_metric_closed_forms():
    assert orc.flops(8192, 8192, 8192, False) == 2 * 8192 ** 3
    assert orc.flops(1000, 3000, 4112, True) == 2 * 1000 * 3000 * 4112 + 2 * 1000 * 3000
    assert orc.moved_bytes(16, 8192, 8192) == 67502080


def test_golden_fixtures_match_oracle():
    with open(os.path.join(GOLDEN, "manifest.json")) as f:
        manifest = json.load(f)
    assert manifest["cases"], "no golden cases"
    for case in manifest["cases"]:
        z = np.load(os.path.join(GOLDEN, case["file"]), allow_pickle=False)
        m, n, k = case["m"], case["n"], case["k"]
        assert z["a"].shape == (m, k) and z["b"].shape == (n, k) and z["c"].shape == (m, n)
        xq = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
        wq = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn)
        bias = torch.from_numpy(z["bias"].view(np.int16)).view(torch.bfloat16) if case["bias"] else None
        out = orc.dequant_matmul(xq, wq, torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"]), bias)
        # the stored output came from this oracle on this machine class; a different BLAS may
        # reorder fp32 sums, so allow one bf16 ulp and demand near-total bit agreement
        got = orc.bf16_bits_to_f32(_bits(out)).astype(np.float64)
        want = orc.bf16_bits_to_f32(z["c"]).astype(np.float64)
        slack = _fp32_sum_slack(z["a"], z["b"], z["a_scale"], z["b_scale"])
        assert np.all(np.abs(got - want) <= _ulp_bf16(want) + slack), case["name"]
        assert np.mean(_bits(out) == z["c"]) > 0.99, case["name"]
        # and the fixture itself is consistent with float64 brute force
        exact = orc.gemm_f64(z["a"], z["b"], z["a_scale"], z["b_scale"], z["bias"] if case["bias"] else None)
        assert np.all(np.abs(want - exact) <= 0.501 * _ulp_bf16(exact) + slack), case["name"]


def test_split_form_equals_dequant_matmul():
    xq, wq, xs, ws, b = orc.make_inputs(40, 72, 144, 1.0, True)
    whole = orc.dequant_matmul(xq, wq, xs, ws, b)
    rows = torch.tensor([0, 7, 39])
    part = orc.dequant_matmul_rows(orc.dequantize(xq[rows], xs[rows]), orc.dequantize(wq, ws), b)
    assert torch.equal(part, whole[rows])


# ---- grouped form -------------------------------------------------------------------------
def _grouped_bruteforce(xq, wq, sizes, xs, ws):
    """Row by row in float64: the group of a row is found from the running sum of the sizes."""
    a = e4m3.decode(xq.view(torch.uint8).numpy()).astype(np.float64)
    b = e4m3.decode(wq.view(torch.uint8).numpy()).astype(np.float64)
    m, n = a.shape[0], b.shape[0] // len(sizes)
    out, mag = np.zeros((m, n)), np.zeros((m, n))
    bounds = np.cumsum([0] + [max(int(s), 0) for s in sizes])
    for r in range(m):
        g = int(np.searchsorted(bounds, r, side="right")) - 1
        if g >= len(sizes):
            continue  # past the last group: stays zero
        for c in range(n):
            out[r, c] = np.dot(a[r], b[g * n + c]) * float(xs[r]) * float(ws[g * n + c])
            mag[r, c] = np.dot(np.abs(a[r]), np.abs(b[g * n + c])) * float(xs[r]) * float(ws[g * n + c])
    # second value: what fp32 accumulation in any order may add to the error
    return out, mag * a.shape[1] * 2.0 ** -24


@pytest.mark.parametrize("g,m,n,k,sizes", [
    (2, 12, 5, 32, None), (3, 20, 7, 48, [5, 0, 9]), (4, 16, 3, 16, [1, 2, 3, 10]), (1, 9, 4, 64, [9]),
    (3, 10, 6, 32, [4, 9, 2]),  # runs past M: cut off at the last row
])
def test_grouped_against_float64_bruteforce(g, m, n, k, sizes):
    xq, wq, ms, xs, ws = orc.make_grouped_inputs(g, m, n, k, sizes=sizes)
    got = orc.grouped_dequant_matmul(xq, wq, ms, xs, ws).float().numpy().astype(np.float64)
    # the brute force applies the same cut at M by construction (rows only run to m - 1)
    want, slack = _grouped_bruteforce(xq, wq, [int(v) for v in ms], xs, ws)
    # one bf16 rounding (2^-9 relative) plus fp32 accumulation noise
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + slack)


def test_grouped_with_one_group_is_the_plain_product():
    xq, wq, ms, xs, ws = orc.make_grouped_inputs(1, 24, 10, 96)
    assert torch.equal(orc.grouped_dequant_matmul(xq, wq, ms, xs, ws), orc.dequant_matmul(xq, wq, xs, ws))


def test_grouped_rows_use_their_own_groups_weights_and_scales():
    # A = ones, B rows of group g all equal to g + 1, K = 16: C = 16 * (g + 1) * a_scale * b_scale
    g, n, k = 3, 4, 16
    sizes = [2, 3, 1]
    m = 8  # two rows more than the sizes cover
    xq = torch.ones(m, k).to(torch.float8_e4m3fn)
    wq = torch.cat([torch.full((n, k), float(i + 1)) for i in range(g)]).to(torch.float8_e4m3fn)
    xs = torch.arange(1, m + 1, dtype=torch.float32)
    ws = torch.full((g * n,), 0.5)
    out = orc.grouped_dequant_matmul(xq, wq, torch.tensor(sizes, dtype=torch.int32), xs, ws).float()
    group_of_row = [0, 0, 1, 1, 1, 2]
    for r, gi in enumerate(group_of_row):
        assert torch.all(out[r] == 16.0 * (gi + 1) * (r + 1) * 0.5)
    assert torch.all(out[6:] == 0)


def test_grouped_golden_fixtures_match_oracle_and_bruteforce():
    with open(os.path.join(GOLDEN, "manifest.json")) as f:
        manifest = json.load(f)
    assert manifest["grouped_cases"], "no grouped golden cases"
    for case in manifest["grouped_cases"]:
        z = np.load(os.path.join(GOLDEN, case["file"]), allow_pickle=False)
        g, m, n, k = case["g"], case["m"], case["n"], case["k"]
        assert z["a"].shape == (m, k) and z["b"].shape == (g * n, k) and z["c"].shape == (m, n)
        assert z["m_sizes"].dtype == np.int32 and z["m_sizes"].shape == (g,)
        xq = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
        wq = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn)
        xs, ws = torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"])
        out = orc.grouped_dequant_matmul(xq, wq, torch.from_numpy(z["m_sizes"]), xs, ws)
        assert np.mean(_bits(out) == z["c"]) > 0.99, case["name"]
        want = orc.bf16_bits_to_f32(z["c"]).astype(np.float64)
        exact, slack = _grouped_bruteforce(xq, wq, z["m_sizes"].tolist(), xs, ws)
        assert np.all(np.abs(want - exact) <= np.abs(exact) * 2.0 ** -8 + slack), case["name"]
