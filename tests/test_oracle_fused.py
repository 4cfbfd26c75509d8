"""Pins the oracle's fused front ends (RMSNorm, SiLU-mul, each followed by the row-wise quantiser)
without a GPU. The kernels the reference operator times for these steps are not part of its
checkout, so the checks are against library routines, float64 loops and closed forms."""
import math

import numpy as np
import pytest
import torch

from oracle import fp8_rowwise as orc


def _bf16(rows, cols, seed, sigma=1.0):
    return orc.randn_f32(rows, cols, sigma, seed=seed).to(torch.bfloat16)


@pytest.mark.parametrize("m,k,eps", [(1, 16, 1e-5), (7, 272, 1e-5), (33, 2048, 1e-6), (4, 6656, 0.0)])
def test_rms_norm_against_library_and_float64_loop(m, k, eps):
    x, w = _bf16(m, k, 3 * m + k), _bf16(1, k, k)[0]
    got = orc.rms_norm(x, w, eps)
    assert got.dtype == torch.float32 and got.shape == (m, k)
    lib = torch.nn.functional.rms_norm(x.float(), (k,), weight=w.float(), eps=eps)
    torch.testing.assert_close(got, lib, rtol=2e-6, atol=1e-7)
    xd, wd = x.double().numpy(), w.double().numpy()
    for r in range(min(m, 5)):
        ms = sum(v * v for v in xd[r]) / k
        want = xd[r] / math.sqrt(ms + eps) * wd
        np.testing.assert_allclose(got[r].numpy(), want, rtol=3e-7, atol=1e-30)


def test_rms_norm_closed_forms():
    k = 64
    w = torch.linspace(-2, 2, k).to(torch.bfloat16)
    # a constant row normalises to its sign: y = sign(c) * w
    x = torch.full((2, k), 3.0, dtype=torch.bfloat16)
    x[1] = -0.5
    y = orc.rms_norm(x, w, eps=0.0)
    assert torch.equal(y[0], w.float()) and torch.equal(y[1], -w.float())
    # scale invariance at eps = 0 (powers of two keep the arithmetic exact)
    x = _bf16(3, k, 9)
    assert torch.equal(orc.rms_norm(x, w, 0.0), orc.rms_norm((x.float() * 4).to(torch.bfloat16), w, 0.0))
    # eps matters: a zero row stays zero instead of dividing by zero
    assert torch.equal(orc.rms_norm(torch.zeros(1, k, dtype=torch.bfloat16), w, 1e-5), torch.zeros(1, k))
    # a dropped weight, a missing square root or a mean taken as a sum would all show here
    x = torch.zeros(1, 4, dtype=torch.bfloat16)
    x[0, 0] = 2.0
    got = orc.rms_norm(x, torch.tensor([3.0, 1.0, 1.0, 1.0]).to(torch.bfloat16), eps=0.0)
    assert got[0, 0].item() == 6.0  # 2 / sqrt(4/4) * 3


@pytest.mark.parametrize("m,k", [(1, 16), (9, 528), (3, 4096)])
def test_silu_mul_against_library_and_definition(m, k):
    x1, x2 = _bf16(m, k, m + k, sigma=3.0), _bf16(m, k, m * k)
    got = orc.silu_mul(x1, x2)
    lib = torch.nn.functional.silu(x1.float()) * x2.float()
    torch.testing.assert_close(got, lib, rtol=2e-6, atol=1e-7)
    a, b = x1.double(), x2.double()
    torch.testing.assert_close(got.double(), a * torch.sigmoid(a) * b, rtol=3e-7, atol=1e-30)
    # special values: silu(0) = 0, large positive passes through, large negative vanishes
    s = orc.silu_mul(torch.tensor([[0.0, 40.0, -40.0, 1.0]]).to(torch.bfloat16), torch.ones(1, 4, dtype=torch.bfloat16))
    assert s[0, 0].item() == 0.0 and s[0, 1].item() == 40.0 and abs(s[0, 2].item()) < 1e-15
    assert s[0, 3].item() == pytest.approx(1.0 / (1.0 + math.exp(-1.0)), rel=1e-6)


def test_fused_quantisers_are_the_front_end_followed_by_the_row_quantiser():
    x1, x2, wq, w_scale, wd = orc.make_fused_inputs(5, 32, 272)
    assert x1.dtype == torch.bfloat16 and wd.shape == (272,) and wq.shape == (32, 272) and w_scale.shape == (32,)
    q, s = orc.rms_norm_fp8_rowwise_quant(x1, wd, 1e-5)
    q2, s2 = orc.fp8_row_quantize(orc.rms_norm(x1, wd, 1e-5))
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
    # the row maximum lands on +-448 and the scale reproduces it
    y = orc.rms_norm(x1, wd, 1e-5)
    assert torch.all(q.float().abs().max(dim=1).values == 448.0)
    torch.testing.assert_close(s * 448.0, y.abs().max(dim=1).values, rtol=1e-6, atol=0)
    q, s = orc.silu_mul_fp8_rowwise_quant(x1, x2)
    y = orc.silu_mul(x1, x2)
    assert torch.all(q.float().abs().max(dim=1).values == 448.0)
    torch.testing.assert_close(s * 448.0, y.abs().max(dim=1).values, rtol=1e-6, atol=0)
