"""Pins the oracle's row-wise quantiser (torch restatement) with an independent numpy
restatement, the C restatement and invariants the arithmetic fixes."""
import numpy as np
import pytest
import torch

from oracle import cref, e4m3
from oracle import fp8_rowwise as orc


def _codes(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.uint8).numpy()


@pytest.mark.parametrize("rows,cols,sigma", [(1, 16, 1.0), (7, 272, 1.0), (128, 512, 1.0), (33, 4112, 0.02), (5, 48, 1e3)])
def test_three_restatements_agree_bitwise(rows, cols, sigma):
    x = orc.randn_f32(rows, cols, sigma, seed=rows * 1000 + cols)
    xq, inv = orc.fp8_row_quantize(x)
    xq_np, inv_np = orc.fp8_row_quantize_numpy(x.numpy())
    xq_c, inv_c = cref.quantize_rows(x.numpy())
    assert np.array_equal(_codes(xq), xq_np)
    assert np.array_equal(_codes(xq), xq_c)
    assert np.array_equal(inv.numpy().view(np.uint32), inv_np.view(np.uint32))
    assert np.array_equal(inv.numpy().view(np.uint32), inv_c.view(np.uint32))


def test_invariants():
    x = orc.randn_f32(64, 1024, 1.0, seed=3)
    xq, inv = orc.fp8_row_quantize(x)
    deq = e4m3.decode(_codes(xq))
    assert np.all(np.isfinite(deq))
    assert np.all(np.abs(deq) <= 448.0)
    # the largest magnitude of every non-zero row maps onto the largest finite code
    assert np.all(np.max(np.abs(deq), axis=1) == 448.0)
    # reconstruction error is at most half a code spacing at that magnitude (relative 2^-4
    # for normals, absolute 2^-10 in scaled units for subnormals), plus fp32 rounding slack
    scaled = x.numpy().astype(np.float64) * (1.0 / inv.numpy().astype(np.float64))[:, None]
    err = np.abs(deq.astype(np.float64) - scaled)
    bound = np.maximum(np.abs(scaled) * 2.0 ** -4, 2.0 ** -10) * (1 + 1e-5) + 1e-4
    assert np.all(err <= bound)
    # signs survive
    nz = deq != 0
    assert np.array_equal(np.sign(deq[nz]), np.sign(x.numpy()[nz]))


def test_inverse_scale_is_reciprocal_of_scale_not_amax_over_448():
    x = orc.randn_f32(4096, 32, 1.0, seed=11)
    _, inv = orc.fp8_row_quantize(x)
    amax = x.abs().max(dim=1).values
    # float / tensor is reciprocal-then-multiply in torch: two roundings
    scale = amax.reciprocal() * 448.0
    assert torch.equal(inv, scale.reciprocal())
    # the neighbouring formulas really differ on some rows, so the assertion above can fail
    assert not torch.equal(inv, amax / 448.0)
    assert not torch.equal(inv, (torch.tensor(448.0) / amax).reciprocal())


def test_zero_row_and_tiny_row():
    x = torch.zeros(3, 32)
    x[1, 5] = 1e-20
    x[2, 7] = -3.0
    xq, inv = orc.fp8_row_quantize(x)
    codes = _codes(xq)
    assert np.all(codes[0] == 0)
    assert inv[0].item() == np.float32(1.0) / ((np.float32(1.0) / np.float32(1e-12)) * np.float32(448.0))
    # a row whose amax is below EPS is scaled by 448/EPS, not by 448/amax
    assert e4m3.decode(codes[1])[5] == np.float32(e4m3.decode(e4m3.encode_rne(np.float32(1e-20) * ((np.float32(1.0) / np.float32(1e-12)) * np.float32(448.0)))))
    assert codes[2, 7] == 0xFE and np.all(np.delete(codes[2], 7) == 0)
    assert inv[2].item() == pytest.approx(3.0 / 448.0, rel=1e-6)


def test_quantise_is_per_row():
    x = orc.randn_f32(8, 64, 1.0, seed=5)
    xq, inv = orc.fp8_row_quantize(x)
    y = x.clone()
    y[3] *= 1000.0
    yq, yinv = orc.fp8_row_quantize(y)
    keep = [0, 1, 2, 4, 5, 6, 7]
    assert torch.equal(xq.view(torch.uint8)[keep], yq.view(torch.uint8)[keep])
    assert torch.equal(inv[keep], yinv[keep])


def test_bf16_source_runs_in_bf16():
    # the reference feeds bf16 tensors (operator.py:283-288); the arithmetic then rounds to bf16
    x = orc.randn_f32(16, 128, 1.0, seed=9).to(torch.bfloat16)
    xq, inv = orc.fp8_row_quantize(x)
    assert xq.dtype == torch.float8_e4m3fn and inv.dtype == torch.float32
    scale = (448.0 / x.abs().max(dim=1).values)
    assert scale.dtype == torch.bfloat16
    assert torch.equal(inv, scale.reciprocal().float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_non_finite_rows_follow_the_torch_program(dtype):
    # what operator.py:136-145 does with NaN and infinities, fixed by torch.max / clamp / the fp8
    # cast: a NaN poisons its row (NaN maximum -> NaN scale -> every code NaN, NaN inverse scale);
    # an infinity gives scale 1/inf * 448 = 0 (finite elements -> signed zero, inf * 0 -> NaN) and
    # inverse scale +inf. Other rows are untouched. The sign bit of a NaN code is whatever the
    # platform's arithmetic leaves in the NaN, so NaN codes are compared as NaN only.
    x = orc.randn_f32(5, 64, 1.0, seed=77).to(dtype)
    x[1, 3] = float("nan")
    x[2, 4] = float("inf")
    x[2, 9] = float("-inf")
    x[3, 5] = float("-inf")
    x[3, 6] = float("nan")
    xq, inv = orc.fp8_row_quantize(x)
    codes = _codes(xq)
    is_nan = (codes & 0x7F) == 0x7F
    assert is_nan[1].all() and is_nan[3].all()
    assert np.isnan(inv[1].item()) and np.isnan(inv[3].item())
    assert inv[2].item() == float("inf")
    inf_at = torch.isinf(x[2].float()).numpy()
    assert is_nan[2][inf_at].all()
    want_zero = np.where(np.signbit(x[2].float().numpy()[~inf_at]), 0x80, 0x00)
    assert np.array_equal(codes[2][~inf_at], want_zero)
    for r in (0, 4):
        alone_q, alone_inv = orc.fp8_row_quantize(x[r:r + 1].clone())
        assert np.array_equal(codes[r], _codes(alone_q)[0]) and inv[r] == alone_inv[0]
        assert not is_nan[r].any()
