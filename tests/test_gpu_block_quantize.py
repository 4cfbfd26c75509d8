"""Parity of the block-wise quantiser kernel (through the C ABI) with the CPU oracle's restatement of
fp8_block_quantize (tritonbench/operators/fp8_gemm_blockwise/operator.py:86-118): codes and inverse
scales bit for bit. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _codes(t):
    return t.view(torch.uint8).cpu().numpy()


def _same(got_q, got_s, want_q, want_s):
    """NaN codes wherever the oracle has NaN codes (the sign bit of a NaN is the platform's), every
    other code and every inverse scale bit for bit."""
    assert got_q.shape == want_q.shape and got_s.shape == want_s.shape and got_s.dtype == torch.float32
    got, want = _codes(got_q), _codes(want_q)
    want_nan = (want & 0x7F) == 0x7F
    assert np.array_equal((got & 0x7F) == 0x7F, want_nan)
    assert np.array_equal(got[~want_nan], want[~want_nan])
    gs, ws = got_s.cpu().numpy(), want_s.numpy()
    assert np.array_equal(np.isnan(gs), np.isnan(ws))
    assert np.array_equal(gs[~np.isnan(ws)].view(np.uint32), ws[~np.isnan(ws)].view(np.uint32))


# whole blocks, ragged edges, one row, K that leaves the 16-byte chunks (element-wise form), long and tall
SHAPES = [(128, 128), (256, 384), (1, 16), (130, 272), (300, 2048), (127, 144), (257, 129), (64, 4100), (1000, 520),
          (5, 3), (129, 130), (2048, 1024)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,k", SHAPES)
@pytest.mark.parametrize("sigma", [1.0, 0.02])
def test_block_quantiser_matches_the_oracle_bit_for_bit(gpu_device, m, k, sigma, dtype):
    print(f"case m={m} k={k} sigma={sigma} dtype={dtype}", flush=True)
    x = orc.randn_f32(m, k, sigma, seed=3 * m + k).to(dtype)
    want_q, want_s = orc.fp8_block_quantize(x)
    got_q, got_s = ops.fp8_block_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    _same(got_q, got_s, want_q, want_s)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_zero_tiny_nan_and_infinite_blocks(gpu_device, dtype):
    x = orc.randn_f32(384, 512, 1.0, seed=11).to(dtype)
    x[:128, :128] = 0.0                      # all-zero block: scale 448 / 1e-12 (in the source type), codes zero
    x[128:256, 128:256] *= 1e-30             # below the clamp: same scale, codes zero or subnormal
    x[200, 300] = float("nan")               # block (1, 2): NaN codes, NaN scale
    x[300, 10] = float("inf")                # block (2, 0): scale 0, finite -> 0, inf -> NaN
    x[300, 11] = float("-inf")
    x[383, 511] = 3e38                       # block (2, 3): huge but finite
    want_q, want_s = orc.fp8_block_quantize(x)
    got_q, got_s = ops.fp8_block_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    _same(got_q, got_s, want_q, want_s)
    s = got_s.cpu()
    assert torch.isnan(s[1, 2]) and torch.isinf(s[2, 0]) and s[2, 0] > 0
    q = got_q.cpu().float()
    assert torch.isnan(q[128:256, 256:384]).all()
    assert torch.isnan(q[300, 10]) and torch.isnan(q[300, 11]) and (q[256:384, :128][~torch.isnan(q[256:384, :128])] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("row_offset,col_offset,k", [(0, 0, 272), (0, 1, 272), (1, 0, 270), (0, 8, 264)])
def test_strided_source_and_guarded_destination(gpu_device, dtype, row_offset, col_offset, k):
    """Source rows out of a wider buffer (aligned and not), destination rows inside a canvas whose
    guard bytes must come back untouched: the vector and the element-wise form through the C ABI."""
    dev = gpu_device
    m = 200
    lib = _lib.load()
    big = orc.randn_f32(m + 2, 320, 1.0, seed=5).to(dtype)
    x = big[row_offset:row_offset + m, col_offset:col_offset + k]
    want_q, want_s = orc.fp8_block_quantize(x.contiguous())
    big_d = big.to(dev)
    xd = big_d[row_offset:row_offset + m, col_offset:col_offset + k]
    canvas = torch.full((m + 2, 336), 0x55, dtype=torch.uint8, device=dev)
    qd = canvas[1:m + 1, 16:16 + k]
    gm, gk = -(-m // 128), -(-k // 128)
    scales = torch.full((gm * gk + 2,), -7.0, dtype=torch.float32, device=dev)
    src = _lib.SRC_F32 if dtype == torch.float32 else _lib.SRC_BF16
    st = lib.mi355x_fp8_blockwise_quantize(xd.data_ptr(), src, qd.data_ptr(), scales[1:].data_ptr(), m, k, xd.stride(0),
                                           qd.stride(0), torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "mi355x_fp8_blockwise_quantize")
    torch.cuda.synchronize()
    assert np.array_equal(qd.cpu().numpy(), _codes(want_q))
    mask = torch.ones_like(canvas, dtype=torch.bool)
    mask[1:m + 1, 16:16 + k] = False
    assert torch.all(canvas[mask] == 0x55)
    assert scales[0].item() == -7.0 and scales[-1].item() == -7.0
    assert np.array_equal(scales[1:-1].cpu().numpy().view(np.uint32), want_s.reshape(-1).numpy().view(np.uint32))


def test_quantised_operands_feed_the_block_scaled_gemm(gpu_device):
    dev = gpu_device
    x = orc.randn_f32(300, 1040, 1.0, seed=1)
    w = orc.randn_f32(520, 1040, 1.0, seed=2)
    xq, xs = ops.fp8_block_quantize(x.to(dev))
    wq, ws = ops.fp8_block_quantize(w.to(dev))
    out = ops.fp8_gemm_blockwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    oxq, oxs = orc.fp8_block_quantize(x)
    owq, ows = orc.fp8_block_quantize(w)
    want = orc.blockwise_dequant_matmul(oxq, owq, oxs, ows)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-2, atol=1e-2)
    # and against the unquantised product: block quantisation costs a few per cent of the norm
    full = x @ w.T
    assert (out.cpu().float() - full).norm() / full.norm() < 0.06


def test_bad_arguments_are_refused(gpu_device):
    lib = _lib.load()
    x = torch.zeros((16, 16), device=gpu_device)
    q = torch.zeros((16, 16), dtype=torch.uint8, device=gpu_device)
    s = torch.zeros((1,), device=gpu_device)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.mi355x_fp8_blockwise_quantize(None, _lib.SRC_F32, q.data_ptr(), s.data_ptr(), 16, 16, 16, 16, stream) == _lib.EINVAL
    assert lib.mi355x_fp8_blockwise_quantize(x.data_ptr(), 9, q.data_ptr(), s.data_ptr(), 16, 16, 16, 16, stream) == _lib.EINVAL
    assert lib.mi355x_fp8_blockwise_quantize(x.data_ptr(), _lib.SRC_F32, q.data_ptr(), s.data_ptr(), 16, 16, 8, 16, stream) == _lib.EINVAL
    with pytest.raises(TypeError):
        ops.fp8_block_quantize(x.to(torch.float16))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fp8_block_quantize(torch.zeros(4, 4))
