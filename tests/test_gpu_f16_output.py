"""float16 output and the tensor-wise scaled form (through the C ABI) against the CPU oracle.
Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to
ATOL = 1e-2


def _tight_f16(out, xq, wq, xs, ws, bias):
    """Within 1 float16 ulp of the float64 value plus fp32 accumulation slack."""
    a = e4m3.decode(xq.view(torch.uint8).numpy()).astype(np.float64)
    b = e4m3.decode(wq.view(torch.uint8).numpy()).astype(np.float64)
    sa, sb = xs.numpy().astype(np.float64), ws.numpy().astype(np.float64)
    exact = (a @ b.T) * sa[:, None] * sb[None, :]
    if bias is not None:
        exact = exact + bias.float().numpy().astype(np.float64)[None, :]
    slack = (np.abs(a) @ np.abs(b).T) * sa[:, None] * sb[None, :] * a.shape[1] * 2.0 ** -24
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** -14))) - 10)  # subnormal spacing below 2^-14
    got = out.float().numpy().astype(np.float64)
    assert np.all(np.abs(got - exact) <= ulp + slack)


SHAPES = [(1, 16, 16, False), (16, 512, 1024, True), (33, 65, 272, True), (64, 1000, 1168, False), (130, 260, 128, True),
          (300, 520, 1040, False), (512, 768, 1024, True), (1000, 3000, 4112, True)]


@pytest.mark.parametrize("m,n,k,bias", SHAPES)
def test_f16_output_every_family(gpu_device, m, n, k, bias):
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 0.25, bias)  # sigma 0.25 keeps |C| inside the float16 range
    want = orc.dequant_matmul(xq, wq, xs, ws, b, out_dtype=torch.float16)
    dev = gpu_device
    d = [None if t is None else t.to(dev) for t in (xq, wq, xs, ws, b)]
    variants = [_lib.VARIANT_AUTO] + ([_lib.VARIANT_SKINNY] if _lib.skinny_family_takes(m, n) else [])
    variants += [_lib.tiled_variant(cfg, s) for cfg in range(_lib.NUM_TILE_CONFIGS) for s in (1, 3)]
    for variant in variants:
        print(f"case m={m} n={n} k={k} bias={bias} variant={variant:#x}", flush=True)
        out = ops.fp8_gemm_rowwise(d[0], d[1], d[2], d[3], bias=d[4], variant=variant, out_dtype=torch.float16)
        torch.cuda.synchronize()
        assert out.dtype == torch.float16
        torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
        _tight_f16(out.cpu(), xq, wq, xs, ws, b)


def test_f16_rounding_and_overflow(gpu_device):
    # one product per output: C = a * b * scale exactly representable in fp32, so the float16
    # result must be the correctly rounded one, ties to even, infinity past 65504
    vals = torch.tensor([1.0, 1.5, 0.0625, 448.0, -448.0, 3.0, -0.001953125, 0.0])
    m, n, k = len(vals), 4, 16
    a = torch.zeros(m, k)
    a[:, 0] = vals
    b = torch.zeros(n, k)
    b[:, 0] = torch.tensor([1.0, 448.0, -1.0, 0.5])
    xs = torch.tensor([1.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0, 1.0, 2.0 ** -24, 1.0, 1.0])
    ws = torch.ones(n)
    xq, wq = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    want = ((xq.float() @ wq.float().t()) * xs[:, None] * ws[None, :]).to(torch.float16)
    assert torch.isinf(want[3, 1]) and torch.isinf(want[4, 1])  # 448 * 448 = 200704 > 65504
    for variant in (_lib.VARIANT_SKINNY, _lib.tiled_variant(1, 1)):
        out = ops.fp8_gemm_rowwise(xq.to(gpu_device), wq.to(gpu_device), xs.to(gpu_device), ws.to(gpu_device),
                                   variant=variant, out_dtype=torch.float16).cpu()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_bf16_entry_point_is_unchanged_by_the_extended_one(gpu_device):
    dev = gpu_device
    xq, wq, xs, ws, b = (t.to(dev) for t in orc.make_inputs(200, 300, 528, 1.0, True))
    lib = _lib.load()
    out_a = torch.empty((200, 300), dtype=torch.bfloat16, device=dev)
    out_b = torch.empty_like(out_a)
    st = torch.cuda.current_stream().cuda_stream
    args = (xq.data_ptr(), wq.data_ptr(), xs.data_ptr(), ws.data_ptr(), b.data_ptr())
    assert lib.mi355x_fp8_rowwise_gemm(*args, out_a.data_ptr(), 200, 300, 528, 528, 528, 300, None, 0, 0, st) == 0
    assert lib.mi355x_fp8_rowwise_gemm_ex(*args, out_b.data_ptr(), _lib.OUT_BF16, 200, 300, 528, 528, 528, 300, None, 0, 0, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b)
    assert lib.mi355x_fp8_rowwise_gemm_ex(*args, out_b.data_ptr(), 7, 200, 300, 528, 528, 528, 300, None, 0, 0, st) == _lib.EINVAL


@pytest.mark.parametrize("m,n,k", [(128, 256, 512), (1024, 1280, 1024), (16, 2048, 2048)])
def test_tensorwise_form_matches_oracle_and_scaled_mm(gpu_device, m, n, k):
    # operands as the reference's fp8_gemm operator makes them: randn cast to fp8, b column-major, scalar scales
    dev = gpu_device
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.float8_e4m3fn)
    bt = torch.randn(n, k, generator=g).to(torch.float8_e4m3fn)  # = b.T, K-contiguous
    sa, sb = torch.tensor(0.5), torch.tensor(0.125)
    want = orc.dequant_matmul(a, bt, sa.expand(m), sb.expand(n), out_dtype=torch.float16)
    da, db = a.to(dev), bt.to(dev).t()  # [K, N] column-major view
    fn = ops.fp8_gemm_tensorwise(da, db, sa.to(dev), sb.to(dev))
    out = fn()
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and tuple(out.shape) == (m, n)
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    _tight_f16(out.cpu(), a, bt, sa.expand(m).contiguous(), sb.expand(n).contiguous(), None)
    try:
        lib_out = torch._scaled_mm(da, db, sa.to(dev), sb.to(dev), out_dtype=torch.float16)
    except Exception as e:  # the vendor path is a cross-check, not a requirement
        pytest.skip(f"torch._scaled_mm tensor-wise float16 not available here: {e}")
    torch.testing.assert_close(out, lib_out, rtol=RTOL, atol=ATOL)
