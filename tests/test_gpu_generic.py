"""The generic kernel family (byte loads, f32 multiply-adds): operands the MFMA families cannot take
(K, lda or ldb not a multiple of 16, A or B not 16-byte aligned) against the CPU oracle, through
the C ABI. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to
ATOL = 1e-2


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _check_tight(out, xq, wq, xs, ws, bias):
    """Within 1 bf16 ulp of the float64 value plus the slack fp32 accumulation is entitled to."""
    a = e4m3.decode(xq.view(torch.uint8).numpy()).astype(np.float64)
    b = e4m3.decode(wq.view(torch.uint8).numpy()).astype(np.float64)
    sa, sb = xs.numpy().astype(np.float64)[:, None], ws.numpy().astype(np.float64)[None, :]
    exact = (a @ b.T) * sa * sb
    slack = (np.abs(a) @ np.abs(b).T) * sa * sb * a.shape[1] * 2.0 ** -24
    if bias is not None:
        exact = exact + bias.float().numpy().astype(np.float64)[None, :]
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** -126))) - 7)
    got = out.float().numpy().astype(np.float64)
    assert np.all(np.abs(got - exact) <= ulp + slack), f"max excess {np.max(np.abs(got - exact) - ulp - slack)}"


# K that is no multiple of 16 (down to 1), ragged M and N, one shape the MFMA families would take
SHAPES = [(5, 7, 3), (1, 1, 1), (64, 64, 17), (130, 70, 100), (33, 257, 1000), (16, 16, 16), (65, 129, 8), (300, 520, 1041),
          (2, 2000, 33)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("bias", [False, True])
def test_generic_family_against_the_oracle(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    dev = gpu_device
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    args = [t.to(dev) for t in (xq, wq, xs, ws)]
    bd = b.to(dev) if b is not None else None
    # K % 16 != 0: the automatic choice must land on the generic family by itself
    variants = [_lib.VARIANT_GENERIC] + ([_lib.VARIANT_AUTO] if k % 16 else [])
    for variant in variants:
        assert (_lib.load().mi355x_fp8_rowwise_select_variant(m, n, k) == _lib.VARIANT_GENERIC) == (k % 16 != 0)
        out = ops.fp8_gemm_rowwise(*args, bias=bd, variant=variant)
        torch.cuda.synchronize()
        torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
        _check_tight(out.cpu(), xq, wq, xs, ws, b)


def test_misaligned_and_oddly_strided_operands_go_to_the_generic_family(gpu_device):
    """A that starts one byte into its buffer, B with a row pitch of 49 bytes, K = 48: AUTO runs
    them (generic family); the MFMA families, pinned, say why they do not."""
    dev = gpu_device
    m, n, k = 40, 72, 48
    xq, wq, xs, ws, _ = orc.make_inputs(m, n, k, 1.0, False)
    want = orc.dequant_matmul(xq, wq, xs, ws, None)
    raw_a = torch.zeros(m * k + 16, dtype=torch.uint8, device=dev)
    raw_a[1:1 + m * k] = xq.view(torch.uint8).reshape(-1).to(dev)
    a_off = raw_a[1:1 + m * k].view(torch.float8_e4m3fn).reshape(m, k)          # misaligned base
    raw_b = torch.zeros((n, 49), dtype=torch.uint8, device=dev)
    raw_b[:, :k] = wq.view(torch.uint8).to(dev)
    b_odd = raw_b.view(torch.float8_e4m3fn)[:, :k]                              # ldb = 49
    a_ok, b_ok = xq.to(dev), wq.to(dev)
    for a, b in ((a_off, b_ok), (a_ok, b_odd), (a_off, b_odd)):
        out = ops.fp8_gemm_rowwise(a, b, xs.to(dev), ws.to(dev))
        torch.cuda.synchronize()
        torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
        for pinned, why in ((_lib.VARIANT_TILED, "aligned|multiples of 16"), (_lib.VARIANT_SKINNY, "aligned|multiples of 16")):
            with pytest.raises(NotImplementedError, match=why):
                ops.fp8_gemm_rowwise(a, b, xs.to(dev), ws.to(dev), variant=pinned)


def test_generic_family_is_bit_exact_on_small_integers_and_decodes_every_code(gpu_device):
    dev = gpu_device
    # integers: every partial sum is exact in f32, so the result must equal the MFMA families' bit for bit
    g = torch.Generator().manual_seed(7)
    a = torch.randint(-3, 4, (70, 160), generator=g).float()
    b = torch.randint(-3, 4, (90, 160), generator=g).float()
    xs, ws = torch.full((70,), 0.5), torch.full((90,), 2.0)
    aq, bq = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    outs = [ops.fp8_gemm_rowwise(aq.to(dev), bq.to(dev), xs.to(dev), ws.to(dev), variant=v).cpu()
            for v in (_lib.VARIANT_GENERIC, _lib.VARIANT_TILED)]
    assert np.array_equal(_bits(outs[0]), _bits(outs[1]))
    assert np.array_equal(_bits(outs[0]), orc.to_bf16_bits((a @ b.T).numpy().astype(np.float32)))
    # every code against 1.0 and against itself: the decode of all 256 codes (NaN, subnormals, -0 included)
    codes = torch.arange(256, dtype=torch.uint8)
    diag = torch.zeros((256, 256), dtype=torch.uint8)
    diag[codes.long(), codes.long()] = codes                                  # row i holds code i at column i
    one_hot = torch.zeros((256, 256), dtype=torch.uint8)
    one_hot[codes.long(), codes.long()] = 0x38                                # 1.0
    out = ops.fp8_gemm_rowwise(diag.view(torch.float8_e4m3fn).to(dev), one_hot.view(torch.float8_e4m3fn).to(dev),
                               torch.ones(256, device=dev), torch.ones(256, device=dev), variant=_lib.VARIANT_GENERIC).cpu().float()
    vals = e4m3.decode(codes.numpy()).astype(np.float32)
    got = torch.diagonal(out).numpy()
    finite = ~np.isnan(vals)
    assert np.array_equal(np.isnan(got), ~finite)
    assert np.array_equal(got[finite], vals[finite])                          # every finite e4m3fn value is a bf16


def test_generic_family_float16_output_and_graph_capture(gpu_device):
    dev = gpu_device
    xq, wq, xs, ws, b = orc.make_inputs(50, 70, 24, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    args = [t.to(dev) for t in (xq, wq, xs, ws)]
    bd = b.to(dev)
    out16 = ops.fp8_gemm_rowwise(*args, bias=bd, out_dtype=torch.float16)
    torch.testing.assert_close(out16.cpu().float(), want.float(), rtol=RTOL, atol=ATOL)
    out = torch.zeros((50, 70), dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.fp8_gemm_rowwise(*args, bias=bd, out=out)
        torch.cuda.synchronize()
        eager = out.clone()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            ops.fp8_gemm_rowwise(*args, bias=bd, out=out)
        for _ in range(3):
            out.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
    torch.testing.assert_close(eager.cpu(), want, rtol=RTOL, atol=ATOL)
