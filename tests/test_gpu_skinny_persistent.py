"""Parity of the skinny kernels that keep A on chip (N % 16 == 0) with the CPU oracle, and against
the one-tile-per-workgroup kernel they replace on their shapes: the pair kernel (M <= 16, N <= 8192,
any K <= 8192: at most two tiles of B per CU, A parked in LDS) and the persistent kernel (M <= 16
with larger N and K in {2048, 4096, 6144, 8192}; M <= 32 with K = 4096: two 16-row blocks of A
resident in registers). All are reached through the C ABI with the skinny family and the form
pinned. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to: rtol 1e-2 / atol 1e-2 on the bf16 output
ATOL = 1e-2

PERSISTENT = _lib.VARIANT_SKINNY | _lib.SKINNY_RESIDENT  # pair or persistent kernel, whichever takes the shape
ONE_TILE = _lib.VARIANT_SKINNY | _lib.SKINNY_ONE_TILE


def _codes(t):
    return t.view(torch.uint8).cpu().numpy()


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _ulp_bf16(x):
    x = np.maximum(np.abs(x), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(x)) - 7)


def _check_tight(out, xq, wq, xs, ws, bias):
    """Within 1 bf16 ulp of the exact (float64) value plus the slack any fp32 summation order
    is entitled to."""
    exact = orc.gemm_f64(_codes(xq), _codes(wq), xs.numpy(), ws.numpy(), _bits(bias) if bias is not None else None)
    a = np.abs(e4m3.decode(_codes(xq)).astype(np.float64))
    b = np.abs(e4m3.decode(_codes(wq)).astype(np.float64))
    slack = (a @ b.T) * xs.numpy().astype(np.float64)[:, None] * ws.numpy().astype(np.float64)[None, :] * a.shape[1] * 2.0 ** -24
    err = np.abs(out.float().numpy().astype(np.float64) - exact)
    assert np.all(err <= 1.0 * _ulp_bf16(exact) + slack), f"max excess {np.max(err - _ulp_bf16(exact) - slack)}"


def _run(dev, xq, wq, xs, ws, bias, variant, **kw):
    d = lambda t: None if t is None else t.to(dev)
    out = ops.fp8_gemm_rowwise(d(xq), d(wq), d(xs), d(ws), bias=d(bias), variant=variant, **kw)
    torch.cuda.synchronize()
    return out.cpu()


# m, n, k, bias: every K the kernel takes (1..4 steps per wave); N from one tile to a few more
# tiles than workgroups (256): runs of 1, 2 and 3 tiles, with and without idle workgroups
SHAPES = [
    (1, 16, 2048, False), (16, 16, 8192, True), (7, 48, 4096, True), (16, 4096, 2048, False),
    (9, 4112, 6144, True), (16, 8192, 4096, False), (3, 8208, 2048, True), (16, 10240, 2048, True),
    (13, 2064, 8192, False), (16, 12304, 2048, False),
    # beyond the pair kernel's two tiles per CU: the persistent kernel with one block of A
    (9, 8208, 6144, True), (16, 16400, 8192, False), (5, 12304, 4096, True), (16, 20480, 6144, False),
    # two blocks of A (M = 17..32, K = 4096): last block full / one row / ragged
    (17, 16, 4096, True), (32, 8192, 4096, False), (25, 4112, 4096, True), (32, 10240, 4096, False),
    (20, 2064, 4096, True), (31, 12304, 4096, False),
]


@pytest.mark.parametrize("m,n,k,bias", SHAPES)
def test_persistent_kernel_against_oracle(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    if m <= 16:
        assert ops.select_variant(m, n, k) == _lib.VARIANT_SKINNY  # the family the automatic choice runs too
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, PERSISTENT)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)
    # the general kernel on the same operands: same tolerance, different summation order
    other = _run(gpu_device, xq, wq, xs, ws, b, ONE_TILE)
    torch.testing.assert_close(other, want, rtol=RTOL, atol=ATOL)
    _check_tight(other, xq, wq, xs, ws, b)


# m, n, k, bias for the pair kernel: K that is no multiple of 2048, of 128 (a partial last step down to one
# 16-byte chunk), shorter than one step per wave (waves without any step), one to four steps per
# wave; one tile, fewer tiles than CUs, exactly one and two per CU, one more than one per CU
PAIR_SHAPES = [
    (1, 16, 16, False), (16, 16, 144, True), (3, 48, 272, True), (16, 4096, 2304, False), (4, 4096, 2304, True),
    (8, 2304, 2304, False), (16, 4096, 6656, True), (8, 8192, 6656, False), (1, 2304, 2048, True),
    (16, 4112, 4112, True), (11, 8192, 8176, False), (16, 8192, 8192, True), (7, 8176, 2064, False),
    (16, 512, 1040, True), (2, 8192, 128, False), (16, 6400, 5136, True),
]


@pytest.mark.parametrize("m,n,k,bias", PAIR_SHAPES)
def test_pair_kernel_against_oracle(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, PERSISTENT)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)
    other = _run(gpu_device, xq, wq, xs, ws, b, ONE_TILE)
    torch.testing.assert_close(other, out, rtol=RTOL, atol=ATOL)


def test_resident_pin_refuses_what_neither_form_takes(gpu_device):
    dev = gpu_device
    for (m, n, k) in [(17, 4096, 2048), (16, 4104, 4096), (16, 16384, 2304), (8, 4096, 8208)]:
        xq, wq, xs, ws, _ = orc.make_inputs(m, n, k, 1.0, False)
        with pytest.raises(NotImplementedError):
            ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), variant=PERSISTENT)


def test_pair_kernel_ignores_what_lies_past_k(gpu_device):
    # K = 2320 (18 whole steps and a 16-byte chunk): rows padded to 2560 bytes with codes of +-448 that must
    # not enter any sum, neither through the partial step nor through the steps past it
    m, n, k, ld = 16, 4096, 2320, 2560
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    a_buf = torch.full((m, ld), 0x7E, dtype=torch.uint8, device=dev)
    b_buf = torch.full((n, ld), 0xFE, dtype=torch.uint8, device=dev)
    a_buf[:, :k] = xq.view(torch.uint8).to(dev)
    b_buf[:, :k] = wq.view(torch.uint8).to(dev)
    out = ops.fp8_gemm_rowwise(a_buf.view(torch.float8_e4m3fn)[:, :k], b_buf.view(torch.float8_e4m3fn)[:, :k],
                               xs.to(dev), ws.to(dev), bias=b.to(dev), variant=PERSISTENT)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    _check_tight(out.cpu(), xq, wq, xs, ws, b)


@pytest.mark.parametrize("m,k", [(16, 2048), (5, 8192), (32, 4096), (19, 4096), (16, 6656), (9, 2320)])
def test_exact_integer_case_is_bit_exact(gpu_device, m, k):
    # small integers, unit scales: every partial sum stays below 2^24, so fp32 summation is
    # exact in any order and both kernels must reproduce the float64 result bit for bit
    rng = np.random.default_rng(21)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4, 0.5, -0.5], dtype=np.float32)
    n = 4128
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    xq, wq = torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn)
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    for variant in (PERSISTENT, ONE_TILE):
        out = _run(gpu_device, xq, wq, torch.ones(m), torch.ones(n), None, variant)
        assert np.array_equal(_bits(out), want)


@pytest.mark.parametrize("n,k", [(4112, 8192), (8192, 6656), (12304, 8192), (4096, 2320)])
def test_one_hot_positions_walk_every_k_step_and_tile(gpu_device, n, k):
    # A[i, ka(i)] = 1 and B[j, kb(j)] = 1: C[i, j] = [ka(i) == kb(j)]. The positions walk all
    # K steps and every byte of a step, so a wrong step rotation, lane layout or tile offset
    # shows as a misplaced one. (N <= 8192: the pair kernel; beyond: the persistent kernel.)
    m = 16
    ka = (np.arange(m) * 517 + 5) % k
    kb = (np.arange(n) * 131 + 2) % k
    kb[: m * 8] = np.repeat(ka, 8)  # guaranteed hits in the first tiles
    a = np.zeros((m, k), np.float32)
    b = np.zeros((n, k), np.float32)
    a[np.arange(m), ka] = 1.0
    b[np.arange(n), kb] = 1.0
    out = _run(gpu_device, torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn),
               torch.ones(m), torch.ones(n), None, PERSISTENT)
    want = (ka[:, None] == kb[None, :]).astype(np.float32)
    assert want.sum() >= m * 8
    assert np.array_equal(out.float().numpy(), want)


def test_padded_operands_unaligned_epilogue_and_canaries(gpu_device):
    # rows padded past K with garbage, output embedded in a larger buffer at an odd column, scale
    # and bias vectors that start 4 and 2 bytes into their allocations: the scalar epilogue
    m, n, k, pad = 11, 2064, 4096, 64
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    a_buf = torch.full((m, k + pad), 0x7E, dtype=torch.uint8, device=dev)  # 448 everywhere
    b_buf = torch.full((n, k + pad), 0xFE, dtype=torch.uint8, device=dev)  # -448 everywhere
    a_buf[:, :k] = xq.view(torch.uint8).to(dev)
    b_buf[:, :k] = wq.view(torch.uint8).to(dev)
    ws_buf = torch.zeros(n + 1, dtype=torch.float32, device=dev)
    ws_buf[1:] = ws.to(dev)
    bias_buf = torch.zeros(n + 1, dtype=torch.bfloat16, device=dev)
    bias_buf[1:] = b.to(dev)
    c_buf = torch.full((m + 2, n + 25), -77.0, dtype=torch.bfloat16, device=dev)
    c_view = c_buf[1:m + 1, 7:7 + n]
    for variant in (PERSISTENT, ONE_TILE):
        c_buf.fill_(-77.0)
        ops.fp8_gemm_rowwise(a_buf.view(torch.float8_e4m3fn)[:, :k], b_buf.view(torch.float8_e4m3fn)[:, :k],
                             xs.to(dev), ws_buf[1:], bias=bias_buf[1:], out=c_view, variant=variant)
        torch.cuda.synchronize()
        torch.testing.assert_close(c_view.cpu(), want, rtol=RTOL, atol=ATOL)
        _check_tight(c_view.cpu(), xq, wq, xs, ws, b)
        mask = torch.ones_like(c_buf, dtype=torch.bool)
        mask[1:m + 1, 7:7 + n] = False
        assert torch.all(c_buf[mask] == -77.0)


def test_float16_output_and_fused_bias_rounding(gpu_device):
    m, n, k = 16, 512, 2048
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b).float()
    out = _run(gpu_device, xq, wq, xs, ws, b, PERSISTENT, out_dtype=torch.float16)
    assert out.dtype == torch.float16
    torch.testing.assert_close(out.float(), want, rtol=RTOL, atol=ATOL)
    # bias joins before the one rounding: 1.00390625 + 2^-8 = 1.0078125 exactly in bf16; rounding
    # the product first would give 1.0 + 2^-8 -> 1.0
    a = torch.zeros(16, 2048)
    a[0, 0] = 1.0
    w = torch.zeros(16, 2048)
    w[0, 0] = 1.0
    xs1 = torch.ones(16)
    xs1[0] = 1.00390625
    bias = torch.zeros(16)
    bias[0] = 2.0 ** -8
    out = _run(gpu_device, a.to(torch.float8_e4m3fn), w.to(torch.float8_e4m3fn), xs1, torch.ones(16),
               bias.to(torch.bfloat16), PERSISTENT)
    assert out[0, 0].item() == 1.0078125


def test_graph_capture_replays_match_eager(gpu_device):
    dev = gpu_device
    m, n, k = 16, 8192, 4096
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    dxq, dwq, dxs, dws, db = (t.to(dev) for t in (xq, wq, xs, ws, b))
    eager = ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db)
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, out=out)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for _ in range(3):
                ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, out=out)
        for _ in range(3):
            out.fill_(-5.0)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)


def test_full_size_decode_shapes(gpu_device):
    # the benchmark's decode shapes at full size, sampled rows against the oracle
    for (m, n, k, sigma) in [(16, 8192, 8192, 1.0), (1, 10240, 8192, 0.02), (1, 57344, 8192, 0.02)]:
        print(f"full size m={m} n={n} k={k}", flush=True)
        xq, wq, xs, ws, _ = orc.make_inputs(m, n, k, sigma, False)
        out = _run(gpu_device, xq, wq, xs, ws, None, _lib.VARIANT_AUTO)
        cols = torch.randint(0, n, (512,), generator=torch.Generator().manual_seed(5))
        cols[:16] = torch.arange(n - 16, n)
        want = orc.dequant_matmul(xq, wq[cols], xs, ws[cols], None)
        torch.testing.assert_close(out[:, cols], want, rtol=RTOL, atol=ATOL)
        _check_tight(out[:, cols], xq, wq[cols], xs, ws[cols], None)
