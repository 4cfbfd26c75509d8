"""Parity of the narrow-tile kernel (one workgroup per 32 or 64 columns of the output owns all of K,
in 512-byte steps of which the last may be partial; M <= 64, and up to 256 rows in row blocks of 64
where that is one workgroup per CU) with the CPU oracle, through the C ABI with the kernel pinned,
and that the automatic choice takes it where its cost estimate says so. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to: rtol 1e-2 / atol 1e-2 on the 16-bit output
ATOL = 1e-2

NARROW = _lib.VARIANT_SKINNY | _lib.SKINNY_NARROW


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


# m, n, k, bias. One and two 32-row blocks of A, full and ragged; N from a single ragged tile to more
# tiles than CUs (two rounds of workgroups), multiples of 32 and not, odd N (element-wise stores);
# K from one step (shorter than either prefetch distance) to 56 steps.
SHAPES = [
    (1, 1, 512, False), (17, 31, 512, True), (32, 32, 1024, False), (32, 40, 1536, True),
    (20, 999, 2048, True), (32, 8192, 4096, False), (31, 4100, 3072, True), (24, 8224, 2048, False),
    (33, 64, 512, True), (64, 8192, 2048, False), (50, 1000, 4096, True), (64, 33, 2560, False),
    (48, 2056, 8192, True), (32, 1024, 28672, False), (64, 520, 8192, True),
    # between one and two 32-column tiles per CU: 64-column tiles, with one and two blocks of A
    (32, 16384, 2048, True), (20, 10250, 1024, False), (7, 12288, 512, True), (32, 8224, 4096, False),
    (64, 16384, 1024, False), (40, 9001, 2560, True), (64, 8250, 512, True),
    # K not in whole 512-byte steps (a partial last step, down to a single 16-byte chunk), not in whole
    # 128-byte slabs either
    (32, 64, 528, True), (17, 100, 48, False), (3, 40, 16, True), (40, 1000, 4112, True), (64, 520, 2304, False), (9, 8192, 6672, True),
    (32, 10240, 1040, False),
    # row blocks (the workgroups of a tile side by side on one XCD) in every tile size: 32x32 tiles with
    # two to five blocks, 64x32 with two and four, 64x64 with two to four; ragged last row block (1, 4, 32
    # and 36 rows), ragged last tile, fewer tiles than XCDs, grids of exactly 256 workgroups, partial last
    # K step; and 64 rows in one block where two would be too many workgroups
    (65, 64, 512, True), (128, 8192, 1024, False), (100, 1000, 2048, True), (96, 4100, 1536, False),
    (256, 4096, 1024, True), (192, 5000, 512, False), (129, 200, 4112, True), (128, 7168, 2320, False),
    (128, 4096, 1024, True), (256, 2000, 528, False), (100, 3000, 1040, True), (64, 7000, 1024, True),
    (64, 4096, 1536, False),
]


@pytest.mark.parametrize("m,n,k,bias", SHAPES)
def test_narrow_kernel_against_oracle(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, NARROW)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)


@pytest.mark.parametrize("m,k", [(32, 512), (19, 2048), (64, 4096), (40, 8192), (32, 2320), (120, 2048), (190, 1040)])
def test_exact_integer_case_is_bit_exact(gpu_device, m, k):
    # small integers, unit scales: every partial sum stays below 2^24, so fp32 summation is exact in
    # any order (four waves' partial sums, rotated K order) and the float64 result must come out bit for bit
    rng = np.random.default_rng(23)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4, 0.5, -0.5], dtype=np.float32)
    n = 4130
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    xq, wq = torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn)
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    out = _run(gpu_device, xq, wq, torch.ones(m), torch.ones(n), None, NARROW)
    assert np.array_equal(_bits(out), want)


def test_one_hot_positions_walk_every_k_byte_and_tile(gpu_device):
    # A[i, ka(i)] = 1 and B[j, kb(j)] = 1: C[i, j] = [ka(i) == kb(j)]. The positions walk all steps,
    # slabs and bytes of a slab, so a wrong rotation, slab assignment, swizzle or tile offset shows as
    # a misplaced one.
    m, n, k = 64, 2080, 8192
    ka = (np.arange(m) * 517 + 5) % k
    kb = (np.arange(n) * 131 + 2) % k
    kb[: m * 8] = np.repeat(ka, 8)  # guaranteed hits in the first tiles
    a = np.zeros((m, k), np.float32)
    b = np.zeros((n, k), np.float32)
    a[np.arange(m), ka] = 1.0
    b[np.arange(n), kb] = 1.0
    out = _run(gpu_device, torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn),
               torch.ones(m), torch.ones(n), None, NARROW)
    want = (ka[:, None] == kb[None, :]).astype(np.float32)
    assert want.sum() >= m * 8
    assert np.array_equal(out.float().numpy(), want)


def test_padded_operands_unaligned_output_and_canaries(gpu_device):
    # rows padded past K with garbage (448 / -448), output embedded in a larger buffer at an odd column,
    # scale and bias vectors that start 4 and 2 bytes into their allocations
    m, n, k, pad = 37, 1030, 2048, 64
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    a_buf = torch.full((m, k + pad), 0x7E, dtype=torch.uint8, device=dev)
    b_buf = torch.full((n, k + pad), 0xFE, dtype=torch.uint8, device=dev)
    a_buf[:, :k] = xq.view(torch.uint8).to(dev)
    b_buf[:, :k] = wq.view(torch.uint8).to(dev)
    ws_buf = torch.zeros(n + 1, dtype=torch.float32, device=dev)
    ws_buf[1:] = ws.to(dev)
    bias_buf = torch.zeros(n + 1, dtype=torch.bfloat16, device=dev)
    bias_buf[1:] = b.to(dev)
    c_buf = torch.full((m + 2, n + 25), -77.0, dtype=torch.bfloat16, device=dev)
    c_view = c_buf[1:m + 1, 7:7 + n]
    ops.fp8_gemm_rowwise(a_buf.view(torch.float8_e4m3fn)[:, :k], b_buf.view(torch.float8_e4m3fn)[:, :k],
                         xs.to(dev), ws_buf[1:], bias=bias_buf[1:], out=c_view, variant=NARROW)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=RTOL, atol=ATOL)
    _check_tight(c_view.cpu(), xq, wq, xs, ws, b)
    mask = torch.ones_like(c_buf, dtype=torch.bool)
    mask[1:m + 1, 7:7 + n] = False
    assert torch.all(c_buf[mask] == -77.0)


def test_float16_output_and_fused_bias_rounding(gpu_device):
    m, n, k = 40, 512, 2048
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b).float()
    out = _run(gpu_device, xq, wq, xs, ws, b, NARROW, out_dtype=torch.float16)
    assert out.dtype == torch.float16
    torch.testing.assert_close(out.float(), want, rtol=RTOL, atol=ATOL)
    # bias joins before the one rounding: 1.00390625 + 2^-8 = 1.0078125 exactly in bf16; rounding
    # the product first would give 1.0 + 2^-8 -> 1.0
    a = torch.zeros(32, 512)
    a[0, 0] = 1.0
    w = torch.zeros(32, 512)
    w[0, 0] = 1.0
    xs1 = torch.ones(32)
    xs1[0] = 1.00390625
    bias = torch.zeros(32)
    bias[0] = 2.0 ** -8
    out = _run(gpu_device, a.to(torch.float8_e4m3fn), w.to(torch.float8_e4m3fn), xs1, torch.ones(32),
               bias.to(torch.bfloat16), NARROW)
    assert out[0, 0].item() == 1.0078125


def test_graph_capture_replays_match_eager(gpu_device):
    dev = gpu_device
    m, n, k = 32, 8192, 4096
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    dxq, dwq, dxs, dws, db = (t.to(dev) for t in (xq, wq, xs, ws, b))
    eager = ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, variant=NARROW)
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, out=out, variant=NARROW)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, out=out, variant=NARROW)
    for _ in range(3):
        out.fill_(0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_one_hot_positions_with_row_blocks(gpu_device):
    # the same walk with three row blocks and 40 tiles (five rounds of the XCDs): a wrong row-block or
    # tile assignment of a workgroup shows as a misplaced one
    m, n, k = 150, 2500, 4096
    ka = (np.arange(m) * 517 + 5) % k
    kb = (np.arange(n) * 131 + 2) % k
    kb[: m * 8] = np.repeat(ka, 8)
    a = np.zeros((m, k), np.float32)
    b = np.zeros((n, k), np.float32)
    a[np.arange(m), ka] = 1.0
    b[np.arange(n), kb] = 1.0
    out = _run(gpu_device, torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn),
               torch.ones(m), torch.ones(n), None, NARROW)
    want = (ka[:, None] == kb[None, :]).astype(np.float32)
    assert np.array_equal(out.float().numpy(), want)


def test_row_blocks_keep_to_their_rows_of_an_embedded_output(gpu_device):
    m, n, k = 130, 700, 1024
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    c_buf = torch.full((m + 2, n + 25), -77.0, dtype=torch.bfloat16, device=dev)
    c_view = c_buf[1:m + 1, 7:7 + n]
    ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), bias=b.to(dev), out=c_view, variant=NARROW)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=RTOL, atol=ATOL)
    mask = torch.ones_like(c_buf, dtype=torch.bool)
    mask[1:m + 1, 7:7 + n] = False
    assert torch.all(c_buf[mask] == -77.0)


def test_shapes_the_kernel_does_not_take_are_refused(gpu_device):
    # more than 64 rows are taken only where 64x64 tiles give every CU at most one workgroup
    for m, n in ((257, 64), (128, 8200), (256, 4160), (65, 16384)):
        assert not _lib.skinny_family_takes(m, n)
        xq, wq, xs, ws, _ = orc.make_inputs(m, n, 512, 1.0, False)
        with pytest.raises(NotImplementedError):
            _run(gpu_device, xq, wq, xs, ws, None, NARROW)
        with pytest.raises(NotImplementedError):
            _run(gpu_device, xq, wq, xs, ws, None, _lib.VARIANT_SKINNY)


def test_other_pins_of_the_family_stop_at_64_rows(gpu_device):
    xq, wq, xs, ws, _ = orc.make_inputs(100, 64, 512, 1.0, False)
    with pytest.raises(NotImplementedError):
        _run(gpu_device, xq, wq, xs, ws, None, _lib.VARIANT_SKINNY | _lib.SKINNY_ONE_TILE)
    want = orc.dequant_matmul(xq, wq, xs, ws, None)
    out = _run(gpu_device, xq, wq, xs, ws, None, _lib.VARIANT_SKINNY)  # unpinned: the narrow-tile form in row blocks
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)


def test_automatic_choice_runs_it_where_it_is_expected_to_win(gpu_device):
    # 32 x 8192 x 8192: one tile per CU, two blocks of A rows more than the persistent kernel keeps
    assert ops.select_variant(32, 8192, 8192) == _lib.VARIANT_SKINNY
    assert _lib.load().mi355x_fp8_rowwise_workspace_bytes(32, 8192, 8192, _lib.VARIANT_AUTO) == 0
    m, n, k = 32, 8192, 8192
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 0.02, False)
    auto = _run(gpu_device, xq, wq, xs, ws, b, _lib.VARIANT_AUTO)
    pinned = _run(gpu_device, xq, wq, xs, ws, b, NARROW)
    assert torch.equal(auto, pinned)  # the same kernel: bit-identical
    # 128 x 8192 x 8192: two row blocks, 256 workgroups, no partial sums in a workspace
    assert ops.select_variant(128, 8192, 8192) == _lib.VARIANT_SKINNY
    assert _lib.load().mi355x_fp8_rowwise_workspace_bytes(128, 8192, 8192, _lib.VARIANT_AUTO) == 0
    assert ops.select_variant(128, 10240, 8192) == _lib.VARIANT_TILED
    xq, wq, xs, ws, b = orc.make_inputs(128, 8192, 2048, 0.02, True)
    assert ops.select_variant(128, 8192, 2048) == _lib.VARIANT_SKINNY
    auto = _run(gpu_device, xq, wq, xs, ws, b, _lib.VARIANT_AUTO)
    pinned = _run(gpu_device, xq, wq, xs, ws, b, NARROW)
    assert torch.equal(auto, pinned)
