"""Parity of the HIP path (through the C ABI) with the CPU oracle. Needs an MI355X."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
RTOL = 1e-2  # the tolerance the path is specified to: rtol 1e-2 / atol 1e-2 on the bf16 output
ATOL = 1e-2


def _codes(t):
    return t.view(torch.uint8).cpu().numpy()


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _ulp_bf16(x):
    x = np.maximum(np.abs(x), 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(x)) - 7)


def _run(dev, xq, wq, xs, ws, bias=None, variant=_lib.VARIANT_AUTO):
    d = lambda t: None if t is None else t.to(dev)
    out = ops.fp8_gemm_rowwise(d(xq), d(wq), d(xs), d(ws), bias=d(bias), variant=variant)
    torch.cuda.synchronize()
    return out.cpu()


def _check_tight(out, xq, wq, xs, ws, bias):
    """Beyond rtol/atol: within 1 bf16 ulp of the exact (float64) value plus the slack any
    fp32 accumulation order is entitled to. Keeps parity meaningful when |C| << atol."""
    exact = orc.gemm_f64(_codes(xq), _codes(wq), xs.numpy(), ws.numpy(), _bits(bias) if bias is not None else None)
    a = np.abs(e4m3.decode(_codes(xq)).astype(np.float64))
    b = np.abs(e4m3.decode(_codes(wq)).astype(np.float64))
    slack = (a @ b.T) * xs.numpy().astype(np.float64)[:, None] * ws.numpy().astype(np.float64)[None, :] * a.shape[1] * 2.0 ** -24
    got = out.float().numpy().astype(np.float64)
    err = np.abs(got - exact)
    assert np.all(err <= 1.0 * _ulp_bf16(exact) + slack), f"max excess {np.max(err - _ulp_bf16(exact) - slack)}"


VARIANTS = [_lib.VARIANT_AUTO, _lib.VARIANT_TILED, _lib.VARIANT_SKINNY]


def test_golden_fixtures(gpu_device):
    with open(os.path.join(GOLDEN, "manifest.json")) as f:
        manifest = json.load(f)
    for case in manifest["cases"]:
        z = np.load(os.path.join(GOLDEN, case["file"]), allow_pickle=False)
        xq = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
        wq = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn)
        xs, ws = torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"])
        bias = torch.from_numpy(z["bias"].view(np.int16)).view(torch.bfloat16) if case["bias"] else None
        want = torch.from_numpy(z["c"].view(np.int16)).view(torch.bfloat16)
        for variant in VARIANTS:
            if variant == _lib.VARIANT_SKINNY and not _lib.skinny_family_takes(case["m"], case["n"]):
                continue
            print(f"golden {case['name']} variant {variant}", flush=True)
            out = _run(gpu_device, xq, wq, xs, ws, bias, variant)
            torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
            _check_tight(out, xq, wq, xs, ws, bias)


SMALL_SHAPES = [
    # m, n, k, bias
    (1, 1, 16, False), (1, 16, 16, True), (3, 5, 32, True), (16, 16, 128, False), (17, 33, 272, True),
    (33, 17, 144, False), (64, 64, 64, True), (65, 63, 80, True), (100, 300, 1040, False),
    (128, 256, 512, False), (255, 257, 384, True), (256, 256, 128, False), (257, 511, 4112, True),
    (300, 200, 2048, False), (512, 768, 1024, True),
]


@pytest.mark.parametrize("m,n,k,bias", SMALL_SHAPES)
@pytest.mark.parametrize("variant", VARIANTS)
def test_seeded_shapes_against_oracle(gpu_device, m, n, k, bias, variant):
    if variant == _lib.VARIANT_SKINNY and not _lib.skinny_family_takes(m, n):
        pytest.skip("the skinny family does not take this shape")
    print(f"case m={m} n={n} k={k} bias={bias} variant={variant}", flush=True)
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, variant)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)


PLAN_SHAPES = [
    # m, n, k, bias: ragged edges in both tile sizes, K tails, K shorter than the split count
    (130, 260, 128, True), (257, 129, 1040, False), (300, 520, 2048, True), (127, 1000, 4112, True),
    (512, 384, 640, False),
    # many more tile columns than K steps: every start position of the rotated K order, tail step included
    (100, 4000, 272, True),
]


@pytest.mark.parametrize("m,n,k,bias", PLAN_SHAPES)
@pytest.mark.parametrize("config", range(_lib.NUM_TILE_CONFIGS))
@pytest.mark.parametrize("splits", [1, 2, 3, 5, 16])
def test_every_tile_config_and_split_factor(gpu_device, m, n, k, bias, config, splits):
    print(f"case m={m} n={n} k={k} bias={bias} config={config} splits={splits}", flush=True)
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, _lib.tiled_variant(config, splits))
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)


@pytest.mark.parametrize("config", range(_lib.NUM_TILE_CONFIGS))
def test_split_k_exact_integer_case_is_bit_exact(gpu_device, config):
    # as test_exact_integer_case_is_bit_exact, with the sum cut into 4 partial sums that meet
    # in the finalize kernel; the output sits inside a larger buffer guarded by canaries
    rng = np.random.default_rng(12)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4, 0.5, -0.5], dtype=np.float32)
    m, n, k = 200, 391, 1296
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    dev = gpu_device
    c_buf = torch.full((m + 2, n + 9), -77.0, dtype=torch.bfloat16, device=dev)
    c_view = c_buf[1:m + 1, 3:3 + n]
    ops.fp8_gemm_rowwise(torch.from_numpy(a).to(torch.float8_e4m3fn).to(dev), torch.from_numpy(b).to(torch.float8_e4m3fn).to(dev),
                         torch.ones(m, device=dev), torch.ones(n, device=dev), out=c_view,
                         variant=_lib.tiled_variant(config, 4))
    torch.cuda.synchronize()
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(_bits(c_view.contiguous()), want)
    mask = torch.ones_like(c_buf, dtype=torch.bool)
    mask[1:m + 1, 3:3 + n] = False
    assert torch.all(c_buf[mask] == -77.0)


def test_workspace_rules(gpu_device):
    dev = gpu_device
    lib = _lib.load()
    m, n, k = 300, 2048, 8192
    xq, wq, xs, ws, _ = orc.make_inputs(m, n, k, 1.0, False)
    dxq, dwq, dxs, dws = (t.to(dev) for t in (xq, wq, xs, ws))
    want = orc.dequant_matmul(xq, wq, xs, ws, None)
    auto = _lib.VARIANT_AUTO
    need = lib.mi355x_fp8_rowwise_workspace_bytes(m, n, k, auto)
    assert need > 0 and need % (m * n * 4) == 0  # few tiles, long K: the library splits K
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)

    def call(variant, wsp, wsp_bytes):
        return lib.mi355x_fp8_rowwise_gemm(dxq.data_ptr(), dwq.data_ptr(), dxs.data_ptr(), dws.data_ptr(), None,
                                           out.data_ptr(), m, n, k, k, k, n, wsp, wsp_bytes, variant,
                                           torch.cuda.current_stream().cuda_stream)

    # automatic plan without workspace: runs a plan that needs none
    out.fill_(-3.0)
    assert call(auto, None, 0) == _lib.OK
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    # pinned split factor without enough workspace: refused, nothing launched
    buf = torch.empty(need, dtype=torch.uint8, device=dev)
    out.fill_(-3.0)
    assert call(_lib.tiled_variant(None, 4), buf.data_ptr(), m * n * 4) == _lib.EINVAL
    assert b"workspace" in lib.mi355x_fp8_rowwise_last_error()
    torch.cuda.synchronize()
    assert torch.all(out == -3.0)
    # with the workspace: the split plan
    assert call(auto, buf.data_ptr(), need) == _lib.OK
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("m", [1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64])
def test_skinny_every_row_count(gpu_device, m):
    n, k = 1000, 1168
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 0.02, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    out = _run(gpu_device, xq, wq, xs, ws, b, _lib.VARIANT_SKINNY)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws, b)


@pytest.mark.parametrize("variant,m", [(_lib.VARIANT_TILED, 320), (_lib.VARIANT_SKINNY, 40)])
def test_exact_integer_case_is_bit_exact(gpu_device, variant, m):
    # small integers, unit scales: all partial sums < 2^24, fp32 accumulation is exact in any
    # order, so the result must match the float64 computation bit for bit
    rng = np.random.default_rng(11)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4, 0.5, -0.5], dtype=np.float32)
    n, k = 384, 1040
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    xq, wq = torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn)
    out = _run(gpu_device, xq, wq, torch.ones(m), torch.ones(n), None, variant)
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(_bits(out), want)


@pytest.mark.parametrize("variant,m", [(_lib.VARIANT_TILED, 300), (_lib.VARIANT_SKINNY, 20)])
def test_every_code_pair_decodes_as_e4m3fn(gpu_device, variant, m):
    # one-hot rows: C[i, j] = value(code_a[i]) * value(code_b[j]) exactly (products of two
    # 4-bit significands fit fp32), so this pins the hardware's reading of every e4m3fn code,
    # including 0x7e = 448, subnormals and negative zero
    k = 16
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    a_codes = np.zeros((m, k), dtype=np.uint8)
    a_pick = finite[(np.arange(m) * 7) % len(finite)]
    a_codes[:, 3] = a_pick
    n = len(finite)
    b_codes = np.zeros((n, k), dtype=np.uint8)
    b_codes[:, 3] = finite
    xq = torch.from_numpy(a_codes).view(torch.float8_e4m3fn)
    wq = torch.from_numpy(b_codes).view(torch.float8_e4m3fn)
    out = _run(gpu_device, xq, wq, torch.ones(m), torch.ones(n), None, variant)
    t = e4m3.decode_table().astype(np.float64)
    want = orc.to_bf16_bits((t[a_pick][:, None] * t[finite][None, :]).astype(np.float32))
    got = _bits(out)
    # +0 and -0 compare equal as values; compare bit patterns modulo the sign of zero
    same = (got == want) | (((got | want) & 0x7FFF) == 0)
    assert np.all(same)


@pytest.mark.parametrize("variant,m", [(_lib.VARIANT_TILED, 270), (_lib.VARIANT_SKINNY, 33)])
def test_one_hot_positions_catch_index_and_swizzle_errors(gpu_device, variant, m):
    # A[i, ka(i)] = 1 and B[j, kb(j)] = 1: C[i, j] = [ka(i) == kb(j)]; walks every k residue
    n, k = 290, 400
    ka = (np.arange(m) * 37 + 5) % k
    kb = (np.arange(n) * 11 + 2) % k
    a = np.zeros((m, k), np.float32)
    b = np.zeros((n, k), np.float32)
    a[np.arange(m), ka] = 1.0
    b[np.arange(n), kb] = 1.0
    out = _run(gpu_device, torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn),
               torch.ones(m), torch.ones(n), None, variant)
    want = (ka[:, None] == kb[None, :]).astype(np.float32)
    assert np.array_equal(out.float().numpy(), want)


@pytest.mark.parametrize("variant,m", [(_lib.VARIANT_TILED, 130), (_lib.VARIANT_SKINNY, 9)])
def test_identity_weight_and_scale_axes(gpu_device, variant, m):
    k = 144
    xq, _, xs, _, _ = orc.make_inputs(m, k, k, 1.0, False)
    eye = torch.eye(k).to(torch.float8_e4m3fn)
    ws = torch.linspace(0.5, 2.0, k)
    out = _run(gpu_device, xq, eye, xs, ws, None, variant)
    want = (xq.float() * xs[:, None] * ws[None, :]).to(torch.bfloat16)
    # a single product chain in fp32: at most 1 ulp from the differently associated reference
    assert np.all(np.abs(out.float().numpy() - want.float().numpy()) <= _ulp_bf16(want.float().numpy()))


@pytest.mark.parametrize("variant,m", [(_lib.VARIANT_TILED, 200), (_lib.VARIANT_SKINNY, 24)])
def test_padded_operands_and_output_canaries(gpu_device, variant, m):
    # rows padded past K with garbage (lda, ldb > K), output embedded in a larger buffer:
    # padding must not leak into sums and nothing outside C[M, N] may be written
    n, k, pad = 150, 272, 48
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    a_buf = torch.full((m, k + pad), 0x7E, dtype=torch.uint8, device=dev)  # 448 everywhere
    b_buf = torch.full((n, k + pad), 0xFE, dtype=torch.uint8, device=dev)  # -448 everywhere
    a_buf[:, :k] = xq.view(torch.uint8).to(dev)
    b_buf[:, :k] = wq.view(torch.uint8).to(dev)
    c_buf = torch.full((m + 2, n + 24), -77.0, dtype=torch.bfloat16, device=dev)
    c_view = c_buf[1:m + 1, 8:8 + n]
    ops.fp8_gemm_rowwise(a_buf.view(torch.float8_e4m3fn)[:, :k], b_buf.view(torch.float8_e4m3fn)[:, :k],
                         xs.to(dev), ws.to(dev), bias=b.to(dev), out=c_view, variant=variant)
    torch.cuda.synchronize()
    torch.testing.assert_close(c_view.cpu(), want, rtol=RTOL, atol=ATOL)
    _check_tight(c_view.cpu(), xq, wq, xs, ws, b)
    mask = torch.ones_like(c_buf, dtype=torch.bool)
    mask[1:m + 1, 8:8 + n] = False
    assert torch.all(c_buf[mask] == -77.0)


@pytest.mark.parametrize("config", range(_lib.NUM_TILE_CONFIGS))
def test_tiled_family_takes_unaligned_scale_and_bias_vectors(gpu_device, config):
    # b_scale 4 bytes and bias 2 bytes into their allocations (a slice of a longer vector): full
    # tiles then take the element-wise epilogue instead of being refused
    m, n, k = 512, 512, 256
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    dev = gpu_device
    ws_buf = torch.zeros(n + 1, dtype=torch.float32, device=dev)
    ws_buf[1:] = ws.to(dev)
    bias_buf = torch.zeros(n + 1, dtype=torch.bfloat16, device=dev)
    bias_buf[1:] = b.to(dev)
    assert ws_buf[1:].data_ptr() % 16 == 4 and bias_buf[1:].data_ptr() % 8 == 2
    out = ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws_buf[1:], bias=bias_buf[1:],
                               variant=_lib.tiled_variant(config, 1))
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    _check_tight(out.cpu(), xq, wq, xs, ws, b)


def test_bias_is_fused_before_the_single_rounding(gpu_device):
    a = torch.zeros(16, 16)
    a[0, 0] = 1.0
    b = torch.zeros(16, 16)
    b[0, 0] = 1.0
    xs = torch.ones(16)
    xs[0] = 1.00390625
    bias = torch.zeros(16)
    bias[0] = 2.0 ** -8
    for variant in (_lib.VARIANT_TILED, _lib.VARIANT_SKINNY):
        out = _run(gpu_device, a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn), xs, torch.ones(16),
                   bias.to(torch.bfloat16), variant)
        assert out[0, 0].item() == 1.0078125


def test_unsupported_and_invalid_arguments_raise(gpu_device):
    dev = gpu_device
    f8 = lambda *s: torch.zeros(*s, device=dev).to(torch.float8_e4m3fn)
    # the MFMA families, pinned, refuse a K that is not a multiple of 16 (the automatic choice runs the generic family)
    for pinned in (_lib.VARIANT_TILED, _lib.VARIANT_SKINNY):
        with pytest.raises(NotImplementedError, match="multiple of 16"):
            ops.fp8_gemm_rowwise(f8(16, 24), f8(16, 24), torch.ones(16, device=dev), torch.ones(16, device=dev), variant=pinned)
    with pytest.raises(NotImplementedError, match="skinny"):
        ops.fp8_gemm_rowwise(f8(320, 32), f8(16, 32), torch.ones(320, device=dev), torch.ones(16, device=dev),
                             variant=_lib.VARIANT_SKINNY)
    with pytest.raises(TypeError):
        ops.fp8_gemm_rowwise(torch.zeros(16, 16, device=dev), f8(16, 16), torch.ones(16, device=dev), torch.ones(16, device=dev))
    with pytest.raises(ValueError):
        ops.fp8_gemm_rowwise(f8(16, 16), f8(16, 32), torch.ones(16, device=dev), torch.ones(16, device=dev))
    with pytest.raises(ValueError):
        ops.fp8_gemm_rowwise(f8(16, 16), f8(16, 16), torch.ones(15, device=dev), torch.ones(16, device=dev))
    with pytest.raises(ValueError, match="unknown variant"):
        ops.fp8_gemm_rowwise(f8(16, 16), f8(16, 16), torch.ones(16, device=dev), torch.ones(16, device=dev), variant=99)
    with pytest.raises(ValueError, match="unknown variant"):
        ops.fp8_gemm_rowwise(f8(16, 16), f8(16, 16), torch.ones(16, device=dev), torch.ones(16, device=dev),
                             variant=_lib.tiled_variant(_lib.NUM_TILE_CONFIGS))


def test_dispatch_is_pinned(gpu_device):
    assert ops.select_variant(16, 8192, 8192) == _lib.VARIANT_SKINNY
    assert ops.select_variant(32, 2048, 2048) == _lib.VARIANT_SKINNY
    assert ops.select_variant(8192, 8192, 8192) == _lib.VARIANT_TILED
    # up to 64 rows against a panel that gives every CU at most one 32-column tile: the M <= 64
    # family's narrow-tile form
    assert ops.select_variant(64, 8192, 8192) == _lib.VARIANT_SKINNY
    assert ops.select_variant(32, 8192, 28672) == _lib.VARIANT_SKINNY
    assert ops.select_variant(48, 10240, 8192) == _lib.VARIANT_SKINNY  # (64-column narrow tiles: one round on 160 CUs)
    # against long weight panels (many more tiles than CUs) split-K tiles that fetch B with the
    # streaming policy win
    assert ops.select_variant(48, 28672, 8192) == _lib.VARIANT_TILED
    assert ops.select_variant(64, 57344, 8192) == _lib.VARIANT_TILED
    assert ops.select_variant(32, 57344, 8192) == _lib.VARIANT_TILED
    assert ops.select_variant(16, 10240, 8192) == _lib.VARIANT_SKINNY
    # 65 .. 256 rows: the narrow-tile form in row blocks where that is one workgroup per CU and K is not too long
    assert ops.select_variant(128, 8192, 8192) == _lib.VARIANT_SKINNY
    assert ops.select_variant(128, 8192, 28672) == _lib.VARIANT_TILED
    assert ops.select_variant(128, 10240, 8192) == _lib.VARIANT_TILED
    assert ops.select_variant(512, 8192, 8192) == _lib.VARIANT_TILED


def test_graph_capture_replays_match_eager(gpu_device):
    # the benchmark harness times the callable inside a captured graph on a side stream
    dev = gpu_device
    for (m, n, k) in [(16, 2048, 2048), (300, 512, 1040), (128, 1024, 8192)]:  # skinny, tiled, split-K
        xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, True)
        dxq, dwq, dxs, dws, db = (t.to(dev) for t in (xq, wq, xs, ws, b))
        eager = ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db)
        torch.cuda.synchronize()
        out = torch.empty_like(eager)
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws, bias=db, out=out)  # warm-up outside capture
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


# ---- quantiser ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,cols,sigma", [(1, 16, 1.0), (7, 272, 1.0), (128, 512, 1.0), (33, 4112, 0.02), (1000, 1000, 3.0), (5, 17, 1.0)])
def test_quantiser_fp32_bit_exact(gpu_device, rows, cols, sigma):
    x = orc.randn_f32(rows, cols, sigma, seed=rows * 131 + cols)
    want_q, want_inv = orc.fp8_row_quantize(x)
    xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


# (bf16 rows of 1025 to 4096 elements go to a wave each only from 513 / 2049 rows up: both sides of each switch)
@pytest.mark.parametrize("rows,cols", [(9, 144), (256, 2048), (512, 2048), (600, 2048), (2048, 4096), (2100, 4096), (2100, 3080)])
def test_quantiser_bf16_bit_exact(gpu_device, rows, cols):
    x = orc.randn_f32(rows, cols, 1.0, seed=rows + cols).to(torch.bfloat16)
    want_q, want_inv = orc.fp8_row_quantize(x)
    xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


@pytest.mark.parametrize("dtype,cols", [(torch.float32, 1024), (torch.float32, 1040), (torch.float32, 2048), (torch.float32, 2064),
                                        (torch.bfloat16, 512), (torch.bfloat16, 1024), (torch.bfloat16, 1040), (torch.bfloat16, 2048), (torch.bfloat16, 2064),
                                        (torch.bfloat16, 4096), (torch.bfloat16, 4112)])
@pytest.mark.parametrize("rows", [1, 6, 8])
def test_quantiser_rows_of_one_wave(gpu_device, dtype, cols, rows):
    # rows short enough for one wave each (four per workgroup, the last workgroup partly empty), at the
    # row lengths where the form and the chunks kept per lane change
    x = orc.randn_f32(rows, cols, 1.0, seed=rows * 7 + cols).to(dtype)
    want_q, want_inv = orc.fp8_row_quantize(x)
    xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


def test_quantiser_rounding_at_every_code_boundary(gpu_device):
    # every finite e4m3fn value, every midpoint between neighbours (the ties) and the fp32
    # numbers just below and above each midpoint, with 448 as the row maximum so the scale is 1:
    # pins the conversion instruction's rounding against the oracle's cast code by code
    t = np.sort(np.unique(e4m3.decode_table()[np.isfinite(e4m3.decode_table())].astype(np.float32)))
    mids = ((t[:-1].astype(np.float64) + t[1:].astype(np.float64)) / 2).astype(np.float32)
    vals = np.concatenate([t, mids, np.nextafter(mids, np.float32(-np.inf)), np.nextafter(mids, np.float32(np.inf)),
                           np.float32([2.0 ** -10, 2.0 ** -11, 3 * 2.0 ** -11, 1e-30, -1e-30])])
    for amax in (448.0, 1.0, 0.013):  # other row maxima move the same grid through other scales
        row = (vals.astype(np.float64) * amax / 448.0).astype(np.float32)
        pad = (-len(row)) % 4
        x = torch.from_numpy(np.concatenate([row, np.zeros(pad, np.float32)])).reshape(1, -1)
        want_q, want_inv = orc.fp8_row_quantize(x)
        xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
        assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
        assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))
        xb = x.to(torch.bfloat16)
        xb = torch.cat([xb, torch.zeros(1, (-xb.shape[1]) % 8, dtype=torch.bfloat16)], dim=1)
        want_q, want_inv = orc.fp8_row_quantize(xb)
        xq, inv = ops.fp8_row_quantize(xb.to(gpu_device))
        assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
        assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


@pytest.mark.parametrize("dtype,rows,cols,width", [(torch.float32, 3, 20000, 20000), (torch.bfloat16, 2, 20480, 20480),
                                                     (torch.bfloat16, 3, 28672, 28672), (torch.bfloat16, 2, 32768, 32776),
                                                     (torch.bfloat16, 2, 32776, 32776), (torch.bfloat16, 2, 53248, 53248),
                                                     (torch.bfloat16, 1, 70000, 70000),
                                                     (torch.float32, 40, 1024, 1040), (torch.bfloat16, 40, 1000, 1024),
                                                     (torch.float32, 6, 1002, 1003)])
def test_quantiser_long_rows_and_strides(gpu_device, dtype, rows, cols, width):
    # rows longer than the register cache of the vector kernel, row strides wider than the
    # row (vector and scalar kernels), untouched bytes beyond each quantised row
    buf = orc.randn_f32(rows, width, 1.0, seed=cols).to(dtype)
    x = buf[:, :cols]
    want_q, want_inv = orc.fp8_row_quantize(x.contiguous())
    xq, inv = ops.fp8_row_quantize(buf.to(gpu_device)[:, :cols])
    assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


def test_quantiser_special_rows(gpu_device):
    x = torch.zeros(4, 64)
    x[1, 5] = 1e-20
    x[2, 7] = -3.0
    x[3] = torch.linspace(-5e4, 5e4, 64)
    want_q, want_inv = orc.fp8_row_quantize(x)
    xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
    assert torch.equal(xq.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert torch.equal(inv.cpu().view(torch.int32), want_inv.view(torch.int32))


@pytest.mark.parametrize("dtype,cols", [(torch.float32, 64), (torch.float32, 4100), (torch.float32, 61),
                                        (torch.bfloat16, 64), (torch.bfloat16, 16400), (torch.bfloat16, 59)])
def test_quantiser_non_finite_rows(gpu_device, dtype, cols):
    # rows holding NaN or infinities come out as the PyTorch program leaves them (vector and scalar
    # kernels, rows longer than the register cache): NaN codes wherever the oracle has NaN codes
    # (the sign bit of a NaN is the platform's), every other code and every inverse scale bit for bit
    x = orc.randn_f32(7, cols, 1.0, seed=cols).to(dtype)
    x[1, 3] = float("nan")
    x[2, 4] = float("inf")
    x[2, cols - 1] = float("-inf")
    x[3, 5] = float("-inf")
    x[3, cols - 2] = float("nan")
    x[5, cols // 2] = float("nan")
    x[6] = 0.0
    x[6, 1] = float("inf")
    want_q, want_inv = orc.fp8_row_quantize(x)
    xq, inv = ops.fp8_row_quantize(x.to(gpu_device))
    torch.cuda.synchronize()
    got, want = xq.cpu().view(torch.uint8).numpy(), want_q.view(torch.uint8).numpy()
    want_nan = (want & 0x7F) == 0x7F
    assert want_nan[1].all() and want_nan[3].all() and want_nan[5].all() and want_nan[2].sum() == 2 and want_nan[6].sum() == 1
    assert np.array_equal((got & 0x7F) == 0x7F, want_nan)
    assert np.array_equal(got[~want_nan], want[~want_nan])
    gi, wi = inv.cpu().numpy(), want_inv.numpy()
    assert np.array_equal(np.isnan(gi), np.isnan(wi))
    assert np.array_equal(gi[~np.isnan(wi)].view(np.uint32), wi[~np.isnan(wi)].view(np.uint32))
    assert np.isinf(gi[2]) and np.isinf(gi[6])


def test_quantise_then_gemm_end_to_end(gpu_device):
    # fp32 -> HIP quantiser -> HIP GEMM, against the same chain in the oracle
    m, n, k = 48, 640, 1024
    x = orc.randn_f32(m, k, 1.0, seed=1)
    w = orc.randn_f32(n, k, 1.0, seed=2)
    oq, os_ = orc.fp8_row_quantize(x)
    wq, ws = orc.fp8_row_quantize(w)
    want = orc.dequant_matmul(oq, wq, os_, ws)
    dxq, dxs = ops.fp8_row_quantize(x.to(gpu_device))
    dwq, dws = ops.fp8_row_quantize(w.to(gpu_device))
    out = ops.fp8_gemm_rowwise(dxq, dwq, dxs, dws)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu(), want, rtol=RTOL, atol=ATOL)
    # and it approximates the unquantised product to fp8 accuracy
    full = (x @ w.t())
    rel = (out.cpu().float() - full).norm() / full.norm()
    assert rel < 0.06
