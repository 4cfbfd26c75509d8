"""Parity of the block-scaled HIP path (through the C ABI) with the CPU oracle. Needs an MI355X."""
import numpy as np
import pytest
import torch

from oracle import e4m3
from oracle import fp8_rowwise as orc
from tritonbench_amd import ops

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # the tolerance the path is specified to
ATOL = 1e-2


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _run(dev, xq, wq, xs, ws, out=None):
    res = ops.fp8_gemm_blockwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), out=out)
    torch.cuda.synchronize()
    return res.cpu()


def _check_tight(out, xq, wq, xs, ws):
    """Within 1 bf16 ulp of the float64 value plus the slack fp32 accumulation is entitled to."""
    a = e4m3.decode(xq.view(torch.uint8).numpy()).astype(np.float64)
    b = e4m3.decode(wq.view(torch.uint8).numpy()).astype(np.float64)
    m, k = a.shape
    n = b.shape[0]
    sa = xs.numpy().astype(np.float64).repeat(128, 0).repeat(128, 1)[:m, :k]
    sb = ws.numpy().astype(np.float64).repeat(128, 0).repeat(128, 1)[:n, :k]
    exact = (a * sa) @ (b * sb).T
    slack = (np.abs(a) * sa) @ (np.abs(b) * sb).T * k * 2.0 ** -24
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** -126))) - 7)
    got = out.float().numpy().astype(np.float64)
    assert np.all(np.abs(got - exact) <= ulp + slack), f"max excess {np.max(np.abs(got - exact) - ulp - slack)}"


def test_blockwise_golden_fixture(gpu_device):
    import json
    import os

    golden = os.path.join(os.path.dirname(__file__), "golden")
    with open(os.path.join(golden, "manifest.json")) as f:
        manifest = json.load(f)
    for case in manifest["blockwise_cases"]:
        z = np.load(os.path.join(golden, case["file"]), allow_pickle=False)
        xq = torch.from_numpy(z["a"]).view(torch.float8_e4m3fn)
        wq = torch.from_numpy(z["b"]).view(torch.float8_e4m3fn)
        xs, ws = torch.from_numpy(z["a_scale"]), torch.from_numpy(z["b_scale"])
        want = torch.from_numpy(z["c"].view(np.int16)).view(torch.bfloat16)
        out = _run(gpu_device, xq, wq, xs, ws)
        torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
        _check_tight(out, xq, wq, xs, ws)


SHAPES = [(128, 128, 128), (256, 384, 512), (1, 16, 16), (130, 260, 272), (300, 200, 2048), (127, 129, 144),
          (512, 768, 1024), (64, 4096, 2048), (1000, 520, 4112), (257, 131, 9 * 128)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("sigma", [1.0, 0.02])
def test_blockwise_against_oracle(gpu_device, m, n, k, sigma):
    print(f"case m={m} n={n} k={k} sigma={sigma}", flush=True)
    xq, wq, xs, ws = orc.make_blockwise_inputs(m, n, k, sigma)
    want = orc.blockwise_dequant_matmul(xq, wq, xs, ws)
    out = _run(gpu_device, xq, wq, xs, ws)
    torch.testing.assert_close(out, want, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws)


def test_blockwise_scales_vary_per_block_and_step(gpu_device):
    # A = B = ones: C[m, n] = sum_kb 128 * xs[m // 128, kb] * ws[n // 128, kb]; with powers of two as
    # scales every value is exact, so a wrong block row, block column or K step shows bit for bit
    m, n, k = 300, 260, 5 * 128
    xq = torch.ones(m, k).to(torch.float8_e4m3fn)
    wq = torch.ones(n, k).to(torch.float8_e4m3fn)
    xs = 2.0 ** torch.arange(15).reshape(3, 5).float()
    ws = 2.0 ** -torch.arange(15).reshape(3, 5).flip(1).float()
    out = _run(gpu_device, xq, wq, xs, ws)
    want = 128.0 * (xs.double() @ ws.double().t())  # [3, 3] block values
    full = want.repeat_interleave(128, 0).repeat_interleave(128, 1)[:m, :n]
    assert np.array_equal(_bits(out), orc.to_bf16_bits(full.float().numpy()))


def test_blockwise_exact_integer_case_is_bit_exact(gpu_device):
    rng = np.random.default_rng(31)
    ints = np.array([0, 1, 2, 3, 4, -1, -2, -3, -4, 0.5, -0.5], dtype=np.float32)
    m, n, k = 200, 391, 1040
    a = rng.choice(ints, size=(m, k)).astype(np.float32)
    b = rng.choice(ints, size=(n, k)).astype(np.float32)
    xs = torch.ones(2, 9)
    ws = torch.ones(4, 9)
    dev = gpu_device
    c_buf = torch.full((m + 2, n + 9), -77.0, dtype=torch.bfloat16, device=dev)
    _run(dev, torch.from_numpy(a).to(torch.float8_e4m3fn), torch.from_numpy(b).to(torch.float8_e4m3fn), xs, ws,
         out=c_buf[1:m + 1, 3:3 + n])
    want = orc.to_bf16_bits((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(_bits(c_buf[1:m + 1, 3:3 + n].contiguous()), want)
    mask = torch.ones_like(c_buf, dtype=torch.bool)
    mask[1:m + 1, 3:3 + n] = False
    assert torch.all(c_buf[mask] == -77.0)


def test_blockwise_with_uniform_scales_equals_rowwise_kernel(gpu_device):
    m, n, k = 384, 512, 1024
    xq, wq, _, _ = orc.make_blockwise_inputs(m, n, k)
    xs = torch.full((3, 8), 0.5)  # powers of two: scaling commutes with every rounding
    ws = torch.full((4, 8), 2.0)
    out = _run(gpu_device, xq, wq, xs, ws)
    dev = gpu_device
    row = ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), torch.full((m,), 0.5, device=dev), torch.full((n,), 2.0, device=dev)).cpu()
    torch.testing.assert_close(out, row, rtol=RTOL, atol=ATOL)
    _check_tight(out, xq, wq, xs, ws)


def test_blockwise_graph_capture_replays_match_eager(gpu_device):
    dev = gpu_device
    xq, wq, xs, ws = (t.to(dev) for t in orc.make_blockwise_inputs(300, 512, 1040))
    eager = ops.fp8_gemm_blockwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.fp8_gemm_blockwise(xq, wq, xs, ws, out=out)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for _ in range(3):
                ops.fp8_gemm_blockwise(xq, wq, xs, ws, out=out)
        for _ in range(3):
            out.fill_(-5.0)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)


def test_blockwise_invalid_arguments_raise(gpu_device):
    dev = gpu_device
    xq, wq, xs, ws = (t.to(dev) for t in orc.make_blockwise_inputs(130, 64, 256))
    with pytest.raises(ValueError, match="expected x_scale"):
        ops.fp8_gemm_blockwise(xq, wq, xs[:1], ws)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fp8_gemm_blockwise(xq.cpu(), wq, xs, ws)
    with pytest.raises(NotImplementedError, match="multiple of 16"):
        ops.fp8_gemm_blockwise(xq[:, :24], wq[:, :24], xs[:, :1].contiguous(), ws[:, :1].contiguous())
