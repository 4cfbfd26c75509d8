"""The entry point that allocates nothing (mi355x_fp8_rowwise_gemm_noalloc), called through the
C ABI: its bf16 output must equal, bit for bit, what mi355x_fp8_rowwise_gemm writes with a
caller-provided workspace (same plan, same fixed summation order), on two calls in a row that
share the built-in scratch buffer, the second on a smaller problem. Needs an MI355X.

The file sorts last among the tests on purpose: a failure here must not hide the others.
"""
import numpy as np
import pytest
import torch

from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib

# (m, n, k, bias): shapes whose automatic plan splits K, i.e. really uses the scratch buffer;
# the second is smaller in every dimension and leaves stale partial sums of the first behind it
SPLIT_SHAPES = [(320, 1536, 8192, True), (264, 640, 4096, False)]
# a shape whose plan needs no scratch at all, after the two above
PLAIN_SHAPE = (512, 1024, 512, True)


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _operands(dev, m, n, k, bias):
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    d = lambda t: None if t is None else t.to(dev)
    return d(xq), d(wq), d(xs), d(ws), d(b), (xq, wq, xs, ws, b)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _with_workspace(lib, xq, wq, xs, ws, b, out, variant):
    m, k = xq.shape
    n = wq.shape[0]
    need = lib.mi355x_fp8_rowwise_workspace_bytes(m, n, k, variant)
    space = torch.empty(max(need, 16), dtype=torch.uint8, device=xq.device)
    st = lib.mi355x_fp8_rowwise_gemm(_ptr(xq), _ptr(wq), _ptr(xs), _ptr(ws), _ptr(b), _ptr(out), m, n, k,
                                     xq.stride(0), wq.stride(0), out.stride(0), space.data_ptr(), need, variant,
                                     torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "mi355x_fp8_rowwise_gemm")
    torch.cuda.synchronize()
    return need


def _no_alloc(lib, xq, wq, xs, ws, b, out, variant):
    m, k = xq.shape
    n = wq.shape[0]
    st = lib.mi355x_fp8_rowwise_gemm_noalloc(_ptr(xq), _ptr(wq), _ptr(xs), _ptr(ws), _ptr(b), _ptr(out), m, n, k,
                                             xq.stride(0), wq.stride(0), out.stride(0), variant,
                                             torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "mi355x_fp8_rowwise_gemm_noalloc")


@pytest.mark.gpu
def test_no_alloc_entry_matches_the_workspace_entry(gpu_device):
    lib = _lib.load()
    variant = _lib.VARIANT_AUTO
    cases = []
    for (m, n, k, bias) in SPLIT_SHAPES + [PLAIN_SHAPE]:
        xq, wq, xs, ws, b, host = _operands(gpu_device, m, n, k, bias)
        want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu_device)
        need = _with_workspace(lib, xq, wq, xs, ws, b, want, variant)
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu_device)
        cases.append((m, n, k, bias, xq, wq, xs, ws, b, host, want, got, need))
    assert all(c[-1] > 0 for c in cases[:2]), "the first two shapes are meant to use the scratch buffer"
    assert cases[2][-1] == 0
    assert cases[1][-1] < cases[0][-1]

    # every output tensor exists by now: between here and the comparison nothing is allocated
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(gpu_device)
    for (m, n, k, bias, xq, wq, xs, ws, b, host, want, got, need) in cases:
        print(f"no-alloc entry {m}x{n}x{k} bias={bias} scratch bytes {need}", flush=True)
        _no_alloc(lib, xq, wq, xs, ws, b, got, variant)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(gpu_device) == before

    for (m, n, k, bias, xq, wq, xs, ws, b, host, want, got, need) in cases:
        assert np.array_equal(_bits(got), _bits(want)), f"{m}x{n}x{k}: differs from the workspace entry point"
        # and both against the oracle, to the tolerance the path is specified to
        ref = orc.dequant_matmul(*host)
        torch.testing.assert_close(got.cpu(), ref, rtol=1e-2, atol=1e-2)

    # a pinned split factor goes the same way (third call on the same buffer, smaller again)
    m, n, k, bias = 64, 384, 2048, False
    xq, wq, xs, ws, b, host = _operands(gpu_device, m, n, k, bias)
    pinned = _lib.tiled_variant(config=1, splits=4)
    want = torch.empty((m, n), dtype=torch.bfloat16, device=gpu_device)
    got = torch.empty_like(want)
    assert _with_workspace(lib, xq, wq, xs, ws, b, want, pinned) == 4 * m * n * 4
    _no_alloc(lib, xq, wq, xs, ws, b, got, pinned)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(got), _bits(want))


def test_no_alloc_entry_refuses_plans_beyond_its_buffer():
    """Host arithmetic only: the request is turned away before any device call."""
    lib = _lib.load()
    m = n = 2048
    k = 4096
    pinned = _lib.tiled_variant(config=1, splits=8)
    need = lib.mi355x_fp8_rowwise_workspace_bytes(m, n, k, pinned)
    assert need == 8 * m * n * 4 > _lib.NOALLOC_SCRATCH_BYTES
    st = lib.mi355x_fp8_rowwise_gemm_noalloc(None, None, None, None, None, None, m, n, k, k, k, n, pinned, None)
    assert st == _lib.ENOTSUP
    msg = _lib.last_error()
    assert str(need) in msg and str(_lib.NOALLOC_SCRATCH_BYTES) in msg
    # bad shapes and variants keep their usual status
    assert lib.mi355x_fp8_rowwise_gemm_noalloc(None, None, None, None, None, None, 16, 16, 24, 32, 32, 16, 0, None) == _lib.ENOTSUP
    assert lib.mi355x_fp8_rowwise_gemm_noalloc(None, None, None, None, None, None, 16, 16, 16, 16, 16, 16, 1 << 25, None) == _lib.EINVAL
