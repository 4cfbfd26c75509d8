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

    # Every output tensor exists by now, and the device was set up (scratch address looked up) when the
    # operands above were made: between here and the comparison nothing is allocated, by PyTorch
    # (its own counter) or by anybody else in the process (the driver's free-memory figure sees a
    # hipMalloc inside the library too).
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(gpu_device)
    free_before, _ = torch.cuda.mem_get_info(gpu_device)
    for (m, n, k, bias, xq, wq, xs, ws, b, host, want, got, need) in cases:
        print(f"no-alloc entry {m}x{n}x{k} bias={bias} scratch bytes {need}", flush=True)
        _no_alloc(lib, xq, wq, xs, ws, b, got, variant)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(gpu_device)
    assert torch.cuda.memory_allocated(gpu_device) == before
    assert free_after >= free_before, f"device memory shrank by {free_before - free_after} bytes across the calls"

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


@pytest.mark.gpu
def test_no_alloc_entry_runs_a_smaller_plan_when_the_automatic_one_does_not_fit(gpu_device):
    """An automatic plan that wants more scratch than the buffer holds is not an error: the call
    runs the cheapest plan that fits, exactly as the workspace entry point does with a workspace of
    the buffer's size (bit-identical), and agrees with the full-workspace plan to the tolerance."""
    from tritonbench_amd import ops

    lib = _lib.load()
    m, n, k = 768, 8192, 65536
    need = lib.mi355x_fp8_rowwise_workspace_bytes(m, n, k, _lib.VARIANT_AUTO)
    assert need > _lib.NOALLOC_SCRATCH_BYTES, "the shape is meant to want more scratch than the buffer holds"
    g = torch.Generator(device=gpu_device)
    g.manual_seed(99)
    xq, xs = ops.fp8_row_quantize(torch.randn((m, k), generator=g, device=gpu_device))
    wq, ws = ops.fp8_row_quantize(torch.randn((n, k), generator=g, device=gpu_device))
    full = torch.empty((m, n), dtype=torch.bfloat16, device=gpu_device)
    _with_workspace(lib, xq, wq, xs, ws, None, full, _lib.VARIANT_AUTO)
    same_size = torch.empty_like(full)
    space = torch.empty(_lib.NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device=gpu_device)
    st = lib.mi355x_fp8_rowwise_gemm(_ptr(xq), _ptr(wq), _ptr(xs), _ptr(ws), None, _ptr(same_size), m, n, k, k, k, n,
                                     space.data_ptr(), _lib.NOALLOC_SCRATCH_BYTES, _lib.VARIANT_AUTO,
                                     torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "mi355x_fp8_rowwise_gemm")
    got = torch.full_like(full, float("nan"))
    print(f"no-alloc entry {m}x{n}x{k}: automatic plan wants {need} bytes", flush=True)
    _no_alloc(lib, xq, wq, xs, ws, None, got, _lib.VARIANT_AUTO)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(got), _bits(same_size))
    torch.testing.assert_close(got, full, rtol=1e-2, atol=1e-2)


def test_no_alloc_entry_refuses_plans_beyond_its_buffer():
    """Host arithmetic only: a split factor the caller named and the buffer cannot hold is turned
    away before any device call."""
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
    assert lib.mi355x_fp8_rowwise_gemm_noalloc(None, None, None, None, None, None, 16, 2 ** 31, 32, 32, 32, 16, 0, None) == _lib.ENOTSUP
    assert lib.mi355x_fp8_rowwise_gemm_noalloc(None, None, None, None, None, None, 16, 16, 16, 16, 16, 16, 1 << 25, None) == _lib.EINVAL
