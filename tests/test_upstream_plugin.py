"""The drop-in boundary: `tritonbench_amd.upstream_plugin.register` against a stand-in for
upstream's `tritonbench.utils.triton_op` (only its `register_benchmark` signature and registry
layout, tritonbench/utils/triton_op.py:583-616, are modelled; nothing of the reference is
imported), and the harness path `run.py --op fp8_gemm_rowwise --metrics accuracy,...` on the GPU."""
import inspect
import sys
import types
from collections import OrderedDict
from dataclasses import dataclass
from typing import Optional

import pytest
import torch


@dataclass
class _Backend:
    name: str
    label: str
    baseline: bool = False
    enabled: bool = True
    fwd_only: bool = False


def _install_upstream_stub(monkeypatch):
    """A module named tritonbench.utils.triton_op whose register_benchmark has upstream's keyword
    signature and fills REGISTERED_BENCHMARKS / BASELINE_BENCHMARKS the way upstream does."""
    mod = types.ModuleType("tritonbench.utils.triton_op")
    mod.REGISTERED_BENCHMARKS = {}
    mod.BASELINE_BENCHMARKS = {}
    calls = []

    def register_benchmark(operator_name: Optional[str] = None, func_name: Optional[str] = None, baseline: bool = False,
                           enabled: bool = True, fwd_only: bool = False, label: Optional[str] = None):
        calls.append(dict(operator_name=operator_name, func_name=func_name, baseline=baseline, enabled=enabled,
                          fwd_only=fwd_only, label=label))

        def decorator(function):
            assert operator_name, "a function outside tritonbench.operators.<op> must name its operator"
            fn_name = func_name or function.__name__
            mod.REGISTERED_BENCHMARKS.setdefault(operator_name, OrderedDict())[fn_name] = _Backend(
                name=fn_name, label=label or fn_name, baseline=baseline, enabled=enabled, fwd_only=fwd_only)
            if baseline:
                mod.BASELINE_BENCHMARKS[operator_name] = fn_name
            return function

        return decorator

    mod.register_benchmark = register_benchmark
    pkg, utils = types.ModuleType("tritonbench"), types.ModuleType("tritonbench.utils")
    pkg.utils, utils.triton_op = utils, mod
    monkeypatch.setitem(sys.modules, "tritonbench", pkg)
    monkeypatch.setitem(sys.modules, "tritonbench.utils", utils)
    monkeypatch.setitem(sys.modules, "tritonbench.utils.triton_op", mod)
    return mod, calls


def test_register_fills_the_upstream_registry(monkeypatch):
    mod, calls = _install_upstream_stub(monkeypatch)
    from tritonbench_amd import upstream_plugin

    class FakeOperator:  # stands for upstream's Operator(BenchmarkOperator) of fp8_gemm_rowwise
        name = "fp8_gemm_rowwise"

    upstream_plugin.register(FakeOperator)
    # one registration, with upstream's keywords only
    assert len(calls) == 1
    assert calls[0]["operator_name"] == "fp8_gemm_rowwise" and calls[0]["func_name"] == "_hip_mi355x"
    assert calls[0]["label"] == "hip_mi355x" and calls[0]["baseline"] is False and calls[0]["fwd_only"] is False
    entry = mod.REGISTERED_BENCHMARKS["fp8_gemm_rowwise"]["_hip_mi355x"]
    assert entry.label == "hip_mi355x" and not entry.baseline
    # enabled exactly when a ROCm device is there (no GPU in a CPU test run: hidden, like upstream's
    # backends whose library is missing)
    assert entry.enabled == (torch.cuda.is_available() and torch.version.hip is not None)
    assert "fp8_gemm_rowwise" not in mod.BASELINE_BENCHMARKS
    # upstream looks the backend up with getattr(self, name) and calls it with the example inputs
    method = getattr(FakeOperator(), "_hip_mi355x")
    assert callable(method)
    params = list(inspect.signature(FakeOperator._hip_mi355x).parameters)
    assert params == ["self", "xq", "wq", "x_scale", "w_scale", "bias"]  # operator.py:187-217
    # registering as the baseline is the caller's choice
    upstream_plugin.register(FakeOperator, baseline=True)
    assert mod.BASELINE_BENCHMARKS["fp8_gemm_rowwise"] == "_hip_mi355x"


def test_backend_method_fails_loudly_without_a_gpu(monkeypatch):
    _install_upstream_stub(monkeypatch)
    from tritonbench_amd import upstream_plugin

    class FakeOperator:
        pass

    upstream_plugin.register(FakeOperator)
    if torch.cuda.is_available():
        pytest.skip("covers the host-tensor error path")
    xq = torch.zeros(16, 32).to(torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        FakeOperator()._hip_mi355x(xq, xq, torch.ones(16), torch.ones(16), None)()


@pytest.mark.gpu
def test_registered_backend_returns_a_capturable_callable(gpu_device, monkeypatch):
    mod, _ = _install_upstream_stub(monkeypatch)
    from oracle import fp8_rowwise as orc
    from tritonbench_amd import upstream_plugin

    class FakeOperator:
        name = "fp8_gemm_rowwise"

    upstream_plugin.register(FakeOperator)
    assert mod.REGISTERED_BENCHMARKS["fp8_gemm_rowwise"]["_hip_mi355x"].enabled
    xq, wq, xs, ws, b = orc.make_inputs(300, 520, 1040, 1.0, True)
    dev = gpu_device
    example_inputs = tuple(t.to(dev) for t in (xq, wq, xs, ws, b))
    fn = getattr(FakeOperator(), "_hip_mi355x")(*example_inputs)  # triton_op.py:765-775
    fn._name = "_hip_mi355x"                                       # triton_op.py:784: must accept attributes
    assert inspect.signature(fn).parameters == {}
    out = fn()
    torch.cuda.synchronize()
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-2, atol=1e-2)
    # the harness times it inside a captured graph on a side stream (operator.py:156)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            res = fn()
        res.fill_(0)
        g.replay()
        torch.cuda.synchronize()
    torch.testing.assert_close(res.cpu(), want, rtol=1e-2, atol=1e-2)


SIBLINGS = {
    # operator name -> (registrar, backend names, parameters of the first backend as upstream declares them)
    "fp8_gemm_rowwise_grouped": ("register_grouped", ["_hip_mi355x"], ["self", "group_A", "group_B", "m_sizes", "a_scale", "b_scale"]),
    "fp8_gemm_blockwise": ("register_blockwise", ["_hip_mi355x"], ["self", "xq", "wq", "x_scale", "w_scale"]),
    "fp8_gemm": ("register_tensorwise", ["_hip_mi355x"], ["self", "a", "b"]),
    "fp8_fused_quant_gemm_rowwise": ("register_fused_quant", ["rms_norm_fused_hip_mi355x", "silu_mul_fused_hip_mi355x"],
                                     ["self", "x1", "x2", "wq", "w_scale", "wd"]),
}


@pytest.mark.parametrize("operator_name", sorted(SIBLINGS))
def test_sibling_operators_register_under_their_own_names(monkeypatch, operator_name):
    """fp8_gemm_rowwise_grouped/operator.py:400-455, fp8_gemm_blockwise/operator.py:139-145,
    fp8_gemm/fp8_gemm.py:87-101, fp8_fused_quant_gemm_rowwise/operator.py:86-131: the backend
    methods take exactly the example inputs those operators yield."""
    mod, calls = _install_upstream_stub(monkeypatch)
    from tritonbench_amd import upstream_plugin

    registrar, names, params = SIBLINGS[operator_name]

    class FakeOperator:
        pass

    upstream_plugin.register_for(operator_name, FakeOperator)
    assert [c["func_name"] for c in calls] == names
    assert all(c["operator_name"] == operator_name and not c["baseline"] for c in calls)
    assert list(mod.REGISTERED_BENCHMARKS) == [operator_name]
    for name in names:
        assert list(inspect.signature(getattr(FakeOperator, name)).parameters) == params
    assert upstream_plugin.REGISTRARS[operator_name] is getattr(upstream_plugin, registrar)
    with pytest.raises(KeyError, match="no MI355X backend"):
        upstream_plugin.register_for("addmm", FakeOperator)


@pytest.mark.gpu
def test_sibling_backends_match_the_oracle(gpu_device, monkeypatch):
    """Each registered sibling backend, called the way upstream calls it, against the CPU oracle."""
    _install_upstream_stub(monkeypatch)
    from oracle import fp8_rowwise as orc
    from tritonbench_amd import upstream_plugin

    dev = gpu_device

    def make(name, **attrs):
        cls = type("FakeOperator", (), dict(attrs))
        upstream_plugin.register_for(name, cls)
        return cls()

    # grouped: G groups of the same N, K; sizes on the device
    g, n, k = 3, 256, 512
    sizes = [70, 0, 130]
    xq, _, xs, _, _ = orc.make_inputs(sum(sizes), 16, k, 1.0, False)
    _, wq, _, ws, _ = orc.make_inputs(16, g * n, k, 1.0, False)
    m_sizes = torch.tensor(sizes, dtype=torch.int32, device=dev)
    fn = make("fp8_gemm_rowwise_grouped")._hip_mi355x(xq.to(dev), wq.to(dev), m_sizes, xs.to(dev), ws.to(dev))
    got = fn().cpu()
    start = 0
    for gi, mg in enumerate(sizes):
        want = orc.dequant_matmul(xq[start:start + mg], wq[gi * n:(gi + 1) * n], xs[start:start + mg], ws[gi * n:(gi + 1) * n], None)
        torch.testing.assert_close(got[start:start + mg], want, rtol=1e-2, atol=1e-2)
        start += mg

    # tensor-wise: b is [K, N] column-major; both scale conventions
    a = torch.randn(200, 384).to(torch.float8_e4m3fn)
    b = torch.randn(384, 272).to(torch.float8_e4m3fn).T.contiguous().T
    want = a.to(torch.float32) @ b.to(torch.float32)
    for rowwise, dtype in ((False, torch.float16), (True, torch.bfloat16)):
        op = make("fp8_gemm", extra_args=types.SimpleNamespace(scaling_rowwise=rowwise))
        got = op._hip_mi355x(a.to(dev), b.to(dev))()
        assert got.dtype == dtype
        torch.testing.assert_close(got.cpu().to(torch.float32), want.to(dtype).to(torch.float32), rtol=1e-2, atol=1e-2)

    # block-wise: one scale per 128 x 128 block of either operand
    xq, wq, x_scale, w_scale = orc.make_blockwise_inputs(192, 256, 512)
    got = make("fp8_gemm_blockwise")._hip_mi355x(xq.to(dev), wq.to(dev), x_scale.to(dev), w_scale.to(dev))().cpu()
    torch.testing.assert_close(got, orc.blockwise_dequant_matmul(xq, wq, x_scale, w_scale), rtol=1e-2, atol=1e-2)

    # fused front ends: same result as the separate steps of this package
    from tritonbench_amd import ops

    x1 = torch.randn(64, 512, dtype=torch.bfloat16, device=dev)
    x2 = torch.randn(64, 512, dtype=torch.bfloat16, device=dev)
    wdn = torch.randn(512, dtype=torch.bfloat16, device=dev)
    wq2, w_scale2 = ops.fp8_row_quantize(torch.randn(128, 512, dtype=torch.bfloat16, device=dev))
    op = make("fp8_fused_quant_gemm_rowwise")
    got = op.rms_norm_fused_hip_mi355x(x1, x2, wq2, w_scale2, wdn)()
    q, s = ops.rms_norm_fp8_rowwise_quant(x1, wdn, 1e-5)
    assert torch.equal(got, ops.fp8_gemm_rowwise(q, wq2, s, w_scale2))
    got = op.silu_mul_fused_hip_mi355x(x1, x2, wq2, w_scale2, wdn)()
    q, s = ops.silu_mul_fp8_rowwise_quant(x1, x2)
    assert torch.equal(got, ops.fp8_gemm_rowwise(q, wq2, s, w_scale2))


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--m", "1000", "--n", "3000", "--k", "4112", "--bias"], ["--m", "16", "--n", "8192", "--k", "2048"]])
def test_harness_accuracy_tflops_gbps_on_the_hip_backend(gpu_device, extra):
    """`run.py --op fp8_gemm_rowwise ... --metrics accuracy,tflops,gbps`: the accuracy cell compares
    the HIP backend with the CPU baseline at rtol/atol 1e-2, tflops = flops / latency."""
    import run as run_py

    out = run_py.run(["--op", "fp8_gemm_rowwise", *extra, "--metrics", "latency,accuracy,tflops,gbps",
                      "--only", "_torch_dequant_cpu,_hip_mi355x"])
    (x_val, per_backend), = out.result
    m, n, k = x_val
    base, hip = per_backend["_torch_dequant_cpu"], per_backend["_hip_mi355x"]
    assert hip.error_msg is None and base.error_msg is None
    assert hip.accuracy is True
    flops = 2 * m * n * k + (2 * m * n if "--bias" in extra else 0)
    assert hip.tflops == pytest.approx(flops / hip.latency.p50 / 1e12 * 1e3, rel=1e-9)
    assert hip.extra_metrics["gbps"] == pytest.approx((m * k + n * k + 2 * m * n) / 1e9 / hip.latency.p50 * 1e3, rel=1e-9)
    text = str(out)
    assert "hip_mi355x-accuracy" in text and "torch_cpu_ref-accuracy" not in text  # the baseline shows no accuracy column
