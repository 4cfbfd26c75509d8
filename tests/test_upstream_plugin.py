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
