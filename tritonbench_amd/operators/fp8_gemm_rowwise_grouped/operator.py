"""`fp8_gemm_rowwise_grouped` operator with the MI355X HIP backend.

Same surface as tritonbench/operators/fp8_gemm_rowwise_grouped/operator.py: op-level flags
(:76-136), the built-in shape and group-size lists (:195-234), inputs
(group_A, group_B, m_sizes, a_scale, b_scale) with equal group sizes M // G (:547-584),
backends that return zero-argument callables (:400-455), the `flops` / `gbps` metrics
(:482-545; flops = 2*M*N*K: every row of A meets one group's N columns) and the
"(group_size, M, N, K)" x axis (:457-480).

Backends here:
  _hip_mi355x          the grouped form of the gfx950 tiled kernel behind the C ABI
  _torch_dequant_cpu   per-group fp32 dequantise + torch.matmul on host cores, group boundaries
                       from m_sizes: accuracy baseline and CPU number
  _hip_mi355x_looped   one plain mi355x_fp8_rowwise_gemm call per group (G launches; needs the
                       sizes on the host): the yardstick the grouped kernel has to beat
"""
import argparse
from typing import Any, Callable, Generator, List, Optional, Tuple

import torch

from tritonbench_amd import ops
from tritonbench_amd.harness import (
    BenchmarkOperator,
    BenchmarkOperatorMetrics,
    register_benchmark,
    register_metric,
    register_x_val,
)
from tritonbench_amd.operators.fp8_gemm_rowwise.operator import (
    HAS_HIP_MI355X,
    PEAK_FP8_TFLOPS,
    PEAK_HBM_GBPS,
    fp8_row_quantize,
)

BUILTIN_SHAPES = [(1024, 1024, 1024), (2048, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 4096, 4096)]
GROUP_SIZES = [2, 4]


def parse_args(args: List[str]) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="grouped fp8 gemm rowwise operator benchmark (MI355X)")
    p.add_argument("--m", type=int)
    p.add_argument("--n", type=int)
    p.add_argument("--k", type=int)
    p.add_argument("--group_size", type=int)
    p.add_argument("--input-dtype", choices=["fp32", "bf16"], default="bf16")
    # NVIDIA-only kernel options of the upstream operator: accepted so command lines keep working
    p.add_argument("--no_fp8_fast_accum", dest="fp8_fast_accum", action="store_false")
    p.add_argument("--no_use_tma", dest="use_tma", default=None, action="store_false")
    p.add_argument("--use_tma", dest="use_tma", action="store_true")
    p.add_argument("--no_use_persistent", dest="no_use_persistent", action="store_true")
    p.add_argument("--warp_specialization", action="store_true")
    a = p.parse_args(args)
    if a.use_tma:
        raise RuntimeError("TMA is not supported on ROCm")
    return a


class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["tflops", "gbps", "speedup", "accuracy"]
    DEFAULT_PRECISION = "fp8"
    DEFAULT_RTOL = 1e-2
    DEFAULT_ATOL = 1e-2

    def __init__(self, tb_args: argparse.Namespace, extra_args: Optional[List[str]] = None):
        super().__init__(tb_args, extra_args)
        self.use_cuda_graphs = True
        a = parse_args(self.extra_args)
        self.shapes = [(a.m, a.n, a.k)] if (a.m and a.n and a.k) else list(BUILTIN_SHAPES)
        self.group_sizes = [a.group_size] if a.group_size else list(GROUP_SIZES)
        self.input_dtype = torch.float32 if a.input_dtype == "fp32" else torch.bfloat16

    def count_example_inputs(self) -> int:
        return len(self.shapes) * len(self.group_sizes)

    # ---- backends -------------------------------------------------------------------
    @register_benchmark(enabled=HAS_HIP_MI355X, label="hip_mi355x")
    def _hip_mi355x(self, group_A, group_B, m_sizes, a_scale, b_scale) -> Callable:
        if not group_A.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        n = group_B.shape[0] // m_sizes.numel()
        out = torch.zeros((group_A.shape[0], n), dtype=torch.bfloat16, device=group_A.device)
        return lambda: ops.fp8_gemm_rowwise_grouped(group_A, group_B, m_sizes, a_scale, b_scale, out=out)

    @register_benchmark(baseline=True, label="torch_cpu_ref")
    def _torch_dequant_cpu(self, group_A, group_B, m_sizes, a_scale, b_scale) -> Callable:
        ha, hb, hsa, hsb = group_A.cpu(), group_B.cpu(), a_scale.cpu(), b_scale.cpu()
        sizes = [int(v) for v in m_sizes.cpu()]
        n = hb.shape[0] // len(sizes)

        def run():
            out = torch.zeros((ha.shape[0], n), dtype=torch.bfloat16)
            start = 0
            for g, mg in enumerate(sizes):
                end = start + mg
                out[start:end] = ((ha[start:end].to(torch.float32) * hsa[start:end, None])
                                  @ (hb[g * n:(g + 1) * n].to(torch.float32) * hsb[g * n:(g + 1) * n, None]).t()
                                  ).to(torch.bfloat16)
                start = end
            return out

        run.device = "cpu"  # timed with the wall-clock loop, never graph-captured
        return run

    @register_benchmark(enabled=HAS_HIP_MI355X, label="hip_mi355x_looped")
    def _hip_mi355x_looped(self, group_A, group_B, m_sizes, a_scale, b_scale) -> Callable:
        if not group_A.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        sizes = [int(v) for v in m_sizes.cpu()]  # host copy, read once outside the timed callable
        n = group_B.shape[0] // len(sizes)
        out = torch.zeros((group_A.shape[0], n), dtype=torch.bfloat16, device=group_A.device)
        bounds, start = [], 0
        for g, mg in enumerate(sizes):
            if mg > 0:
                bounds.append((start, start + mg, g))
            start += mg
        spaces = [ops.gemm_workspace(e - s, n, group_A.shape[1], group_A.device) for s, e, _ in bounds]

        def run():
            for (s, e, g), ws in zip(bounds, spaces):
                ops.fp8_gemm_rowwise(group_A[s:e], group_B[g * n:(g + 1) * n], a_scale[s:e], b_scale[g * n:(g + 1) * n],
                                     out=out[s:e], workspace=ws)
            return out

        return run

    # ---- metrics --------------------------------------------------------------------
    @staticmethod
    def _dims(example_inputs) -> Tuple[int, int, int, int]:
        group_A, group_B, m_sizes, _, _ = example_inputs
        g = len(m_sizes)
        m, k = group_A.size()
        return g, m, group_B.size(0) // g, k

    @register_metric()
    def flops(self, fn_name: str, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        _, m, n, k = self._dims(example_inputs)
        return n * m * k * 2

    @register_metric()
    def gbps(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        g, m, n, k = self._dims(example_inputs)
        return (m * k + g * n * k + 2 * m * n) / 1e9 / metrics.latency * 1e3

    @register_metric()
    def mfma_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        return self.flops(None, example_inputs, metrics) / metrics.latency / 1e12 * 1e3 / PEAK_FP8_TFLOPS

    @register_metric()
    def hbm_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        return self.gbps(fn, example_inputs, metrics) / PEAK_HBM_GBPS

    def accuracy(self, fn: Callable, baseline_fn: Callable) -> bool:
        rtol = self.tb_args.rtol if getattr(self.tb_args, "rtol", None) is not None else self.DEFAULT_RTOL
        atol = self.tb_args.atol if getattr(self.tb_args, "atol", None) is not None else self.DEFAULT_ATOL
        try:
            torch.testing.assert_close(fn().cpu(), baseline_fn().cpu(), rtol=rtol, atol=atol)
            return True
        except Exception:
            return False

    @register_x_val(label="(group_size, M, N, K)")
    def get_x_val(self, example_inputs) -> Tuple[int, int, int, int]:
        return self._dims(example_inputs)

    # ---- inputs ---------------------------------------------------------------------
    def get_input_iter(self) -> Generator:
        for group_size in self.group_sizes:
            for m, n, k in self.shapes:
                B = torch.randn((group_size * n, k), device=self.device, dtype=self.input_dtype)
                group_B, b_scale = fp8_row_quantize(B)
                m_sizes = torch.tensor([m // group_size] * group_size, device=self.device, dtype=torch.int32)
                A = torch.randn((m, k), device=self.device, dtype=self.input_dtype)
                group_A, a_scale = fp8_row_quantize(A)
                del A, B
                yield group_A, group_B, m_sizes, a_scale, b_scale
