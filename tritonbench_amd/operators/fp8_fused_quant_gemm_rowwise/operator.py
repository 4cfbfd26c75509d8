"""`fp8_fused_quant_gemm_rowwise` operator with the MI355X HIP backends.

Same surface as tritonbench/operators/fp8_fused_quant_gemm_rowwise/operator.py: flags
`--m/--n/--k` (:33-42), the built-in shape list (:49-70), inputs `(x1, x2, wq, w_scale, wd)` of
bf16 standard normals with the weight quantised row-wise (:154-165), the four backends that
chain a front end (RMSNorm with the weight vector `wd`, or SiLU(x1) * x2), the row-wise
quantiser and the row-wise GEMM (:86-131), and the `flops` metric and x value (:133-152).

The front-end kernels upstream imports (`gen_ai.llm_inference.fb.llm.kernel`) are not part of the
reference checkout; here the fused backends run this package's one-pass HIP kernels and the
unfused ones run the same arithmetic as separate steps (front end in PyTorch, then the HIP
quantiser), every one followed by the HIP row-wise GEMM.
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
from tritonbench_amd.operators.fp8_gemm_rowwise.operator import HAS_HIP_MI355X, PEAK_FP8_TFLOPS, fp8_row_quantize

RMS_NORM_EPS = 1e-5

BUILDIN_SHAPES = [
    (1, 2304, 2048), (1, 8192, 16384), (4, 4096, 2304), (4, 13312, 2048), (8, 2304, 2304),
    (8, 8192, 6656), (16, 4096, 6656), (16, 13312, 13312), (32, 2304, 16384), (32, 8192, 13312),
    (64, 4096, 2048), (64, 13312, 2048), (128, 2304, 6656), (128, 8192, 2304), (2048, 8192, 2048),
    (2048, 13312, 6656), (4096, 2304, 13312), (4096, 13312, 2304), (16384, 4096, 16384), (16384, 8192, 13312),
]


def parse_args(args: List[str]) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="fp8 fused quant gemm rowwise operator benchmark (MI355X)")
    p.add_argument("--m", type=int)
    p.add_argument("--n", type=int)
    p.add_argument("--k", type=int)
    return p.parse_args(args)


def _rms_norm(x: torch.Tensor, wd: torch.Tensor) -> torch.Tensor:
    xf = x.to(torch.float32)
    rstd = torch.rsqrt(xf.pow(2).mean(dim=1, keepdim=True) + RMS_NORM_EPS)
    return ((xf * rstd) * wd.to(torch.float32)).to(x.dtype)


def _silu_mul(x1: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    return (torch.nn.functional.silu(x1.to(torch.float32)) * x2.to(torch.float32)).to(x1.dtype)


class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["tflops"]
    DEFAULT_PRECISION = "fp8"
    # the unfused backends round the front end's result to bf16 before quantising it, the fused
    # ones do not: their fp8 codes differ by a step here and there, which the GEMM's K-long sums average out
    DEFAULT_RTOL = 5e-2
    DEFAULT_ATOL = 5e-2

    def __init__(self, tb_args: argparse.Namespace, extra_args: Optional[List[str]] = None):
        super().__init__(tb_args, extra_args)
        self.use_cuda_graphs = True
        a = parse_args(self.extra_args)
        self.shapes = [(a.m, a.n, a.k)] if a.m and a.n and a.k else BUILDIN_SHAPES

    def count_example_inputs(self) -> int:
        return len(self.shapes)

    @staticmethod
    def _need_gpu(x: torch.Tensor) -> None:
        if not x.is_cuda:
            raise NotImplementedError("the MI355X backends need device tensors (run with --device cuda)")

    @register_benchmark(enabled=HAS_HIP_MI355X)
    def rms_norm_fused(self, x1, x2, wq, w_scale, wd) -> Callable:
        self._need_gpu(x1)

        def run():
            xq, x_scale = ops.rms_norm_fp8_rowwise_quant(x1, wd, RMS_NORM_EPS)
            return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

        return run

    @register_benchmark(enabled=HAS_HIP_MI355X)
    def rms_norm_quant(self, x1, x2, wq, w_scale, wd) -> Callable:
        self._need_gpu(x1)

        def run():
            xq, x_scale = ops.fp8_row_quantize(_rms_norm(x1, wd))
            return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

        return run

    @register_benchmark(enabled=HAS_HIP_MI355X)
    def silu_mul_fused(self, x1, x2, wq, w_scale, wd) -> Callable:
        self._need_gpu(x1)

        def run():
            xq, x_scale = ops.silu_mul_fp8_rowwise_quant(x1, x2)
            return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

        return run

    @register_benchmark(enabled=HAS_HIP_MI355X)
    def silu_mul_quant(self, x1, x2, wq, w_scale, wd) -> Callable:
        self._need_gpu(x1)

        def run():
            xq, x_scale = ops.fp8_row_quantize(_silu_mul(x1, x2))
            return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

        return run

    @register_benchmark(label="rms_norm_cpu_ref")
    def _rms_norm_dequant_cpu(self, x1, x2, wq, w_scale, wd) -> Callable:
        """fp32 RMSNorm, row-wise quantisation and dequantised matmul on host cores (accuracy
        check of the two RMSNorm backends, and the backend a CPU-only run can time)."""
        hx, hw, hws, hwd = x1.cpu(), wq.cpu().to(torch.float32), w_scale.cpu(), wd.cpu()

        def run():
            xf = hx.to(torch.float32)
            y = (xf * torch.rsqrt(xf.pow(2).mean(dim=1, keepdim=True) + RMS_NORM_EPS)) * hwd.to(torch.float32)
            xq, xs = fp8_row_quantize(y)
            return ((xq.to(torch.float32) * xs[:, None]) @ (hw * hws[:, None]).T).to(torch.bfloat16)

        run.device = "cpu"
        return run

    @register_metric()
    def flops(self, fn_name: str, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        x1, _, wq, _, _ = example_inputs
        m, k = x1.size()
        n, k = wq.size()
        return m * k * 2 * n

    @register_metric()
    def mfma_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        return self.flops(None, example_inputs, metrics) / metrics.latency / 1e12 * 1e3 / PEAK_FP8_TFLOPS

    def accuracy(self, fn: Callable, baseline_fn: Callable) -> bool:
        rtol = self.tb_args.rtol if getattr(self.tb_args, "rtol", None) is not None else self.DEFAULT_RTOL
        atol = self.tb_args.atol if getattr(self.tb_args, "atol", None) is not None else self.DEFAULT_ATOL
        try:
            torch.testing.assert_close(fn().cpu(), baseline_fn().cpu(), rtol=rtol, atol=atol)
            return True
        except Exception as e:  # noqa: BLE001
            print(f"[accuracy] {type(e).__name__}: {str(e).splitlines()[0] if str(e) else ''}")
            return False

    @register_x_val(label="(M, N, K)")
    def get_x_val(self, example_inputs) -> Tuple[int, int, int]:
        x1, _, wq, _, _ = example_inputs
        m, k = x1.size()
        n, k = wq.size()
        return (m, n, k)

    def get_input_iter(self) -> Generator:
        for m, n, k in self.shapes:
            x1 = torch.randn((m, k), device=self.device, dtype=torch.bfloat16)
            x2 = torch.randn((m, k), device=self.device, dtype=torch.bfloat16)
            w = torch.randn((n, k), device=self.device, dtype=torch.bfloat16)
            wd = torch.randn((k,), device=self.device, dtype=torch.bfloat16)
            wq, w_scale = (ops.fp8_row_quantize(w) if w.is_cuda else fp8_row_quantize(w))
            yield x1, x2, wq, w_scale, wd
