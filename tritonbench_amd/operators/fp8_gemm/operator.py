"""`fp8_gemm` operator (tensor-wise scaled FP8 GEMM) with the MI355X HIP backend.

Same surface as tritonbench/operators/fp8_gemm/fp8_gemm.py: flags `--llama`,
`--scaling_rowwise`, `--m/--n/--k` (:36-43), inputs `(a, b)` with `a = randn(m, k)` cast to
e4m3fn and `b` of shape [K, N] in column-major order (:52-66), the default shape sweep
(:72-78), unit scales — one-element tensors and float16 output, or [M,1]/[1,N] vectors and
bfloat16 output with `--scaling_rowwise` (:87-101) — and the `flops` / `gbps` metrics
(:143-165).

Backends here:
  _hip_mi355x        the row-wise kernels of this package with constant scale vectors
  torch_fp8_gemm     torch._scaled_mm (hipBLASLt), as upstream's baseline of the same name
  _torch_dequant_cpu fp32 widen + torch.matmul on host cores (accuracy baseline off-GPU)
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
    HAS_SCALED_MM,
    LLAMA3_70B_M_PREFILL,
    LLAMA3_70B_NK,
    PEAK_FP8_TFLOPS,
)


def parse_args(args: List[str]) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="fp8_gemm operator benchmark (MI355X)")
    p.add_argument("--llama", action="store_true")
    p.add_argument("--scaling_rowwise", action="store_true")
    p.add_argument("--m", type=int)
    p.add_argument("--k", type=int)
    p.add_argument("--n", type=int)
    return p.parse_args(args)


class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["tflops", "gbps", "latency"]
    DEFAULT_PRECISION = "fp8"
    DEFAULT_RTOL = 1e-2
    DEFAULT_ATOL = 1e-2

    def __init__(self, tb_args: argparse.Namespace, extra_args: Optional[List[str]] = None):
        super().__init__(tb_args, extra_args)
        self.use_cuda_graphs = True
        self.op_args = parse_args(self.extra_args)

    def _shapes(self) -> List[Tuple[int, int, int]]:
        a = self.op_args
        if a.llama:
            return [(m, n, k) for (n, k) in LLAMA3_70B_NK for m in LLAMA3_70B_M_PREFILL]
        if a.m:
            return [(a.m, a.n, a.k)]
        shapes = []
        for i in range(10, 15):
            for j in range(0, 4):
                k = 2 ** i
                k += k // 4 * j
                shapes.append((k, k, k))
        return shapes

    def count_example_inputs(self) -> int:
        return len(self._shapes())

    def _scales(self, a: torch.Tensor, b: torch.Tensor):
        if self.op_args.scaling_rowwise:
            return (torch.ones((a.shape[0], 1), dtype=torch.float32, device=a.device),
                    torch.ones((1, b.shape[1]), dtype=torch.float32, device=b.device), torch.bfloat16)
        return torch.tensor(1.0, device=a.device), torch.tensor(1.0, device=a.device), torch.float16

    @register_benchmark(enabled=HAS_HIP_MI355X, label="hip_mi355x")
    def _hip_mi355x(self, a, b) -> Callable:
        if not a.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        scale_a, scale_b, out_dtype = self._scales(a, b)
        return ops.fp8_gemm_tensorwise(a, b, scale_a, scale_b, out_dtype=out_dtype)

    @register_benchmark(enabled=HAS_SCALED_MM, label="torch_fp8_gemm")
    def torch_fp8_gemm(self, a, b) -> Callable:
        if not a.is_cuda:
            raise NotImplementedError("torch._scaled_mm needs a GPU")
        scale_a, scale_b, out_dtype = self._scales(a, b)
        return lambda: torch._scaled_mm(a, b, scale_a, scale_b, use_fast_accum=True, out_dtype=out_dtype)

    @register_benchmark(baseline=True, label="torch_cpu_ref")
    def _torch_dequant_cpu(self, a, b) -> Callable:
        ha, hb = a.cpu().to(torch.float32), b.cpu().to(torch.float32)
        out_dtype = torch.bfloat16 if self.op_args.scaling_rowwise else torch.float16

        def run():
            return (ha @ hb).to(out_dtype)

        run.device = "cpu"  # timed with the wall-clock loop, never graph-captured
        return run

    @register_metric()
    def flops(self, fn_name: str, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        a, b = example_inputs
        m, k = a.size()
        return 2 * m * b.size(1) * k

    @register_metric()
    def gbps(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        a, b = example_inputs
        m, k = a.size()
        n = b.size(1)
        return (m * k + k * n + 2 * m * n) / 1e9 / metrics.latency * 1e3

    @register_metric()
    def mfma_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        return self.flops(None, example_inputs, metrics) / metrics.latency / 1e12 * 1e3 / PEAK_FP8_TFLOPS

    def accuracy(self, fn: Callable, baseline_fn: Callable) -> bool:
        rtol = self.tb_args.rtol if getattr(self.tb_args, "rtol", None) is not None else self.DEFAULT_RTOL
        atol = self.tb_args.atol if getattr(self.tb_args, "atol", None) is not None else self.DEFAULT_ATOL
        try:
            torch.testing.assert_close(fn().cpu(), baseline_fn().cpu(), rtol=rtol, atol=atol)
            return True
        except Exception:
            return False

    @register_x_val(label="(M, N, K)")
    def get_x_val(self, example_inputs) -> Tuple[int, int, int]:
        a, b = example_inputs
        m, k = a.size()
        return (m, b.size(1), k)

    def get_input_iter(self) -> Generator:
        for m, n, k in self._shapes():
            a = torch.randn(m, k, device=self.device).to(torch.float8_e4m3fn)
            b = torch.randn(k, n, device=self.device).to(torch.float8_e4m3fn).T.contiguous().T
            yield a, b
