"""`fp8_gemm_blockwise` operator with the MI355X HIP backend.

Same surface as tritonbench/operators/fp8_gemm_blockwise/operator.py: flags (:21-28), the
built-in shape list (:59-80), 128x128 block quantisation of both operands (:86-118,
:164-176), backends that return zero-argument callables (:139-145), the `flops` metric
(:147-156) and the "(M, N, K)" x axis (:158-162). Upstream marks its Triton backend as
unsupported on AMD GPUs (:40-41); this operator supplies one.

Backends here:
  _hip_mi355x          the block-scaled form of the gfx950 tiled kernel behind the C ABI
  _torch_dequant_cpu   fp32 dequantise (every element times its block's scale) + torch.matmul
                       on host cores: accuracy baseline and CPU number
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
    BUILDIN_SHAPES,
    HAS_HIP_MI355X,
    PEAK_FP8_TFLOPS,
)

E4M3_MAX_POS: float = torch.finfo(torch.float8_e4m3fn).max
EPS: float = 1e-12
BLOCK = 128


def parse_args(args: List[str]) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="block-scaled fp8 gemm operator benchmark (MI355X)")
    p.add_argument("--m", type=int)
    p.add_argument("--n", type=int)
    p.add_argument("--k", type=int)
    p.add_argument("--llama", action="store_true")
    return p.parse_args(args)


def fp8_block_quantize_torch(x: torch.Tensor, block_m: int = BLOCK, block_k: int = BLOCK) -> Tuple[torch.Tensor, torch.Tensor]:
    """Eager PyTorch form (operator.py:86-118): one scale per block_m x block_k block; returns the
    fp8 tensor and the inverse scales [ceil(M/block_m), ceil(K/block_k)]. Used for host tensors."""
    m, k = x.shape
    gm, gk = -(-m // block_m), -(-k // block_k)
    padded = torch.zeros(gm * block_m, gk * block_k, dtype=x.dtype, device=x.device)
    padded[:m, :k] = x
    block_max = torch.clamp(padded.abs().reshape(gm, block_m, gk, block_k).amax(dim=(1, 3)), min=EPS)
    scale = E4M3_MAX_POS / block_max.to(torch.float32)
    scale[scale == float("inf")] = 1.0
    xq = (padded * scale.repeat_interleave(block_m, dim=0).repeat_interleave(block_k, dim=1))[:m, :k]
    return xq.to(torch.float8_e4m3fn), 1 / scale


def fp8_block_quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """128 x 128 block quantisation: the HIP kernel for device tensors, eager PyTorch for host tensors."""
    if x.is_cuda:
        return ops.fp8_block_quantize(x)
    return fp8_block_quantize_torch(x)


class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["tflops", "speedup", "accuracy"]
    DEFAULT_PRECISION = "fp8"
    DEFAULT_RTOL = 1e-2
    DEFAULT_ATOL = 1e-2

    def __init__(self, tb_args: argparse.Namespace, extra_args: Optional[List[str]] = None):
        super().__init__(tb_args, extra_args)
        self.use_cuda_graphs = True
        a = parse_args(self.extra_args)
        if a.m and a.n and a.k:
            self.shapes = [(a.m, a.n, a.k)]
        else:
            self.shapes = list(BUILDIN_SHAPES)

    def count_example_inputs(self) -> int:
        return len(self.shapes)

    @register_benchmark(enabled=HAS_HIP_MI355X, label="hip_mi355x")
    def _hip_mi355x(self, xq, wq, x_scale, w_scale) -> Callable:
        if not xq.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        out = torch.empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16, device=xq.device)
        return lambda: ops.fp8_gemm_blockwise(xq, wq, x_scale, w_scale, out=out)

    @register_benchmark(baseline=True, label="torch_cpu_ref")
    def _torch_dequant_cpu(self, xq, wq, x_scale, w_scale) -> Callable:
        hx, hw, hxs, hws = xq.cpu(), wq.cpu(), x_scale.cpu(), w_scale.cpu()
        m, k = hx.shape
        n = hw.shape[0]

        def run():
            xs = hxs.repeat_interleave(BLOCK, dim=0).repeat_interleave(BLOCK, dim=1)[:m, :k]
            ws = hws.repeat_interleave(BLOCK, dim=0).repeat_interleave(BLOCK, dim=1)[:n, :k]
            return ((hx.to(torch.float32) * xs) @ (hw.to(torch.float32) * ws).t()).to(torch.bfloat16)

        run.device = "cpu"  # timed with the wall-clock loop, never graph-captured
        return run

    @register_metric()
    def flops(self, fn_name: str, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        xq, wq, _, _ = example_inputs
        m, k = xq.size()
        return m * k * 2 * wq.size(0)

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
        xq, wq, _, _ = example_inputs
        m, k = xq.size()
        return (m, wq.size(0), k)

    def get_input_iter(self) -> Generator:
        for m, n, k in self.shapes:
            x = torch.randn((m, k), device=self.device, dtype=torch.bfloat16)
            w = torch.randn((n, k), device=self.device, dtype=torch.bfloat16)
            xq, x_scale = fp8_block_quantize(x)
            wq, w_scale = fp8_block_quantize(w)
            del x, w
            yield xq, wq, x_scale, w_scale
