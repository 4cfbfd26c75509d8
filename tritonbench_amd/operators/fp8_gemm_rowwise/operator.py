"""`fp8_gemm_rowwise` operator with the MI355X HIP backend.

Same surface as tritonbench/operators/fp8_gemm_rowwise/operator.py: op-level flags
(:21-63), the built-in shape list (:107-128), row-wise quantised inputs
(xq, wq, x_scale, w_scale, bias) (:280-297), backends that return zero-argument callables
(:187-235), the `flops` / `gbps` metrics (:248-271) and the "(M, N, K)" x axis (:273-278).

Backends here:
  _hip_mi355x          hand-written gfx950 kernels behind the C ABI (the point of this package)
  _torch_dequant_cpu   fp32 dequantise + torch.matmul on host cores: the accuracy baseline and
                       the CPU number reported beside the GPU one; never used to produce
                       the HIP backend's result
  _scaled_mm           torch._scaled_mm with row-wise scales (hipBLASLt): a vendor yardstick,
                       the variant upstream leaves commented out at :237-246
"""
import argparse
import logging
from typing import Any, Callable, Generator, List, Optional, Tuple

import torch

from tritonbench_amd import _lib, ops
from tritonbench_amd.harness import (
    BenchmarkOperator,
    BenchmarkOperatorMetrics,
    register_benchmark,
    register_metric,
    register_x_val,
)

logger = logging.getLogger(__name__)

FP8_DTYPE = torch.float8_e4m3fn
E4M3_MAX_POS: float = torch.finfo(FP8_DTYPE).max
EPS: float = 1e-12
FP16_MAX_POS: float = torch.finfo(torch.float16).max

# MI355X datasheet peaks used by the roofline metrics (dense FP8 MFMA; HBM3E).
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBPS = 8000.0

BUILDIN_SHAPES = [
    (1, 2304, 2048), (1, 8192, 16384), (4, 4096, 2304), (4, 13312, 2048), (8, 2304, 2304),
    (8, 8192, 6656), (16, 4096, 6656), (16, 13312, 13312), (32, 2304, 16384), (32, 8192, 13312),
    (64, 4096, 2048), (64, 13312, 2048), (128, 2304, 6656), (128, 8192, 2304), (2048, 8192, 2048),
    (2048, 13312, 6656), (4096, 2304, 13312), (4096, 13312, 2304), (16384, 4096, 16384),
    (16384, 8192, 13312),
]

# Llama-3-70B projections as (N, K), full unsharded weights. Upstream's --llama list is
# Meta-internal (utils/triton_op.py:159-165 returns None outside fbcode), so this one is ours.
LLAMA3_70B_NK = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]
LLAMA3_70B_M_DECODE = [1, 32, 128]
LLAMA3_70B_M_PREFILL = [1024, 4096]


def parse_args(args: List[str]) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="fp8 gemm rowwise operator benchmark (MI355X)")
    p.add_argument("--m", type=int)
    p.add_argument("--n", type=int)
    p.add_argument("--k", type=int)
    p.add_argument("--bias", action="store_true", default=False)
    p.add_argument("--llama", action="store_true")
    p.add_argument("--prefill", default=False, action="store_true")
    p.add_argument("--sigma", type=float, default=1.0, help="std-dev of the fp32/bf16 source tensors")
    p.add_argument("--input-dtype", choices=["fp32", "bf16"], default="fp32",
                   help="dtype of the tensors that get quantised (upstream draws bf16)")
    # Flags of the upstream operator that select NVIDIA-only kernel variants. They are parsed so
    # existing command lines keep working, and rejected where upstream rejects them on ROCm.
    p.add_argument("--no_fp8_fast_accum", dest="fp8_fast_accum", action="store_false")
    p.add_argument("--no_use_tma", dest="use_tma", default=None, action="store_false")
    p.add_argument("--use_tma", dest="use_tma", action="store_true")
    p.add_argument("--use_persistent", dest="no_use_persistent", default=None, action="store_false")
    p.add_argument("--no_use_persistent", dest="no_use_persistent", action="store_true")
    p.add_argument("--warp_specialization", action="store_true")
    a = p.parse_args(args)
    if a.use_tma is None:
        a.use_tma = False
    if a.use_tma:
        raise RuntimeError("TMA is not supported on ROCm")
    if a.no_use_persistent is None:
        a.no_use_persistent = True
    if a.warp_specialization:
        a.warp_specialization = False
        print("Warp specialization is not supported on ROCm defaulting to False")
    return a


def fp8_row_quantize_torch(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Eager PyTorch form of the quantiser (operator.py:136-145); used for host tensors."""
    row_max = torch.max(torch.abs(x), dim=1).values
    scale = E4M3_MAX_POS / torch.clamp(row_max, EPS)
    if x.dtype is torch.float16:
        scale = torch.clamp(scale, max=FP16_MAX_POS)
    xq = torch.clamp(x * scale[:, None], min=-E4M3_MAX_POS, max=E4M3_MAX_POS).to(FP8_DTYPE)
    return xq, scale.reciprocal().to(torch.float32)


def fp8_row_quantize(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise a tensor row-wise and return the fp8 tensor and its inverse scale: the HIP
    kernel for device tensors, eager PyTorch for host tensors."""
    if x.is_cuda:
        return ops.fp8_row_quantize(x)
    return fp8_row_quantize_torch(x)


def _hip_backend_available() -> bool:
    if not torch.cuda.is_available() or torch.version.hip is None:
        return False
    _lib.load()  # raises if the library was not built: never silently absent on a GPU box
    return True


HAS_HIP_MI355X = _hip_backend_available()
HAS_SCALED_MM = torch.cuda.is_available() and hasattr(torch, "_scaled_mm")


class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["tflops", "gbps", "speedup", "accuracy"]
    DEFAULT_PRECISION = "fp8"
    DEFAULT_RTOL = 1e-2
    DEFAULT_ATOL = 1e-2

    def __init__(self, tb_args: argparse.Namespace, extra_args: Optional[List[str]] = None):
        super().__init__(tb_args, extra_args)
        self.use_cuda_graphs = True
        a = parse_args(self.extra_args)
        if a.m and a.n and a.k:
            self.shapes = [(a.m, a.n, a.k)]
        elif a.llama:
            ms = LLAMA3_70B_M_PREFILL if a.prefill else LLAMA3_70B_M_DECODE
            self.shapes = [(m, n, k) for (n, k) in LLAMA3_70B_NK for m in ms]
        else:
            self.shapes = list(BUILDIN_SHAPES)
        self.bias = a.bias
        self.sigma = a.sigma
        self.input_dtype = torch.float32 if a.input_dtype == "fp32" else torch.bfloat16
        self.fp8_fast_accum = a.fp8_fast_accum  # accumulation here is always full fp32
        self.use_tma = a.use_tma
        self.no_use_persistent = a.no_use_persistent
        self.warp_specialization = a.warp_specialization

    def count_example_inputs(self) -> int:
        return len(self.shapes)

    # ---- backends -------------------------------------------------------------------
    @register_benchmark(enabled=HAS_HIP_MI355X, label="hip_mi355x")
    def _hip_mi355x(self, xq, wq, x_scale, w_scale, bias) -> Callable:
        if not xq.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        out = torch.empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16, device=xq.device)
        workspace = ops.gemm_workspace(xq.shape[0], wq.shape[0], xq.shape[1], xq.device)
        return lambda: ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale, bias=bias, out=out, workspace=workspace)

    @register_benchmark(enabled=False, label="hip_mi355x_autotuned")
    def _hip_mi355x_autotuned(self, xq, wq, x_scale, w_scale, bias) -> Callable:
        """The same library with the plan chosen by timing every candidate for the shape once (outside
        the timed callable; cached per shape), the way the reference's Triton kernels are autotuned.
        Off by default (the sweep costs a second or two per shape): ask for it with --only."""
        if not xq.is_cuda:
            raise NotImplementedError("the MI355X backend needs device tensors (run with --device cuda)")
        from tritonbench_amd import tuning

        m, k = xq.shape
        n = wq.shape[0]
        variant, _, _ = tuning.autotune(m, n, k, xq.device, bias=bias is not None)
        out = torch.empty((m, n), dtype=torch.bfloat16, device=xq.device)
        workspace = ops.gemm_workspace(m, n, k, xq.device, variant)
        return lambda: ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale, bias=bias, out=out, workspace=workspace, variant=variant)

    @register_benchmark(baseline=True, label="torch_cpu_ref")
    def _torch_dequant_cpu(self, xq, wq, x_scale, w_scale, bias) -> Callable:
        hx, hw = xq.cpu(), wq.cpu()
        hxs, hws = x_scale.cpu(), w_scale.cpu()
        hb = bias.cpu().to(torch.float32) if bias is not None else None

        def run():
            out = (hx.to(torch.float32) * hxs[:, None]) @ (hw.to(torch.float32) * hws[:, None]).t()
            if hb is not None:
                out = out + hb
            return out.to(torch.bfloat16)

        run.device = "cpu"  # timed with the wall-clock loop, never graph-captured
        return run

    @register_benchmark(enabled=HAS_SCALED_MM, label="hipblaslt_scaled_mm")
    def _scaled_mm(self, xq, wq, x_scale, w_scale, bias) -> Callable:
        if not xq.is_cuda:
            raise NotImplementedError("torch._scaled_mm row-wise scaling needs a GPU")
        if xq.shape[1] % 16 or wq.shape[0] % 16:
            # the library refuses these at call time with a RuntimeError; the table shows "not supported" instead
            raise NotImplementedError("torch._scaled_mm needs K and N divisible by 16")
        xs, ws = x_scale[:, None].contiguous(), w_scale[None, :].contiguous()
        return lambda: torch._scaled_mm(xq, wq.t(), scale_a=xs, scale_b=ws, bias=bias, out_dtype=torch.bfloat16)

    # ---- metrics --------------------------------------------------------------------
    @register_metric()
    def flops(self, fn_name: str, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        xq, wq, _, _, bias = example_inputs
        m, k = xq.size()
        n = wq.size(0)
        return 2 * m * n * k + (2 * m * n if bias is not None else 0)

    @staticmethod
    def _moved_bytes(example_inputs) -> int:
        xq, wq, _, _, _ = example_inputs
        m, k = xq.size()
        n = wq.size(0)
        return m * k + n * k + 2 * m * n  # fp8 A + fp8 B + bf16 C; scales and bias not counted

    @register_metric()
    def gbps(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        return self._moved_bytes(example_inputs) / 1e9 / metrics.latency * 1e3

    @register_metric()
    def mfma_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        """Fraction of the dense FP8 MFMA peak."""
        return self.flops(None, example_inputs, metrics) / metrics.latency / 1e12 * 1e3 / PEAK_FP8_TFLOPS

    @register_metric()
    def hbm_frac(self, fn, example_inputs: Any, metrics: BenchmarkOperatorMetrics) -> float:
        """Fraction of peak HBM bandwidth the algorithmic bytes would need."""
        return self.gbps(fn, example_inputs, metrics) / PEAK_HBM_GBPS

    def accuracy(self, fn: Callable, baseline_fn: Callable) -> bool:
        rtol = self.tb_args.rtol if getattr(self.tb_args, "rtol", None) is not None else self.DEFAULT_RTOL
        atol = self.tb_args.atol if getattr(self.tb_args, "atol", None) is not None else self.DEFAULT_ATOL
        try:
            out, ref = fn(), baseline_fn()
            torch.testing.assert_close(out.cpu(), ref.cpu(), rtol=rtol, atol=atol)
            return True
        except Exception as e:  # the cell reads False; the reason goes to the log, not into the void
            logger.warning("accuracy of %s against %s failed: %s", getattr(fn, "_name", fn),
                           getattr(baseline_fn, "_name", baseline_fn), str(e).strip().splitlines()[0] if str(e).strip() else repr(e))
            return False

    @register_x_val(label="(M, N, K)")
    def get_x_val(self, example_inputs) -> Tuple[int, int, int]:
        xq, wq, _, _, _ = example_inputs
        m, k = xq.size()
        n = wq.size(0)
        return (m, n, k)

    # ---- inputs ---------------------------------------------------------------------
    def get_input_iter(self) -> Generator:
        for m, n, k in self.shapes:
            x = torch.randn((m, k), device=self.device, dtype=self.input_dtype)
            w = torch.randn((n, k), device=self.device, dtype=self.input_dtype)
            if self.sigma != 1.0:
                x.mul_(self.sigma)
                w.mul_(self.sigma)
            xq, x_scale = fp8_row_quantize(x)
            wq, w_scale = fp8_row_quantize(w)
            del x, w
            bias = None
            if self.bias:
                bias = (0.1 * torch.randn((n,), device=self.device, dtype=torch.float32)).to(torch.bfloat16)
            yield xq, wq, x_scale, w_scale, bias
