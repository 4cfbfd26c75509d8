"""Registers the MI355X backend on an upstream tritonbench checkout.

Upstream keys a backend by (operator name, method name) in
tritonbench.utils.triton_op.REGISTERED_BENCHMARKS and looks the method up on the operator
class with getattr (tritonbench/utils/triton_op.py:583-616, :765-785); code outside the
operator's module registers with explicit names, as
tritonbench/operator_loader/aten/loader.py:66-71 does. Usage, before `run.py` builds the
operator (for example at the bottom of tritonbench/operators/fp8_gemm_rowwise/operator.py):

    from tritonbench_amd.upstream_plugin import register
    register(Operator)

The sibling operators that run on the same kernels register the same way: `register_grouped`,
`register_blockwise`, `register_tensorwise`, `register_fused_quant`, or `register_for(name, cls)`.

Only names importable from tritonbench.utils.triton_op are used; nothing from this
repository's own harness is involved.
"""
from typing import Callable

import torch

from . import ops

OPERATOR_NAME = "fp8_gemm_rowwise"
BACKEND_NAME = "_hip_mi355x"
LABEL = "hip_mi355x"


def _hip_mi355x(self, xq, wq, x_scale, w_scale, bias) -> Callable:
    """Backend method: same signature as the upstream `_triton` / `_cutlass_or_ck`
    methods (operator.py:187-217), returns a zero-argument callable."""
    out = torch.empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16, device=xq.device)
    workspace = ops.gemm_workspace(xq.shape[0], wq.shape[0], xq.shape[1], xq.device)
    return lambda: ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale, bias=bias, out=out, workspace=workspace)


def _register(operator_cls, operator_name: str, methods, baseline: bool) -> None:
    from tritonbench.utils.triton_op import register_benchmark  # upstream's decorator

    enabled = torch.cuda.is_available() and torch.version.hip is not None
    for position, (func_name, label, method) in enumerate(methods):
        register_benchmark(
            operator_name=operator_name, func_name=func_name, baseline=baseline and position == 0,
            enabled=enabled, label=label,
        )(method)
        setattr(operator_cls, func_name, method)


def register(operator_cls, baseline: bool = False) -> None:
    """fp8_gemm_rowwise (tritonbench/operators/fp8_gemm_rowwise/operator.py)."""
    _register(operator_cls, OPERATOR_NAME, [(BACKEND_NAME, LABEL, _hip_mi355x)], baseline)


# --- the sibling operators that share the row-wise kernels -------------------------------------

def _grouped_hip_mi355x(self, group_A, group_B, m_sizes, a_scale, b_scale) -> Callable:
    """Same signature as `_triton` / `_cutlass_or_ck` of the grouped operator
    (fp8_gemm_rowwise_grouped/operator.py:400-455): group_A [sum M, K], group_B [G*N, K],
    m_sizes on the device, read by the kernel and never by the host."""
    n = group_B.shape[0] // m_sizes.numel()
    out = torch.zeros((group_A.shape[0], n), dtype=torch.bfloat16, device=group_A.device)
    return lambda: ops.fp8_gemm_rowwise_grouped(group_A, group_B, m_sizes, a_scale, b_scale, out=out)


def register_grouped(operator_cls, baseline: bool = False) -> None:
    _register(operator_cls, "fp8_gemm_rowwise_grouped", [(BACKEND_NAME, LABEL, _grouped_hip_mi355x)], baseline)


def _blockwise_hip_mi355x(self, xq, wq, x_scale, w_scale) -> Callable:
    """Same signature as `_triton` / `_cutlass` of the block-scaled operator
    (fp8_gemm_blockwise/operator.py:139-145): x_scale [M, K/128], w_scale [N/128, K/128]."""
    out = torch.empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16, device=xq.device)
    return lambda: ops.fp8_gemm_blockwise(xq, wq, x_scale, w_scale, out=out)


def register_blockwise(operator_cls, baseline: bool = False) -> None:
    _register(operator_cls, "fp8_gemm_blockwise", [(BACKEND_NAME, LABEL, _blockwise_hip_mi355x)], baseline)


def _tensorwise_hip_mi355x(self, a, b) -> Callable:
    """Same signature as `torch_fp8_gemm` of the tensor-wise operator (fp8_gemm/fp8_gemm.py:87-101),
    and the same scales: ones of shape [M,1] / [1,N] and bf16 out under its --scaling_rowwise,
    else two one-element tensors and fp16 out."""
    if self.extra_args.scaling_rowwise:
        scale_a = torch.ones((a.shape[0], 1), dtype=torch.float32, device=a.device)
        scale_b = torch.ones((1, b.shape[1]), dtype=torch.float32, device=a.device)
        out_dtype = torch.bfloat16
    else:
        scale_a = torch.tensor(1.0, device=a.device)
        scale_b = torch.tensor(1.0, device=a.device)
        out_dtype = torch.float16
    return ops.fp8_gemm_tensorwise(a, b, scale_a, scale_b, out_dtype=out_dtype)


def register_tensorwise(operator_cls, baseline: bool = False) -> None:
    _register(operator_cls, "fp8_gemm", [(BACKEND_NAME, LABEL, _tensorwise_hip_mi355x)], baseline)


FUSED_RMS_NORM_EPS = 1e-5  # torch.ops.fbgemm.rms_norm_fp8_rowwise_quant's default, which the operator relies on


def _fused_rms_norm_hip_mi355x(self, x1, x2, wq, w_scale, wd) -> Callable:
    """Counterpart of `rms_norm_fused` (fp8_fused_quant_gemm_rowwise/operator.py:86-95): one HIP
    kernel normalises and quantises the rows, then the row-wise GEMM."""
    def run():
        xq, x_scale = ops.rms_norm_fp8_rowwise_quant(x1, wd, FUSED_RMS_NORM_EPS)
        return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

    return run


def _fused_silu_mul_hip_mi355x(self, x1, x2, wq, w_scale, wd) -> Callable:
    """Counterpart of `silu_mul_fused` (fp8_fused_quant_gemm_rowwise/operator.py:110-119)."""
    def run():
        xq, x_scale = ops.silu_mul_fp8_rowwise_quant(x1, x2)
        return ops.fp8_gemm_rowwise(xq, wq, x_scale, w_scale)

    return run


def register_fused_quant(operator_cls) -> None:
    _register(
        operator_cls, "fp8_fused_quant_gemm_rowwise",
        [("rms_norm_fused_hip_mi355x", "rms_norm_fused_hip_mi355x", _fused_rms_norm_hip_mi355x),
         ("silu_mul_fused_hip_mi355x", "silu_mul_fused_hip_mi355x", _fused_silu_mul_hip_mi355x)],
        baseline=False,
    )


REGISTRARS = {
    "fp8_gemm_rowwise": register,
    "fp8_gemm_rowwise_grouped": register_grouped,
    "fp8_gemm_blockwise": register_blockwise,
    "fp8_gemm": register_tensorwise,
    "fp8_fused_quant_gemm_rowwise": register_fused_quant,
}


def register_for(operator_name: str, operator_cls) -> None:
    """Registers the backend(s) of the named upstream operator on its class."""
    if operator_name not in REGISTRARS:
        raise KeyError(f"no MI355X backend for operator {operator_name!r}; have {sorted(REGISTRARS)}")
    REGISTRARS[operator_name](operator_cls)
