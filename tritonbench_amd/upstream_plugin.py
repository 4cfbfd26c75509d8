"""Registers the MI355X backend on an upstream tritonbench checkout.

Upstream keys a backend by (operator name, method name) in
tritonbench.utils.triton_op.REGISTERED_BENCHMARKS and looks the method up on the operator
class with getattr (tritonbench/utils/triton_op.py:583-616, :765-785); code outside the
operator's module registers with explicit names, as
tritonbench/operator_loader/aten/loader.py:66-71 does. Usage, before `run.py` builds the
operator (for example at the bottom of tritonbench/operators/fp8_gemm_rowwise/operator.py):

    from tritonbench_amd.upstream_plugin import register
    register(Operator)

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


def register(operator_cls, baseline: bool = False) -> None:
    from tritonbench.utils.triton_op import register_benchmark  # upstream's decorator

    enabled = torch.cuda.is_available() and torch.version.hip is not None
    register_benchmark(
        operator_name=OPERATOR_NAME, func_name=BACKEND_NAME, baseline=baseline, enabled=enabled, label=LABEL
    )(_hip_mi355x)
    setattr(operator_cls, BACKEND_NAME, _hip_mi355x)
