"""Registries and decorators that tie backends, metrics and the x-axis label to an operator.

Mirrors the registration surface of tritonbench/utils/triton_op.py:84-95 (the global
tables) and :570-644 (register_x_val / register_benchmark / register_metric): a backend is a
method of the operator class, keyed by operator name; the operator name comes from the
defining module's path (`...operators.<name>.`) unless passed explicitly, which is how
code living outside the operator's module adds a backend
(tritonbench/operator_loader/aten/loader.py:66-71 does the same upstream).
"""
from collections import OrderedDict
from dataclasses import dataclass, fields
from typing import Callable, Dict, List, Optional, Set

REGISTERED_BENCHMARKS: Dict[str, "OrderedDict[str, BenchmarkOperatorBackend]"] = {}
REGISTERED_METRICS: Dict[str, List[str]] = {}
REGISTERED_X_VALS: Dict[str, str] = {}
BASELINE_BENCHMARKS: Dict[str, str] = {}
OVERRIDDEN_METRICS: Dict[str, List[str]] = {}
BASELINE_SKIP_METRICS: Set[str] = {"speedup", "accuracy", "mem_footprint_compression_ratio", "nsys_gpu_speedup"}
X_ONLY_METRICS: Set[str] = {"hw_roofline"}

_OPERATORS_MARKER = ".operators."


@dataclass
class BenchmarkOperatorBackend:
    """One registered backend (tritonbench/utils/triton_op.py:62-78)."""

    name: str  # method name on the operator class
    label: str  # what table headers show
    baseline: bool = False
    enabled: bool = True
    fwd_only: bool = False


def operator_name_from_module(module_path: str) -> str:
    """`pkg.operators.<name>.operator` -> `<name>` (triton_op.py:195-208)."""
    if _OPERATORS_MARKER not in module_path:
        raise AssertionError(
            f"cannot tell the operator from module path {module_path!r}: expected '...operators.<operator_name>...'; "
            "pass operator_name= explicitly when registering from elsewhere"
        )
    return module_path.partition(_OPERATORS_MARKER)[2].split(".")[0]


def _builtin_metric_names() -> Set[str]:
    from .operator_base import BenchmarkOperatorMetrics

    return {f.name for f in fields(BenchmarkOperatorMetrics)} - {"extra_metrics"}


def register_x_val(label: str = "x_val", operator_name: Optional[str] = None):
    def decorator(function: Callable):
        REGISTERED_X_VALS[operator_name or operator_name_from_module(function.__module__)] = label
        return function

    return decorator


def register_benchmark(
    operator_name: Optional[str] = None,
    func_name: Optional[str] = None,
    baseline: bool = False,
    enabled: bool = True,
    fwd_only: bool = False,
    label: Optional[str] = None,
):
    def decorator(function: Callable):
        op = operator_name or operator_name_from_module(function.__module__)
        name = func_name or function.__name__
        REGISTERED_BENCHMARKS.setdefault(op, OrderedDict())[name] = BenchmarkOperatorBackend(
            name=name, label=label or name, baseline=baseline, enabled=enabled, fwd_only=fwd_only
        )
        if baseline:
            BASELINE_BENCHMARKS[op] = name
        return function

    return decorator


def register_metric(skip_baseline: bool = False, x_only: bool = False, operator_name: Optional[str] = None):
    """skip_baseline: not reported for the baseline backend (like speedup);
    x_only: one column per input instead of one per backend (like hw_roofline)."""

    def decorator(function: Callable):
        op = operator_name or operator_name_from_module(function.__module__)
        name = function.__name__
        if name in _builtin_metric_names():
            OVERRIDDEN_METRICS.setdefault(op, []).append(name)
        else:
            lst = REGISTERED_METRICS.setdefault(op, [])
            if name not in lst:
                lst.append(name)
        if skip_baseline:
            BASELINE_SKIP_METRICS.add(name)
        if x_only:
            X_ONLY_METRICS.add(name)
        return function

    return decorator


def enabled_benchmarks(op_name: str, mode_is_backward: bool, skip: List[str]) -> List[str]:
    """Backends that are enabled, not skipped and able to run in this mode
    (triton_op.py:545-567)."""
    out = []
    for name, cfg in REGISTERED_BENCHMARKS.get(op_name, {}).items():
        if name in skip or not cfg.enabled:
            continue
        if mode_is_backward and cfg.fwd_only:
            continue
        out.append(name)
    return out
