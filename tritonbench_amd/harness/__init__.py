"""Host-side benchmark harness: a small re-creation of the tritonbench surface the
`fp8_gemm_rowwise` operator needs (registries and decorators, BenchmarkOperator, metrics,
result table, latency measurement, CLI parser, operator loader)."""
from .latency import Latency, do_bench_wrapper  # noqa: F401
from .registry import (  # noqa: F401
    BASELINE_BENCHMARKS,
    REGISTERED_BENCHMARKS,
    REGISTERED_METRICS,
    REGISTERED_X_VALS,
    BenchmarkOperatorBackend,
    register_benchmark,
    register_metric,
    register_x_val,
)
from .operator_base import (  # noqa: F401
    BenchmarkOperator,
    BenchmarkOperatorMetrics,
    BenchmarkOperatorResult,
    Mode,
)
