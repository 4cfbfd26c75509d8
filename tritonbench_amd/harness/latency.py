"""Latency container and timing loops.

Behaviour follows tritonbench/components/do_bench/run.py: `Latency` (:12-114) drops IQR
outliers, reports p50 = median_low and does arithmetic on p50; `_do_bench_cpu` (:128-166)
is a wall-clock loop; `do_bench_wrapper` (:169-213) picks CPU, graph-captured or eager
device timing. The device loops are written here against torch.cuda events and graphs
directly (the upstream ones call triton.testing).
"""
import statistics
import time
from typing import Callable, List, Optional

NS_TO_MS = 1e-6
FLUSH_BYTES = 512 * 1024 * 1024  # > the 256 MB memory-side cache, so a flush really evicts


class Latency:
    def __init__(self, times: List[float]):
        self.times = self._drop_outliers(list(times))

    @staticmethod
    def _drop_outliers(data: List[float]) -> List[float]:
        n = len(data)
        if n <= 3:
            return data
        data.sort()
        cuts = statistics.quantiles(data, n=100)
        q1, q3 = cuts[25], cuts[75]
        lo, hi = q1 - 1.5 * (q3 - q1), q3 + 1.5 * (q3 - q1)
        kept = [x for x in data if lo <= x <= hi]
        if len(kept) != n:
            print(f"Removed {n - len(kept)} outliers from {n} samples")
        return kept

    @property
    def p50(self) -> float:
        return statistics.median_low(self.times)

    @property
    def min(self) -> float:
        return min(self.times)

    @property
    def max(self) -> float:
        return max(self.times)

    @staticmethod
    def _v(x):
        return x.p50 if isinstance(x, Latency) else x

    def __add__(self, o): return self.p50 + self._v(o)
    def __radd__(self, o): return self._v(o) + self.p50
    def __sub__(self, o): return self.p50 - self._v(o)
    def __rsub__(self, o): return self._v(o) - self.p50
    def __mul__(self, o): return self.p50 * self._v(o)
    def __rmul__(self, o): return self._v(o) * self.p50
    def __truediv__(self, o): return self.p50 / self._v(o)
    def __rtruediv__(self, o): return self._v(o) / self.p50
    def __floordiv__(self, o): return self.p50 // self._v(o)
    def __rfloordiv__(self, o): return self._v(o) // self.p50

    def __str__(self) -> str:
        return self.to_str()

    def to_str(self, mode: str = "p50") -> str:
        if mode == "p50":
            return str(self.p50)
        if mode == "with_variance":
            spread = max(self.max - self.p50, self.p50 - self.min) / self.p50
            return f"{self.p50:6f} (±{spread * 100:.2f}%)"
        if mode == "max":
            return str(self.max)
        if mode == "min":
            return str(self.min)
        if mode == "mean":
            return str(statistics.mean(self.times))
        raise ValueError(f"Unsupported latency output mode: {mode}")


def do_bench_cpu(fn: Callable, warmup: float, rep: float, grad_to_none=None) -> List[float]:
    """Wall-clock ms per call: 1 call, a 5-call estimate, then warmup/rep milliseconds worth
    of calls, each timed with time_ns (do_bench/run.py:128-166)."""
    fn()
    t0 = time.time_ns()
    for _ in range(5):
        fn()
    estimate_ms = (time.time_ns() - t0) * NS_TO_MS / 5
    n_warmup = max(1, int(warmup / estimate_ms)) if estimate_ms > 0 else 1
    n_repeat = max(1, int(rep / estimate_ms)) if estimate_ms > 0 else 1
    for _ in range(n_warmup):
        fn()
    out = []
    for _ in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        t0 = time.time_ns()
        fn()
        out.append((time.time_ns() - t0) * NS_TO_MS)
    return out


def do_bench_graph(fn: Callable, rep: float = 100, n_replays: int = 10) -> List[float]:
    """Device ms per call from a captured graph of back-to-back calls, replayed
    `n_replays` times. Caches are NOT flushed between calls: what a steady-state serving
    loop sees, and what the upstream operator reports (it sets use_cuda_graphs,
    operators/fp8_gemm_rowwise/operator.py:156)."""
    import torch

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(5):
            fn()
        end.record()
        torch.cuda.synchronize()
        estimate_ms = start.elapsed_time(end) / 5
        n_repeat = 1000 if estimate_ms == 0 else max(1, int(rep / estimate_ms))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(n_repeat):
                fn()
        torch.cuda.synchronize()
        out = []
        for _ in range(n_replays):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            graph.replay()
            end.record()
            torch.cuda.synchronize()
            out.append(start.elapsed_time(end) / n_repeat)
    torch.cuda.synchronize()
    return out


_flush_buf = None


def do_bench_eager(fn: Callable, warmup: float, rep: float, grad_to_none=None) -> List[float]:
    """Device ms per call, one event pair per call, with a cache-evicting fill in front of
    every timed call."""
    import torch

    global _flush_buf
    if _flush_buf is None:
        _flush_buf = torch.empty(FLUSH_BYTES // 4, dtype=torch.int32, device="cuda")
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        _flush_buf.zero_()
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate_ms = start.elapsed_time(end) / 5
    n_warmup = max(1, int(warmup / estimate_ms))
    n_repeat = max(1, int(rep / estimate_ms))
    for _ in range(n_warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        _flush_buf.zero_()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    return [s.elapsed_time(e) for s, e in zip(starts, ends)]


def do_bench_wrapper(
    fn: Callable,
    warmup: float,
    rep: float,
    grad_to_none: Optional[list],
    device: str = "cuda",
    use_cuda_graphs: bool = False,
    bypass_fail: bool = False,
) -> Optional[Latency]:
    """Same contract as do_bench/run.py:169-213: returns Latency, or None when the call
    failed and bypass_fail is set."""
    try:
        if device == "cpu":
            return Latency(do_bench_cpu(fn, warmup, rep, grad_to_none))
        if use_cuda_graphs:
            return Latency(do_bench_graph(fn, rep))
        return Latency(do_bench_eager(fn, warmup, rep, grad_to_none))
    except Exception as e:
        if not bypass_fail:
            raise
        print(f"do_bench failed ({e!r}); bypassing")
        return None
