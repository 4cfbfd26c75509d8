"""`cuda_time` metric: device time of the kernels one call launches, cold caches.

The upstream metric (tritonbench/components/do_bench/cuda_time.py:12-110) profiles repeated
`cache.zero_(); fn()` pairs with the PyTorch profiler and adds up, per call, the durations of
every device kernel except the cache-clearing fill, which it recognises by its full CUDA
kernel name. Here the fill is recognised by the functor it instantiates (`FillFunctor<int>`: the
flush buffer is int32; the same on ROCm and CUDA builds, whatever the rest of the template spells), the flush buffer is
twice the MI355X memory-side cache (upstream's 256 MB equals that cache and leaves operands
in it), and a call's kernels are the ones between two fills in start order, so backends that
launch a different number of kernels per call (a split-K plan launches two) need no
special case. Unlike `latency` this leaves out launch gaps and host time."""
from typing import Callable, List

from .latency import FLUSH_BYTES, Latency

# the flush buffer is int32, so its fill instantiates FillFunctor<int>: a backend whose callable
# zero-fills its own (bf16, float, ...) output inside the call is not mistaken for the flush
FLUSH_KERNEL_MARK = "FillFunctor<int>"


def split_calls(events) -> List[float]:
    """events: (start, duration_us, name) of device kernels. Returns ms per call: the sum of
    the kernels that follow each flush kernel, up to the next one."""
    calls, cur = [], None
    for _, dur_us, name in sorted(events):
        if FLUSH_KERNEL_MARK in name:
            if cur is not None:
                calls.append(cur)
            cur = 0.0
        elif cur is not None:
            cur += dur_us / 1e3
    if cur is not None:
        calls.append(cur)
    return calls


def do_bench_cuda_time(fn: Callable, warmup: float, rep: float, max_calls: int = 200) -> Latency:
    import torch
    from torch.profiler import ProfilerActivity, profile

    flush = torch.empty(FLUSH_BYTES // 4, dtype=torch.int32, device="cuda")
    fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        flush.zero_()
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate_ms = max(start.elapsed_time(end) / 5, 1e-3)
    n_warmup = max(1, min(max_calls, int(warmup / estimate_ms)))
    n_repeat = max(1, min(max_calls, int(rep / estimate_ms)))
    for _ in range(n_warmup):
        flush.zero_()
        fn()
    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        for _ in range(n_repeat):
            flush.zero_()
            fn()
        torch.cuda.synchronize()
    device = torch.autograd.DeviceType.CUDA
    events = [(e.time_range.start, e.device_time, e.name) for e in prof.events() if e.device_type == device]
    calls = split_calls(events)
    if len(calls) != n_repeat or not all(c > 0 for c in calls):
        raise RuntimeError(f"cuda_time: expected {n_repeat} profiled calls with device kernels, found {len(calls)}")
    return Latency(times=calls)
