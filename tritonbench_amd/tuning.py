"""Measured choice of kernel family and plan for one shape.

The library picks a kernel family, tile configuration and split factor from tables of measured
constants (no call ever times anything). This module is the other way to choose: it times every
candidate plan for a shape on the device and remembers the fastest, the way the reference's FBGEMM
kernels are autotuned per shape by Triton (`matmul_fp8_row`, reached from
tritonbench/operators/fp8_gemm_rowwise/operator.py:187-199). It is used by the operator's
`_hip_mi355x_autotuned` backend, outside the timed callable, and by the test that holds the
library's own choice against the measured best.

Timing follows how the benchmarks time: a captured graph of 16 launches over rotating operand
sets (cold weights, as a model's are), sustained bursts of a few milliseconds, the median of
three.
"""
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib, ops

# (m, n, k, bias, device index) -> (variant word, microseconds, {candidate name: microseconds})
_CACHE: Dict[Tuple[int, int, int, bool, int], Tuple[int, float, Dict[str, float]]] = {}

OperandSet = Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor], torch.Tensor]


def candidates(m: int, n: int, k: int) -> Dict[str, int]:
    """Every pinned plan the library can run the shape with: name -> variant word."""
    if k % 16:
        return {"generic": _lib.VARIANT_GENERIC}
    out = {f"tiled config {c}": _lib.tiled_variant(c, 0) for c in range(_lib.NUM_TILE_CONFIGS)}
    if m <= 64:
        out["skinny"] = _lib.VARIANT_SKINNY
        out["skinny, one tile per workgroup"] = _lib.VARIANT_SKINNY | _lib.SKINNY_ONE_TILE
    # (the narrow-tile form also takes up to 256 rows where 64x64 tiles are one round of workgroups)
    if _lib.skinny_family_takes(m, n):
        out["skinny, narrow tiles"] = _lib.VARIANT_SKINNY | _lib.SKINNY_NARROW
    return out


def make_operand_sets(m: int, n: int, k: int, bias: bool, device, seed: int = 0, min_bytes: int = 600_000_000,
                      max_sets: int = 10) -> List[OperandSet]:
    """Quantised random operands to rotate through: more than twice the 256 MB memory-side cache in
    total where the count allows, so that the weights of a call come from HBM."""
    g = torch.Generator(device=device).manual_seed(seed + m + n + k)
    sets = []
    for _ in range(min(max_sets, max(4, min_bytes // (n * k) + 1))):
        xq, xs = ops.fp8_row_quantize(torch.randn((m, k), generator=g, device=device))
        wq, w_s = ops.fp8_row_quantize(torch.randn((n, k), generator=g, device=device))
        b = (0.1 * torch.randn((n,), generator=g, device=device)).to(torch.bfloat16) if bias else None
        sets.append((xq, wq, xs, w_s, b, torch.empty((m, n), dtype=torch.bfloat16, device=device)))
    return sets


def time_variant_us(sets: Sequence[OperandSet], variant: int, burst_us: float = 6000.0) -> float:
    """Microseconds per call of `variant` on the shape of `sets`."""
    xq0, wq0 = sets[0][0], sets[0][1]
    m, k = xq0.shape
    n = wq0.shape[0]
    dev = xq0.device
    ws = ops.gemm_workspace(m, n, k, dev, variant)
    # A fresh stream per call, on purpose: the time of a launch depends on the hardware queue its stream
    # is mapped to (one captured graph replayed on consecutively created streams: 12.2 / 11.5 / 12.2 /
    # 13.2 us per launch of 8 x 3072 x 16384, and the same again on the next four), so callers that take
    # the best of several calls see every plan on several queues.
    stream = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(stream):
        def call(i):
            xq, wq, xs, w_s, b, out = sets[i % len(sets)]
            ops.fp8_gemm_rowwise(xq, wq, xs, w_s, bias=b, out=out, workspace=ws, variant=variant)
        call(0)
        torch.cuda.synchronize(dev)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(16):
                call(i)
        g.replay()
        torch.cuda.synchronize(dev)

        # Sustained bursts (as the benchmark times its rows), the median of three: the cost tables are
        # calibrated on mean step times under sustained load, and short bursts flatter the candidates
        # that are bound by HBM.
        def burst(replays):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(stream)
            for _ in range(replays):
                g.replay()
            end.record(stream)
            torch.cuda.synchronize(dev)
            return start.elapsed_time(end) * 1e3 / (16 * replays)
        replays = max(1, int(burst_us / (16 * max(burst(1), 1.0))))
        samples = [burst(replays) for _ in range(3)]
    return sorted(samples)[len(samples) // 2]


def autotune(m: int, n: int, k: int, device, bias: bool = False, sets: Optional[Sequence[OperandSet]] = None,
             rounds: int = 2) -> Tuple[int, float, Dict[str, float]]:
    """Times every candidate plan of the shape (best of `rounds` passes over all of them) and
    returns (variant word of the fastest, its microseconds, all timings by name). Cached per
    shape, bias and device for the life of the process."""
    device = torch.device(device)
    key = (m, n, k, bool(bias), device.index or 0)
    if key in _CACHE:
        return _CACHE[key]
    if sets is None:
        sets = make_operand_sets(m, n, k, bias, device)
    cands = candidates(m, n, k)
    times = {name: float("inf") for name in cands}
    for _ in range(rounds):
        for name, v in cands.items():
            times[name] = min(times[name], time_variant_us(sets, v))
    best = min(times, key=times.get)
    _CACHE[key] = (cands[best], times[best], times)
    return _CACHE[key]


def clear_cache() -> None:
    _CACHE.clear()
