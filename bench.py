"""Benchmark of the row-wise FP8 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra] [--vendor]

One step = one pass of the hot path (one mi355x_fp8_rowwise_gemm call through the C ABI) over
the headline workload M=N=K=8192 with operands resident in HBM. Prints ONE JSON line: the
headline TFLOP/s, the roofline of the dominant kernel measured with HIP events on the launch
stream, the CPU baseline (the oracle's fp32 dequantise + torch.matmul, timed on this machine's
host cores), the HBM-bound headline (M=16) with a roofline block of its own, and under
"configs" one row per benchmark configuration (microseconds, TFLOP/s, GB/s, bound, fraction of
that bound's peak): the decode shape, all twenty Llama-3-70B projection shapes, the two ragged
shapes with bias (each of these with its own CPU baseline where that takes seconds), and the
neighbouring kernels (grouped, block-scaled, quantiser).

The device runs its first milliseconds of matrix work after an idle spell well below the
sustained clock, so whatever --warmup says the workload is launched untimed for --preheat-ms
first; the K timed steps follow at once.
"""
import argparse
import hashlib
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # dense FP8 MFMA, MI355X datasheet
PEAK_HBM_GBPS = 8000.0    # HBM3E, MI355X datasheet
SEED = 1337
KERNEL_SOURCE = os.path.join(ROOT, "tritonbench_amd", "csrc", "fp8_rowwise_gemm.hip")
TRAFFIC_FILES = {  # written by `python -m tritonbench_amd.harness.traffic` from two rocprofv3 counter passes
    "tiled": os.path.join(ROOT, "profiles", "tiled_8192cubed_traffic.json"),
    "skinny": os.path.join(ROOT, "profiles", "skinny_16x8192x8192_traffic.json"),
}
LLAMA3_70B_NK = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]
LLAMA3_70B_M = [1, 32, 128, 1024, 4096]
# the reference operator's own default sweep (tritonbench/operators/fp8_gemm_rowwise/operator.py:107-128);
# entry 7, (16, 13312, 13312), is the shape of its one stored run configuration
# (benchmarks/run_config/fp8_gemm_rowwise_fwd.yaml:1-3)
REFERENCE_BUILTIN_SHAPES = [
    (1, 2304, 2048), (1, 8192, 16384), (4, 4096, 2304), (4, 13312, 2048), (8, 2304, 2304),
    (8, 8192, 6656), (16, 4096, 6656), (16, 13312, 13312), (32, 2304, 16384), (32, 8192, 13312),
    (64, 4096, 2048), (64, 13312, 2048), (128, 2304, 6656), (128, 8192, 2304), (2048, 8192, 2048),
    (2048, 13312, 6656), (4096, 2304, 13312), (4096, 13312, 2304), (16384, 4096, 16384),
    (16384, 8192, 13312),
]


def source_sha() -> str:
    with open(KERNEL_SOURCE, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def measured_traffic(which: str):
    """HBM-side bytes per launch from the committed counter summary, or None. The summary names
    the kernel source it was measured on: a figure from an older source is still reported, marked
    stale, so that it cannot pass for a measurement of the present kernel."""
    path = TRAFFIC_FILES[which]
    if not os.path.exists(path):
        return None, {"traffic_source": None}
    with open(path) as f:
        t = json.load(f)
    note = {"traffic_source": os.path.relpath(path, ROOT), "traffic_kernel": t.get("kernel"),
            "traffic_stale": t.get("source_sha") != source_sha()}
    return t.get("traffic_bytes"), note


def _generator(dev, *key):
    g = torch.Generator(device=dev)
    g.manual_seed(SEED + sum(int(k) * w for k, w in zip(key, (7, 3, 1, 11))))
    return g


def make_weights(n, k, sigma, bias, dev, copies):
    """`copies` independent (wq, w_scale, bias) sets, generated and quantised on the device (the
    HIP quantiser is bit-exact against the oracle)."""
    from tritonbench_amd import ops

    g = _generator(dev, 0, n, k)
    sets = []
    for _ in range(copies):
        w = torch.randn((n, k), generator=g, device=dev, dtype=torch.float32) * sigma
        wq, ws = ops.fp8_row_quantize(w)
        del w
        b = (0.1 * torch.randn((n,), generator=g, device=dev, dtype=torch.float32)).to(torch.bfloat16) if bias else None
        sets.append((wq, ws, b))
    return sets


def make_sets(m, weights, sigma, dev):
    """One operand set per weight copy: (xq, wq, x_scale, w_scale, bias, out). Rotating through
    sets larger than the caches means no call finds its operands in L2 or the 256 MB memory-side
    cache."""
    from tritonbench_amd import ops

    n, k = weights[0][0].shape
    g = _generator(dev, m, n, k)
    sets = []
    for (wq, ws, b) in weights:
        x = torch.randn((m, k), generator=g, device=dev, dtype=torch.float32) * sigma
        xq, xs = ops.fp8_row_quantize(x)
        sets.append((xq, wq, xs, ws, b, torch.empty((m, n), dtype=torch.bfloat16, device=dev)))
    return sets, ops.gemm_workspace(m, n, k, dev)


def copies_for(n, k, cap=8):
    """Operand sets needed for the rotation to out-run the 256 MB memory-side cache."""
    return max(2, min(cap, int(600e6 // (n * k)) + 1))


def launch(s, workspace):
    from tritonbench_amd import ops

    xq, wq, xs, ws, b, out = s
    ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=workspace)


def preheat(sets, workspace, ms):
    """Untimed launches of the workload for about `ms` milliseconds of wall time."""
    t0, i = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(10):
            launch(sets[i % len(sets)], workspace)
            i += 1
        torch.cuda.synchronize()


def time_steps(sets, workspace, steps, warmup):
    """Average ms per call over exactly `steps` calls, HIP events on the launch stream."""
    stream = torch.cuda.current_stream()
    for i in range(warmup):
        launch(sets[i % len(sets)], workspace)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for i in range(steps):
        launch(sets[i % len(sets)], workspace)
    end.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_steps_graph(sets, workspace, steps, warmup, preheat_ms, replays=5):
    """The headline's timed region as the reference operator times its backends
    (use_cuda_graphs, tritonbench/operators/fp8_gemm_rowwise/operator.py:156): exactly `steps` calls
    recorded into one HIP graph; `warmup` eager calls first, then untimed replays for `preheat_ms`
    (recording the graph leaves the device idle for tens of milliseconds and its clock falls back);
    then ONE replay between two events on the graph's stream, synchronised on both sides. Returns
    (ms per step of that replay, [ms per step of `replays` further replays])."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(max(warmup, 1)):
            launch(sets[i % len(sets)], workspace)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for i in range(steps):
                launch(sets[i % len(sets)], workspace)
        t0 = time.perf_counter()
        g.replay()
        while (time.perf_counter() - t0) * 1e3 < preheat_ms:
            g.replay()
        torch.cuda.synchronize()

        def one():
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record(side)
            g.replay()
            end.record(side)
            torch.cuda.synchronize()
            return start.elapsed_time(end) / steps

        timed = one()
        more = [one() for _ in range(replays)]
    return timed, more


def time_graph(call, steps, min_replay_ms=6.0, preheat_ms=30.0, replays=5):
    """ms per call of call(i) with the calls captured in one HIP graph (no per-launch host gaps:
    how the benchmark harness times the operator). The graph holds at least `steps` calls and
    enough of them for a replay to last `min_replay_ms`; replays run untimed for `preheat_ms`
    first. Returns (best, median) over `replays` timed replays."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        call(0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(5):
            call(i)
        torch.cuda.synchronize()
        est_ms = max((time.perf_counter() - t0) * 1e3 / 5, 1e-3)
        steps = int(min(max(steps, min_replay_ms / est_ms), 2000))
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for i in range(steps):
                call(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < preheat_ms:
            g.replay()
            torch.cuda.synchronize()
        times = []
        for _ in range(replays):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(side)
            g.replay()
            end.record(side)
            torch.cuda.synchronize()
            times.append(start.elapsed_time(end) / steps)
    return min(times), statistics.median(times)


def figures(m, n, k, bias, ms, ms_median=None):
    flops = 2 * m * n * k + (2 * m * n if bias else 0)
    nbytes = m * k + n * k + 2 * m * n
    tflops = flops / ms / 1e9
    gbps = nbytes / ms / 1e6
    t_mfma = flops / (PEAK_FP8_TFLOPS * 1e12)
    t_hbm = nbytes / (PEAK_HBM_GBPS * 1e9)
    bound = "mfma" if t_mfma >= t_hbm else "hbm"
    frac = tflops / PEAK_FP8_TFLOPS if bound == "mfma" else gbps / PEAK_HBM_GBPS
    row = dict(us=ms * 1e3, tflops=tflops, gbps=gbps, bound=bound, frac=frac)
    if ms_median is not None:
        row["us_median"] = ms_median * 1e3
    return row


VENDOR = False  # --vendor: time torch._scaled_mm (hipBLASLt's row-wise FP8 GEMM) on the same operand sets


def vendor_us(sets, steps):
    """Microseconds per call of torch._scaled_mm with row-wise scales on the same rotated operand
    sets, timed like our own rows (captured graph, best replay); None where the library refuses
    the shape. The scale views are made once, outside the timed calls."""
    prepared = [(xq, wq.t(), xs[:, None].contiguous(), ws[None, :].contiguous(), b) for (xq, wq, xs, ws, b, _) in sets]

    def call(i):
        a, bt, sa, sb, bias = prepared[i % len(prepared)]
        torch._scaled_mm(a, bt, scale_a=sa, scale_b=sb, bias=bias, out_dtype=torch.bfloat16)

    try:
        best, _ = time_graph(call, steps)
    except Exception as e:  # noqa: BLE001 - e.g. N or K not a multiple of 16
        print(f"bench.py: torch._scaled_mm refused {tuple(sets[0][0].shape)} x {tuple(sets[0][1].shape)}: {e}",
              file=sys.stderr, flush=True)
        return None
    return best * 1e3


def gemm_row(m, sets, workspace, steps):
    xq, wq, _, _, b, _ = sets[0]
    best, med = time_graph(lambda i: launch(sets[i % len(sets)], workspace), steps)
    row = figures(m, wq.shape[0], wq.shape[1], b is not None, best, med)
    if VENDOR:
        row["hipblaslt_us"] = vendor_us(sets, steps)
    return row


def timed_calls(call, steps, preheat_ms=30.0):
    """ms per call of call(i) over `steps` calls (HIP events on the launch stream), after untimed
    calls for `preheat_ms`."""
    call(0)  # (the first call of a kernel loads its code object: not part of the preheat)
    torch.cuda.synchronize()
    t0, i = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < preheat_ms:
        for _ in range(5):
            call(i)
            i += 1
        torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for i in range(steps):
        call(i)
    end.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_quantiser(r, k, dtype, dev, steps=60, copies=3):
    """Row-wise quantiser (the step in front of the GEMM): algorithmic bytes = source + fp8
    output + one f32 scale per row; sources rotate so no call finds its row in a cache."""
    from tritonbench_amd import ops

    g = _generator(dev, r, k)
    xs = [torch.randn((r, k), generator=g, device=dev, dtype=torch.float32).to(dtype) for _ in range(copies)]
    ms = timed_calls(lambda i: ops.fp8_row_quantize(xs[i % copies]), steps)
    nbytes = r * k * (xs[0].element_size() + 1) + 4 * r
    return dict(us=ms * 1e3, gbps=nbytes / ms / 1e6, bound="hbm", frac=nbytes / ms / 1e6 / PEAK_HBM_GBPS)


def time_block_quantiser(r, k, dtype, dev, steps=60, copies=3):
    """128 x 128 block-wise quantiser (the input step of the block-scaled GEMM): algorithmic bytes =
    source + fp8 output + one f32 scale per block; sources rotate."""
    from tritonbench_amd import ops

    g = _generator(dev, r, k, 9)
    xs = [torch.randn((r, k), generator=g, device=dev, dtype=torch.float32).to(dtype) for _ in range(copies)]
    ms = timed_calls(lambda i: ops.fp8_block_quantize(xs[i % copies]), steps)
    nbytes = r * k * (xs[0].element_size() + 1) + 4 * (-(-r // 128)) * (-(-k // 128))
    return dict(us=ms * 1e3, gbps=nbytes / ms / 1e6, bound="hbm", frac=nbytes / ms / 1e6 / PEAK_HBM_GBPS)


def time_fused_front_end(which, r, k, dev, steps=60, copies=3):
    """Fused front ends (RMSNorm or SiLU-mul, then the row-wise quantiser, one kernel): algorithmic
    bytes = the bf16 source row(s) + fp8 output + one f32 scale per row (the RMSNorm weight vector is
    shared by all rows and stays in cache); sources rotate."""
    from tritonbench_amd import ops

    g = _generator(dev, r, k, 5)
    x1 = [torch.randn((r, k), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(copies)]
    if which == "rmsnorm":
        w = torch.randn((k,), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        ms = timed_calls(lambda i: ops.rms_norm_fp8_rowwise_quant(x1[i % copies], w), steps)
        nbytes = r * k * 3 + 4 * r + 2 * k
    else:
        x2 = [torch.randn((r, k), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16) for _ in range(copies)]
        ms = timed_calls(lambda i: ops.silu_mul_fp8_rowwise_quant(x1[i % copies], x2[i % copies]), steps)
        nbytes = r * k * 5 + 4 * r
    return dict(us=ms * 1e3, gbps=nbytes / ms / 1e6, bound="hbm", frac=nbytes / ms / 1e6 / PEAK_HBM_GBPS)


def time_grouped(g, m, n, k, dev, steps=40, copies=2):
    """Grouped form (equal groups, as the reference's input generator makes them):
    flops = 2*M*N*K, bytes = M*K + G*N*K + 2*M*N."""
    from tritonbench_amd import ops

    gen = _generator(dev, g, m, n, k)
    sets = []
    for _ in range(copies):
        xq, xs = ops.fp8_row_quantize(torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32))
        wq, ws = ops.fp8_row_quantize(torch.randn((g * n, k), generator=gen, device=dev, dtype=torch.float32))
        sets.append((xq, wq, xs, ws, torch.zeros((m, n), dtype=torch.bfloat16, device=dev)))
    sizes = torch.tensor([m // g] * g, dtype=torch.int32, device=dev)

    def call(i):
        xq, wq, xs, ws, out = sets[i % copies]
        ops.fp8_gemm_rowwise_grouped(xq, wq, sizes, xs, ws, out=out)

    ms = timed_calls(call, steps)
    flops, nbytes = 2 * m * n * k, m * k + g * n * k + 2 * m * n
    return dict(us=ms * 1e3, tflops=flops / ms / 1e9, gbps=nbytes / ms / 1e6, bound="mfma",
                frac=flops / ms / 1e9 / PEAK_FP8_TFLOPS)


def time_blockwise(m, n, k, dev, steps=30):
    """Block-scaled form (128x128 blocks of seeded N(0,1) data, quantised on the device with
    torch ops as the reference's input generator does): flops = 2*M*N*K."""
    from tritonbench_amd import ops
    from tritonbench_amd.operators.fp8_gemm_blockwise.operator import fp8_block_quantize

    gen = _generator(dev, 5 * m, n, k)
    xq, xs = fp8_block_quantize(torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32))
    wq, ws = fp8_block_quantize(torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32))
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ms = timed_calls(lambda i: ops.fp8_gemm_blockwise(xq, wq, xs, ws, out=out), steps)
    flops, nbytes = 2 * m * n * k, m * k + n * k + 2 * m * n
    return dict(us=ms * 1e3, tflops=flops / ms / 1e9, gbps=nbytes / ms / 1e6, bound="mfma",
                frac=flops / ms / 1e9 / PEAK_FP8_TFLOPS)


def cpu_weight(s):
    """The weight of operand set `s` on the host, dequantised to fp32 (the first half of the CPU path);
    returns (tensor, seconds). Rows of one (N, K) pair share it across their M sweep."""
    from oracle import fp8_rowwise as orc

    _, wq, _, ws, _, _ = s
    hwq, hws = wq.cpu(), ws.cpu()
    orc.dequantize(hwq[:64], hws[:64])  # (pages the conversion code in)
    t0 = time.perf_counter()
    w = orc.dequantize(hwq, hws)
    return w, time.perf_counter() - t0


def cpu_baseline(s, what, budget_s=12.0, max_calls=5, weight=None):
    """The oracle (fp32 dequantise + torch.matmul) on host cores, on the same operands, the two
    halves timed separately. `weight` = (dequantised fp32 weight, seconds it took) from cpu_weight()
    when several rows share one weight: its time is charged to every row as if it had been redone."""
    from oracle import fp8_rowwise as orc

    xq, wq, xs, ws, b, _ = s
    hxq, hxs = xq.cpu(), xs.cpu()
    hb = None if b is None else b.cpu()
    m, k = hxq.shape
    n = wq.shape[0]
    flops = 2 * m * n * k + (2 * m * n if b is not None else 0)
    if weight is None:
        weight = cpu_weight(s)
    w, w_seconds = weight
    t0 = time.perf_counter()
    a = orc.dequantize(hxq, hxs)
    deq = w_seconds + (time.perf_counter() - t0)
    # (a call that takes a second is timed once; short ones take the best of a few after a warm-up)
    t0 = time.perf_counter()
    orc.dequant_matmul_rows(a, w, hb)
    first = time.perf_counter() - t0
    times, spent = [first] if first > 0.5 else [], first
    while spent < budget_s and len(times) < max_calls and first <= 0.5 * budget_s:
        t0 = time.perf_counter()
        orc.dequant_matmul_rows(a, w, hb)
        dt = time.perf_counter() - t0
        times.append(dt)
        spent += dt
    mm = min(times) if times else first
    total = deq + mm
    return {
        "value": flops / total / 1e12,
        "unit": "TFLOP/s",
        "gbps": (m * k + n * k + 2 * m * n) / total / 1e9,
        "ms": total * 1e3,
        "dequant_ms": deq * 1e3,
        "matmul_ms": mm * 1e3,
        "cores": torch.get_num_threads(),
        "cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": f"full {what} workload: fp32 dequantise of both operands ({deq:.4f} s) + torch.matmul, bias and bf16 rounding "
                  f"({mm:.4f} s, best of {max(len(times), 1)} call(s))",
    }


def profile_kernel(which, dev):
    """A short run of one kernel's workload for rocprofv3 counter passes, preceded by a copy
    kernel of known size (an elementwise negation of a 256 MiB tensor: reads it once, writes as
    much) that the counter readings are scaled by."""
    cal = torch.ones((8192, 8192), dtype=torch.float32, device=dev)
    for _ in range(3):
        torch.neg(cal)  # (a negation: no other kernel of the run shares its name)
    torch.cuda.synchronize()
    if which == "tiled":
        sets, wsp = make_sets(8192, make_weights(8192, 8192, 1.0, False, dev, 1), 1.0, dev)
        fig = figures(8192, 8192, 8192, False, time_steps(sets, wsp, 20, 5))
    elif which == "tiled_cold":  # (five operand sets: A and B of a call come from HBM, not from the memory-side cache)
        sets, wsp = make_sets(8192, make_weights(8192, 8192, 1.0, False, dev, 5), 1.0, dev)
        fig = figures(8192, 8192, 8192, False, time_steps(sets, wsp, 20, 5))
    elif which == "skinny":
        sets, wsp = make_sets(16, make_weights(8192, 8192, 1.0, False, dev, 10), 1.0, dev)
        fig = figures(16, 8192, 8192, False, time_steps(sets, wsp, 40, 10))
    elif which == "quantise":
        fig = {"f32": time_quantiser(8192, 8192, torch.float32, dev, steps=20),
               "bf16": time_quantiser(8192, 8192, torch.bfloat16, dev, steps=20)}
    elif which == "fused":
        fig = {"rmsnorm": time_fused_front_end("rmsnorm", 8192, 8192, dev, steps=20),
               "silu_mul": time_fused_front_end("silu_mul", 8192, 8192, dev, steps=20)}
    elif which == "grouped":
        fig = time_grouped(4, 8192, 4096, 4096, dev, steps=20)
    elif which == "decode128":
        sets, wsp = make_sets(128, make_weights(8192, 8192, 0.02, False, dev, 8), 0.02, dev)
        fig = figures(128, 8192, 8192, False, time_steps(sets, wsp, 40, 10))
    elif which == "decode128_n10240":  # (more 64-column tiles than fit one round: the split-K pair of kernels)
        sets, wsp = make_sets(128, make_weights(10240, 8192, 0.02, False, dev, 8), 0.02, dev)
        fig = figures(128, 10240, 8192, False, time_steps(sets, wsp, 40, 10))
    elif which == "decode128_n57344":  # (one tile row against the widest panel of the sweep: 128x256 tiles, all of K each)
        sets, wsp = make_sets(128, make_weights(57344, 8192, 0.02, False, dev, 2), 0.02, dev)
        fig = figures(128, 57344, 8192, False, time_steps(sets, wsp, 40, 10))
    elif which == "decode32":
        sets, wsp = make_sets(32, make_weights(8192, 8192, 0.02, False, dev, 8), 0.02, dev)
        fig = figures(32, 8192, 8192, False, time_steps(sets, wsp, 40, 10))
    elif which == "ragged":
        sets, wsp = make_sets(1000, make_weights(3000, 4112, 1.0, True, dev, 2), 1.0, dev)
        fig = figures(1000, 3000, 4112, True, time_steps(sets, wsp, 40, 10))
    else:
        raise ValueError(which)
    print(json.dumps({"profile_kernel": which, "figures": fig, "source_sha": source_sha(),
                      "calibration": {"kernel": "neg_kernel", "read_bytes": cal.numel() * 4, "write_bytes": cal.numel() * 4}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--preheat-ms", type=float, default=150.0,
                    help="untimed launches before the warmup steps, until the device clock has settled")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--vendor", action="store_true",
                    help="also time torch._scaled_mm (hipBLASLt, row-wise scales) on every GEMM row's operands")
    ap.add_argument("--profile-kernel", choices=["tiled", "tiled_cold", "skinny", "quantise", "fused", "grouped", "decode32", "decode128", "decode128_n10240", "decode128_n57344", "ragged"],
                    help="run only that kernel's workload a few times (for rocprofv3 counter passes) and print its figures")
    args = ap.parse_args()
    global VENDOR
    VENDOR = args.vendor
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this hot path is a single-device kernel and nothing here "
              "uses a second GPU; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU (the HIP path has no CPU fallback)", file=sys.stderr)
        sys.exit(2)
    from tritonbench_amd import _lib

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.profile_kernel:
        profile_kernel(args.profile_kernel, dev)
        return

    m = n = k = 8192
    head_sets, head_ws = make_sets(m, make_weights(n, k, 1.0, False, dev, 1), 1.0, dev)
    torch.cuda.synchronize()
    preheat(head_sets, head_ws, args.preheat_ms)
    ms, replays_ms = time_steps_graph(head_sets, head_ws, args.steps, args.warmup, args.preheat_ms)
    head = figures(m, n, k, False, ms)
    # the same steps as plain launches on a stream (what a caller without a graph sees: the gap between
    # two dependent launches is several microseconds longer than between two nodes of a graph)
    ms_stream = time_steps(head_sets, head_ws, args.steps, args.warmup)
    # one launch with clock readings, while the device is still under load: cycles belong to the kernel,
    # the clock to the box (and to each XCD: the slowest one ends the launch)
    try:
        from tritonbench_amd import ops

        clocks = ops.fp8_gemm_rowwise_clocks(*head_sets[0][:4], head_sets[0][5], workspace=head_ws)
    except Exception as e:  # noqa: BLE001 - a diagnostic: its failure must not cost the line
        clocks = {"error": f"{type(e).__name__}: {e}"}
    traffic, traffic_note = measured_traffic("tiled")

    line = {
        "metric": "fp8_gemm_rowwise TFLOP/s at M=N=K=8192 (1 GPU)",
        "value": head["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_ms": args.preheat_ms,
        "ms_per_step": ms,
        "us_min": min(replays_ms + [ms]) * 1e3,
        "us_median": statistics.median(replays_ms + [ms]) * 1e3,
        "ms_per_step_stream_launches": ms_stream,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> f32 accumulate -> bf16",
        "data": "synthetic (seeded N(0,1) fp32, row-wise e4m3fn quantised on device)",
        "config": {"workload": "c2_square M=N=K=8192, row-wise scales, no bias, bf16 out", "variant": "tiled",
                   "launch": "the timed steps are one replay of a HIP graph holding exactly `steps` calls, as the reference "
                             "operator times its backends (use_cuda_graphs); ms_per_step_stream_launches is the same "
                             "count of plain launches"},
        "roofline": {
            "bound": "mfma",
            "achieved": head["tflops"],
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": head["tflops"] / PEAK_FP8_TFLOPS,
            # HBM-side bytes per launch of the dominant kernel from two rocprofv3 counter passes
            # (FETCH_SIZE, WRITE_SIZE), each scaled by a copy kernel of known size in the same run
            "traffic": traffic,
            **traffic_note,
        },
        # What part of the fraction is the kernel's and what the box's: the MFMA instructions of one launch
        # occupy every SIMD for mfma_cycles; a workgroup takes cycles_per_workgroup_* shader cycles for
        # them; the XCDs run at clocks of their own (the peak is quoted at 2.4 GHz) and the slowest ends
        # the launch.
        "clock": {**(clocks or {}), "mfma_cycles": 2 * m * n * k // (2048 * 1024), "peak_quoted_at_ghz": 2.4},
    }

    if not args.no_extra:
        configs = {}
        cpu = not args.no_cpu_baseline

        def attempt(name, fn):
            """One side workload. A failure is recorded in its place (and on stderr) and the
            line, whose headline is already measured, is still printed."""
            try:
                configs[name] = fn()
            except Exception as e:  # noqa: BLE001 - whatever it was, the record says so
                configs[name] = {"error": f"{type(e).__name__}: {e}"}
                print(f"bench.py: {name} failed: {type(e).__name__}: {e}", file=sys.stderr, flush=True)

        def c3():
            # C3: decode-sized, HBM-bound. Cold = rotate through operand sets larger than every cache.
            cm, cn, ck = 16, 8192, 8192
            cold_sets, cws = make_sets(cm, make_weights(cn, ck, 1.0, False, dev, 10), 1.0, dev)
            cold = gemm_row(cm, cold_sets, cws, 200)
            warm = gemm_row(cm, cold_sets[:1], cws, 200)
            row = {"cold": cold, "cache_resident": warm}
            if cpu:
                row["cpu_baseline"] = cpu_baseline(cold_sets[0], "M=16, N=K=8192", budget_s=4.0)
            del cold_sets
            straffic, snote = measured_traffic("skinny")
            # What one launch costs before any byte moves: the period of back-to-back launches of a kernel
            # that touches 4 bytes, in the same kind of captured graph. It is part of every step above
            # (10 % of the decode shape's), and no kernel of ours can remove it.
            tiny = torch.zeros(1, device=dev)
            floor_ms, _ = time_graph(lambda i: tiny.add_(1.0), 400)
            line["launch_floor_us"] = floor_ms * 1e3
            line["hbm_metric"] = {
                "metric": "fp8_gemm_rowwise HBM GB/s at M=16,N=K=8192 (cold operands)",
                "value": cold["gbps"], "unit": "GB/s", "us": cold["us"], "us_median": cold["us_median"],
                "roofline": {"bound": "hbm", "achieved": cold["gbps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                             "frac": cold["gbps"] / PEAK_HBM_GBPS, "traffic": straffic, **snote},
                "frac_net_of_launch_floor": cold["gbps"] / PEAK_HBM_GBPS * cold["us"] / max(cold["us"] - floor_ms * 1e3, 1e-3),
            }
            return row

        attempt("c3_skinny_16x8192x8192", c3)

        def c5(rm, rn, rk):
            # C5: ragged shapes with fused bias
            rs, rws = make_sets(rm, make_weights(rn, rk, 1.0, True, dev, 2), 1.0, dev)
            row = gemm_row(rm, rs, rws, 50)
            if cpu:
                row["cpu_baseline"] = cpu_baseline(rs[0], f"{rm}x{rn}x{rk} + bias", budget_s=4.0, max_calls=3)
            return row

        for (rm, rn, rk) in [(1000, 3000, 4112), (4097, 7168, 2048)]:
            attempt(f"c5_ragged_bias_{rm}x{rn}x{rk}", lambda: c5(rm, rn, rk))
        attempt("c2_square_8192_graph", lambda: gemm_row(m, head_sets, head_ws, 20))

        def c2_cold():
            # five operand sets (1.9 GB: A, B and C of each are out of every cache when their turn comes again)
            cs, cws = make_sets(m, make_weights(n, k, 1.0, False, dev, 5), 1.0, dev)
            return gemm_row(m, cs, cws, 20)

        attempt("c2_square_8192_cold", c2_cold)

        def c1():
            # C1: the reference's CPU-runnable plumbing case, here on the device with the host figure beside it
            ps, pws = make_sets(128, make_weights(256, 512, 1.0, False, dev, 1), 1.0, dev)
            row = gemm_row(128, ps, pws, 200)
            if cpu:
                row["cpu_baseline"] = cpu_baseline(ps[0], "128x256x512", budget_s=1.0)
            return row

        attempt("c1_plumbing_128x256x512", c1)

        def c4(lm, ln, lk, weights, host_weight):
            ls, lws = make_sets(lm, weights, 0.02, dev)
            row = gemm_row(lm, ls, lws, 30 if lm < 1024 else 10)
            if host_weight is not None:
                row["cpu_baseline"] = cpu_baseline(ls[0], f"{lm}x{ln}x{lk}", budget_s=1.0, max_calls=3, weight=host_weight)
            return row

        # C4: Llama-3-70B projections, sigma 0.02; the weight copies of an (N, K) pair serve its whole M sweep,
        # and so does the fp32 copy of the first one on the host for the CPU figure beside every row
        for (ln, lk) in LLAMA3_70B_NK:
            try:
                weights = make_weights(ln, lk, 0.02, False, dev, copies_for(ln, lk))
                host_weight = cpu_weight((None, weights[0][0], None, weights[0][1], None, None)) if cpu else None
            except Exception as e:  # noqa: BLE001 - the weights did not fit or could not be made: every row of the pair says so
                for lm in LLAMA3_70B_M:
                    configs[f"c4_llama70b_{lm}x{ln}x{lk}"] = {"error": f"{type(e).__name__}: {e}"}
                print(f"bench.py: weights {ln}x{lk} failed: {type(e).__name__}: {e}", file=sys.stderr, flush=True)
                continue
            for lm in LLAMA3_70B_M:
                attempt(f"c4_llama70b_{lm}x{ln}x{lk}", lambda: c4(lm, ln, lk, weights, host_weight))
            del weights, host_weight
            torch.cuda.empty_cache()

        # the reference operator's own default sweep (no CPU figure: these are not configurations of the baseline)
        def builtin(bm, bn, bk):
            bs, bws = make_sets(bm, make_weights(bn, bk, 1.0, False, dev, copies_for(bn, bk)), 1.0, dev)
            return gemm_row(bm, bs, bws, 30 if bm < 1024 else 10)

        for (bm, bn, bk) in REFERENCE_BUILTIN_SHAPES:
            attempt(f"ref_builtin_{bm}x{bn}x{bk}", lambda: builtin(bm, bn, bk))
            torch.cuda.empty_cache()
        attempt("grouped_g4_8192x4096x4096", lambda: time_grouped(4, 8192, 4096, 4096, dev))
        attempt("grouped_g16_8192x8192x8192", lambda: time_grouped(16, 8192, 8192, 8192, dev, steps=20))
        attempt("blockwise_8192x8192x8192", lambda: time_blockwise(8192, 8192, 8192, dev))
        attempt("quantise_f32_8192x8192", lambda: time_quantiser(8192, 8192, torch.float32, dev))
        attempt("quantise_bf16_8192x8192", lambda: time_quantiser(8192, 8192, torch.bfloat16, dev))
        attempt("quantise_bf16_57344x8192", lambda: time_quantiser(57344, 8192, torch.bfloat16, dev, steps=20, copies=2))
        # (the activation in front of the Llama-3-70B down projection: rows of 28672)
        attempt("quantise_bf16_4096x28672", lambda: time_quantiser(4096, 28672, torch.bfloat16, dev))
        attempt("block_quantise_bf16_8192x8192", lambda: time_block_quantiser(8192, 8192, torch.bfloat16, dev))
        attempt("block_quantise_f32_8192x8192", lambda: time_block_quantiser(8192, 8192, torch.float32, dev))
        attempt("rmsnorm_quantise_bf16_8192x8192", lambda: time_fused_front_end("rmsnorm", 8192, 8192, dev))
        attempt("silu_mul_quantise_bf16_8192x8192", lambda: time_fused_front_end("silu_mul", 8192, 8192, dev))
        attempt("silu_mul_quantise_bf16_4096x28672", lambda: time_fused_front_end("silu_mul", 4096, 28672, dev))
        # (rows of 2048 elements: the forms with a wave per row; eight sources in rotation, 0.5 GB)
        attempt("quantise_bf16_16384x2048", lambda: time_quantiser(16384, 2048, torch.bfloat16, dev, copies=8))
        attempt("rmsnorm_quantise_bf16_16384x2048", lambda: time_fused_front_end("rmsnorm", 16384, 2048, dev, copies=8))
        attempt("silu_mul_quantise_bf16_16384x2048", lambda: time_fused_front_end("silu_mul", 16384, 2048, dev, copies=4))
        line["configs"] = configs

    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(head_sets[0], "M=N=K=8192")
        line["vs_cpu_baseline"] = line["value"] / line["cpu_baseline"]["value"]

    print(json.dumps(line))


if __name__ == "__main__":
    main()
