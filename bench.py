"""Benchmark of the row-wise FP8 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all-configs] [--no-cpu-baseline]

The defaults (100 warm-up, 400 timed steps, about 0.2 s of GPU time) are long enough for the
GPU's clock governor to settle: the first few milliseconds of a burst run well below the
sustained clock, so a handful of steps under-reports throughput by 20-30 %.

One step = one pass of the hot path (one mi355x_fp8_rowwise_gemm call through the C ABI)
over the headline workload M=N=K=8192 with operands resident in HBM. Prints ONE JSON line:
the headline TFLOP/s, the roofline of the dominant kernel measured with HIP events on the
launch stream, the CPU baseline (the oracle's fp32 dequantise + torch.matmul, timed on this
machine's host cores), and per-configuration figures for the skinny (HBM-bound) and the
other benchmark shapes under "configs".
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # dense FP8 MFMA, MI355X datasheet
PEAK_HBM_GBPS = 8000.0    # HBM3E, MI355X datasheet
SEED = 1337
TILED_8192_TRAFFIC_BYTES = (790326 + 131841) * 1024


def make_device_inputs(m, n, k, sigma, bias, dev, copies=1):
    """Seeded synthetic operands generated and quantised on the device (the HIP quantiser is
    bit-exact against the oracle). `copies` > 1 returns independent operand sets to rotate
    through so that no call finds its operands in L2 or the 256 MB memory-side cache."""
    from tritonbench_amd import ops

    g = torch.Generator(device=dev)
    g.manual_seed(SEED + m * 7 + n * 3 + k)
    sets = []
    for _ in range(copies):
        x = torch.randn((m, k), generator=g, device=dev, dtype=torch.float32) * sigma
        w = torch.randn((n, k), generator=g, device=dev, dtype=torch.float32) * sigma
        xq, xs = ops.fp8_row_quantize(x)
        wq, ws = ops.fp8_row_quantize(w)
        del x, w
        b = (0.1 * torch.randn((n,), generator=g, device=dev, dtype=torch.float32)).to(torch.bfloat16) if bias else None
        out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        sets.append((xq, wq, xs, ws, b, out))
    global _workspace
    _workspace = ops.gemm_workspace(m, n, k, dev)  # split-K partial sums, when the plan has them
    return sets


_workspace = None


def preheat(sets, ms):
    """Untimed launches of the workload for about `ms` milliseconds. After idling the device runs
    its first 15-20 ms of matrix work at a lower clock (8192^3: 474 us per launch against 405 us in
    the steady state on the same device); a short --warmup would leave part of that ramp inside
    the timed region."""
    import time
    from tritonbench_amd import ops

    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for i in range(10):
            xq, wq, xs, ws, b, out = sets[i % len(sets)]
            ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
        torch.cuda.synchronize()


def time_steps(sets, steps, warmup):
    """Average ms per call over exactly `steps` calls, HIP events on the launch stream."""
    from tritonbench_amd import ops

    stream = torch.cuda.current_stream()
    for i in range(warmup):
        xq, wq, xs, ws, b, out = sets[i % len(sets)]
        ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for i in range(steps):
        xq, wq, xs, ws, b, out = sets[i % len(sets)]
        ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
    end.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_steps_graph(sets, steps, warmup, min_replay_ms=6.0, preheat_ms=30.0):
    """Same, with the calls captured in one HIP graph (no per-launch host gaps); this is how the
    benchmark harness times the operator. The graph holds at least `steps` calls and enough of
    them for a replay to last `min_replay_ms`; replays run untimed for `preheat_ms` first (the
    device clock needs that after an idle spell), then the best of three timed replays counts."""
    import time
    from tritonbench_amd import ops

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(max(warmup, 1)):
            xq, wq, xs, ws, b, out = sets[i % len(sets)]
            ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(5):
            xq, wq, xs, ws, b, out = sets[i % len(sets)]
            ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
        torch.cuda.synchronize()
        est_ms = max((time.perf_counter() - t0) * 1e3 / 5, 1e-3)
        steps = int(min(max(steps, min_replay_ms / est_ms), 2000))
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for i in range(steps):
                xq, wq, xs, ws, b, out = sets[i % len(sets)]
                ops.fp8_gemm_rowwise(xq, wq, xs, ws, bias=b, out=out, workspace=_workspace)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < preheat_ms:
            g.replay()
            torch.cuda.synchronize()
        best = None
        for _ in range(3):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(side)
            g.replay()
            end.record(side)
            torch.cuda.synchronize()
            ms = start.elapsed_time(end) / steps
            best = ms if best is None else min(best, ms)
    return best


def timed_calls(call, steps, preheat_ms=30.0):
    """ms per call of call(i) over `steps` calls (HIP events on the launch stream), after untimed
    calls for `preheat_ms` so the device clock has settled."""
    import time

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

    g = torch.Generator(device=dev)
    g.manual_seed(SEED + r + k)
    xs = [torch.randn((r, k), generator=g, device=dev, dtype=torch.float32).to(dtype) for _ in range(copies)]
    ms = timed_calls(lambda i: ops.fp8_row_quantize(xs[i % copies]), steps)
    nbytes = r * k * (xs[0].element_size() + 1) + 4 * r
    return dict(us=ms * 1e3, gbps=nbytes / ms / 1e6, bound="hbm", frac=nbytes / ms / 1e6 / PEAK_HBM_GBPS)


def time_grouped(g, m, n, k, dev, steps=40, copies=2):
    """Grouped form (equal groups, as the reference's input generator makes them):
    flops = 2*M*N*K, bytes = M*K + G*N*K + 2*M*N."""
    from tritonbench_amd import ops

    gen = torch.Generator(device=dev)
    gen.manual_seed(SEED + g + m + n + k)
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

    gen = torch.Generator(device=dev)
    gen.manual_seed(SEED + 5 * m + n + k)
    xq, xs = fp8_block_quantize(torch.randn((m, k), generator=gen, device=dev, dtype=torch.float32))
    wq, ws = fp8_block_quantize(torch.randn((n, k), generator=gen, device=dev, dtype=torch.float32))
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ms = timed_calls(lambda i: ops.fp8_gemm_blockwise(xq, wq, xs, ws, out=out), steps)
    flops, nbytes = 2 * m * n * k, m * k + n * k + 2 * m * n
    return dict(us=ms * 1e3, tflops=flops / ms / 1e9, gbps=nbytes / ms / 1e6, bound="mfma",
                frac=flops / ms / 1e9 / PEAK_FP8_TFLOPS)


def figures(m, n, k, bias, ms):
    flops = 2 * m * n * k + (2 * m * n if bias else 0)
    nbytes = m * k + n * k + 2 * m * n
    tflops = flops / ms / 1e9
    gbps = nbytes / ms / 1e6
    t_mfma = flops / (PEAK_FP8_TFLOPS * 1e12)
    t_hbm = nbytes / (PEAK_HBM_GBPS * 1e9)
    bound = "mfma" if t_mfma >= t_hbm else "hbm"
    frac = tflops / PEAK_FP8_TFLOPS if bound == "mfma" else gbps / PEAK_HBM_GBPS
    return dict(us=ms * 1e3, tflops=tflops, gbps=gbps, bound=bound, frac=frac)


def cpu_baseline(xq, wq, xs, ws, budget_s=12.0):
    """The oracle (fp32 dequantise + torch.matmul) on host cores, on the same operands."""
    from oracle import fp8_rowwise as orc

    hxq, hwq, hxs, hws = xq.cpu(), wq.cpu(), xs.cpu(), ws.cpu()
    m, k = hxq.shape
    n = hwq.shape[0]
    t0 = time.perf_counter()
    orc.dequant_matmul(hxq, hwq, hxs, hws)  # warm-up (also pages in the BLAS)
    first = time.perf_counter() - t0
    times = []
    spent = 0.0
    while spent < budget_s and len(times) < 5:
        t0 = time.perf_counter()
        orc.dequant_matmul(hxq, hwq, hxs, hws)
        dt = time.perf_counter() - t0
        times.append(dt)
        spent += dt
    best = min(times) if times else first
    return {
        "value": 2 * m * n * k / best / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"full M=N=K=8192 workload, best of {len(times)} calls after 1 warm-up ({best:.3f} s/call, "
                  f"dequantise included, host cpu_count {os.cpu_count()})",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--preheat-ms", type=float, default=80.0,
                    help="untimed launches before the warmup steps, until the device clock has settled")
    ap.add_argument("--all-configs", action="store_true", help="also time every Llama-3-70B projection shape")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--profile-kernel", choices=["skinny", "quantise", "grouped"],
                    help="run only that kernel's workload a few times (for rocprofv3 counter passes) and print its figures")
    args = ap.parse_args()
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
        if args.profile_kernel == "skinny":
            ps = make_device_inputs(16, 8192, 8192, 1.0, False, dev, copies=10)
            fig = figures(16, 8192, 8192, False, time_steps(ps, 40, 10))
        elif args.profile_kernel == "quantise":
            fig = {"f32": time_quantiser(8192, 8192, torch.float32, dev, steps=20),
                   "bf16": time_quantiser(8192, 8192, torch.bfloat16, dev, steps=20)}
        else:
            fig = time_grouped(4, 8192, 4096, 4096, dev, steps=20)
        print(json.dumps({"profile_kernel": args.profile_kernel, "figures": fig}))
        return

    m = n = k = 8192
    sets = make_device_inputs(m, n, k, 1.0, False, dev, copies=1)
    torch.cuda.synchronize()
    preheat(sets, args.preheat_ms)
    ms = time_steps(sets, args.steps, args.warmup)
    head = figures(m, n, k, False, ms)

    line = {
        "metric": "fp8_gemm_rowwise TFLOP/s at M=N=K=8192 (1 GPU)",
        "value": head["tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_ms": args.preheat_ms,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn x fp8_e4m3fn -> f32 accumulate -> bf16",
        "data": "synthetic (seeded N(0,1) fp32, row-wise e4m3fn quantised on device)",
        "config": {"workload": "c2_square M=N=K=8192, row-wise scales, no bias, bf16 out", "variant": "tiled"},
        "roofline": {
            "bound": "mfma",
            "achieved": head["tflops"],
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": head["tflops"] / PEAK_FP8_TFLOPS,
            # HBM-side bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE /
            # WRITE_SIZE scaled by a copy kernel of known size (FETCH x2.0, WRITE x1.0); a property
            # of the kernel's tile walk on this workload, re-profiled whenever the kernel changes
            "traffic": TILED_8192_TRAFFIC_BYTES,
        },
    }

    if not args.no_extra:
        configs = {}
        # C3: decode-sized, HBM-bound. Cold = rotate through operand sets larger than every cache.
        cm, cn, ck = 16, 8192, 8192
        cold_sets = make_device_inputs(cm, cn, ck, 1.0, False, dev, copies=10)
        cold = figures(cm, cn, ck, False, time_steps_graph(cold_sets, 200, 5))
        warm = figures(cm, cn, ck, False, time_steps_graph(cold_sets[:1], 200, 5))
        configs["c3_skinny_16x8192x8192"] = {"cold": cold, "cache_resident": warm}
        del cold_sets
        line["hbm_metric"] = {
            "metric": "fp8_gemm_rowwise HBM GB/s at M=16,N=K=8192 (cold operands)",
            "value": cold["gbps"], "unit": "GB/s", "frac": cold["gbps"] / PEAK_HBM_GBPS,
        }
        for (rm, rn, rk) in [(1000, 3000, 4112), (4097, 7168, 2048)]:
            rs = make_device_inputs(rm, rn, rk, 1.0, True, dev, copies=2)
            configs[f"c5_ragged_bias_{rm}x{rn}x{rk}"] = figures(rm, rn, rk, True, time_steps_graph(rs, 50, 3))
            del rs
        make_device_inputs(m, n, k, 1.0, False, dev, copies=0)  # workspace of the headline plan again
        configs["c2_square_8192_graph"] = figures(m, n, k, False, time_steps_graph(sets, 20, 2))
        configs["grouped_g4_8192x4096x4096"] = time_grouped(4, 8192, 4096, 4096, dev)
        configs["grouped_g16_8192x8192x8192"] = time_grouped(16, 8192, 8192, 8192, dev, steps=20)
        configs["blockwise_8192x8192x8192"] = time_blockwise(8192, 8192, 8192, dev)
        configs["quantise_f32_8192x8192"] = time_quantiser(8192, 8192, torch.float32, dev)
        configs["quantise_bf16_8192x8192"] = time_quantiser(8192, 8192, torch.bfloat16, dev)
        configs["quantise_bf16_57344x8192"] = time_quantiser(57344, 8192, torch.bfloat16, dev, steps=20, copies=2)
        if args.all_configs:
            for (ln, lk) in [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]:
                for lm in (1, 32, 128, 1024, 4096):
                    copies = max(2, min(8, int(600e6 // (ln * lk)) + 1))
                    ls = make_device_inputs(lm, ln, lk, 0.02, False, dev, copies=copies)
                    configs[f"c4_llama70b_{lm}x{ln}x{lk}"] = figures(lm, ln, lk, False, time_steps_graph(ls, 30, 3))
                    del ls
                    torch.cuda.empty_cache()
        line["configs"] = configs

    if not args.no_cpu_baseline:
        xq, wq, xs, ws, _, _ = sets[0]
        line["cpu_baseline"] = cpu_baseline(xq, wq, xs, ws)

    print(json.dumps(line))


if __name__ == "__main__":
    main()
