"""Host-side harness behaviour, on CPU. The table-shape cases restate what tritonbench's own
CPU tests check (test/test_cpu/main.py:20-65: "<label>-<metric>" headers, accuracy cell,
x-only metric header, label override); the rest pins Latency, the error mapping and the
registration surface."""
import argparse
import io
import json
import statistics
import sys
import types

import pytest
import torch

from tritonbench_amd.harness import (
    BASELINE_BENCHMARKS,
    REGISTERED_BENCHMARKS,
    BenchmarkOperator,
    BenchmarkOperatorMetrics,
    Latency,
    register_benchmark,
    register_metric,
    register_x_val,
)
from tritonbench_amd.harness import registry as R
from tritonbench_amd.harness.latency import do_bench_cpu, do_bench_wrapper
from tritonbench_amd.harness.parser import get_parser


def _make_fake_operator(op_name="test_op"):
    """An operator defined in a synthetic module so name-from-module-path works."""
    mod_name = f"fakepkg.operators.{op_name}.operator"
    for k in (R.REGISTERED_BENCHMARKS, R.REGISTERED_METRICS, R.REGISTERED_X_VALS, R.BASELINE_BENCHMARKS, R.OVERRIDDEN_METRICS):
        k.pop(op_name, None)
    src = '''
import torch
from tritonbench_amd.harness import BenchmarkOperator, register_benchmark, register_metric, register_x_val

class Operator(BenchmarkOperator):
    DEFAULT_METRICS = ["latency"]

    @register_benchmark(baseline=True)
    def ref(self, x):
        return lambda: x * 2

    @register_benchmark(label="new-label")
    def cand(self, x):
        return lambda: x + x

    @register_benchmark()
    def wrong(self, x):
        return lambda: x * 3

    @register_benchmark()
    def unsupported(self, x):
        raise NotImplementedError("nope")

    @register_benchmark(enabled=False)
    def hidden(self, x):
        return lambda: x

    @register_benchmark()
    def boom(self, x):
        raise RuntimeError("kaboom")

    @register_metric(x_only=True)
    def test_metric(self, fn, example_inputs, metrics):
        return [0, 1, 2]

    @register_metric()
    def numel(self, fn, example_inputs, metrics):
        return example_inputs[0].numel()

    @register_x_val(label="size")
    def get_x_val(self, example_inputs):
        return example_inputs[0].numel()

    def get_input_iter(self):
        for n in (8, 16, 32):
            yield (torch.ones(n),)
'''
    mod = types.ModuleType(mod_name)
    mod.__dict__["__name__"] = mod_name
    sys.modules[mod_name] = mod
    exec(compile(src, mod_name, "exec"), mod.__dict__)
    return mod.Operator


def _args(*argv):
    return get_parser().parse_known_args(["--op", "test_op", "--device", "cpu", *argv])


def _run(*argv):
    Op = _make_fake_operator()
    args, extra = _args(*argv)
    op = Op(tb_args=args, extra_args=extra)
    op.run(1, 2)
    return op.output


def test_headers_are_label_dash_metric_and_baseline_first_without_accuracy():
    out = _run("--only", "cand,ref", "--metrics", "latency,accuracy,speedup")
    headers, table = out._table()
    assert headers == ["size", "ref-latency", "new-label-latency", "new-label-accuracy", "new-label-speedup"]
    assert [r[0] for r in table] == [8, 16, 32, "average"]
    acc_col = headers.index("new-label-accuracy")
    assert all(table[i][acc_col] is True for i in range(3))


def test_wrong_backend_fails_accuracy():
    out = _run("--only", "ref,wrong", "--metrics", "accuracy")
    headers, table = out._table()
    assert headers == ["size", "wrong-accuracy"]
    assert all(table[i][1] is False for i in range(3))
    assert table[-1] == ["average", 0.0]


def test_x_only_metric_has_bare_header():
    out = _run("--only", "ref", "--metrics", "test_metric")
    headers, table = out._table()
    assert "test_metric" in headers and "ref-test_metric" not in headers
    assert table[0][headers.index("test_metric")] == [0, 1, 2]
    assert "1" in str(out)  # rendered as the median of the list


def test_custom_metric_and_num_inputs_and_input_id():
    out = _run("--only", "ref", "--metrics", "numel", "--input-id", "1", "--num-inputs", "1")
    headers, table = out._table()
    assert headers == ["size", "ref-numel"]
    assert table[0] == [16, 16] and table[1] == ["average", 16.0]


def test_disabled_backend_is_hidden_and_unsupported_reports_cell():
    Op = _make_fake_operator()
    args, extra = _args("--skip", "boom", "--metrics", "latency")
    op = Op(tb_args=args, extra_args=extra)
    op.run(1, 2)
    headers, table = op.output._table()
    assert "hidden-latency" not in headers
    assert table[0][headers.index("unsupported-latency")] == "not supported"


def test_exception_propagates_unless_keep_going():
    Op = _make_fake_operator()
    args, extra = _args("--only", "ref,boom", "--metrics", "latency")
    op = Op(tb_args=args, extra_args=extra)
    with pytest.raises(RuntimeError, match="kaboom"):
        op.run(1, 2)
    assert op.output is not None  # partial result object is still attached
    Op = _make_fake_operator()
    args, extra = _args("--only", "ref,boom", "--metrics", "latency", "--keep-going")
    op = Op(tb_args=args, extra_args=extra)
    op.run(1, 2)
    headers, table = op.output._table()
    assert table[0][headers.index("boom-latency")] == "kaboom"


def test_baseline_flag_overrides_registered_baseline():
    out = _run("--only", "ref,cand", "--baseline", "cand", "--metrics", "latency,speedup")
    headers, _ = out._table()
    assert headers[1] == "new-label-latency" and "ref-speedup" in headers and "new-label-speedup" not in headers


def test_csv_and_json_exports():
    out = _run("--only", "ref,cand", "--metrics", "latency,accuracy")
    buf = io.StringIO()
    out.write_csv_to_file(buf)
    lines = buf.getvalue().strip().splitlines()
    assert lines[0] == "size;ref-latency;new-label-latency;new-label-accuracy"
    assert lines[1].split(";")[0] == "8" and lines[1].split(";")[-1] == "1.0"
    d = out.userbenchmark_dict
    assert "tritonbench_test_op_fwd[x_8-ref]_latency" in d
    assert d["tritonbench_test_op_fwd[x_16-new-label]_accuracy"] == 1.0
    assert "tritonbench_test_op_fwd[new-label]-accuracy-avg" in d
    json.dumps(d)


def test_register_from_outside_the_module_with_explicit_names():
    Op = _make_fake_operator()

    def extra(self, x):
        return lambda: x * 2

    register_benchmark(operator_name="test_op", func_name="extra_backend", label="extra")(extra)
    setattr(Op, "extra_backend", extra)
    args, rest = _args("--only", "ref,extra_backend", "--metrics", "accuracy")
    op = Op(tb_args=args, extra_args=rest)
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["size", "extra-accuracy"] and table[0][1] is True


def test_operator_name_needs_operators_in_module_path():
    def f(self):
        pass

    f.__module__ = "somewhere.else"
    with pytest.raises(AssertionError):
        register_benchmark()(f)


def test_backend_must_return_callable():
    Op = _make_fake_operator()
    Op.bad = lambda self, x: 42
    register_benchmark(operator_name="test_op", func_name="bad")(Op.bad)
    args, rest = _args("--only", "bad", "--metrics", "latency")
    op = Op(tb_args=args, extra_args=rest)
    with pytest.raises(TypeError):
        op.run(1, 2)


# ---- Latency -----------------------------------------------------------------------------
def test_latency_p50_is_median_low_and_small_samples_untouched():
    assert Latency([3.0, 1.0, 2.0, 4.0]).p50 == 2.0
    assert Latency([5.0, 1.0]).times == [5.0, 1.0]


def test_latency_drops_iqr_outliers(capsys):
    data = [1.0 + 0.001 * i for i in range(40)] + [100.0]
    lat = Latency(data)
    assert 100.0 not in lat.times and len(lat.times) == 40
    assert "Removed 1 outliers from 41 samples" in capsys.readouterr().out


def test_latency_arithmetic_uses_p50():
    a, b = Latency([2.0, 2.0, 2.0]), Latency([4.0, 4.0, 4.0])
    assert a + b == 6.0 and b - a == 2.0 and a * b == 8.0 and b / a == 2.0 and 8.0 / a == 4.0
    assert 1.0 + a == 3.0 and b // a == 2.0
    assert str(a) == "2.0"
    assert a.to_str("with_variance").startswith("2.000000 (±0.00%)")
    assert Latency([1.0, 2.0, 3.0]).to_str("mean") == str(statistics.mean([1.0, 2.0, 3.0]))
    with pytest.raises(ValueError):
        a.to_str("bogus")


def test_cpu_timing_loop_and_wrapper():
    calls = []
    times = do_bench_cpu(lambda: calls.append(1), warmup=1, rep=2)
    assert len(times) >= 1 and len(calls) >= 1 + 5 + 1 + len(times)
    lat = do_bench_wrapper(lambda: None, 1, 2, None, device="cpu")
    assert isinstance(lat, Latency)

    def bad():
        raise RuntimeError("x")

    with pytest.raises(RuntimeError):
        do_bench_wrapper(bad, 1, 2, None, device="cpu")
    assert do_bench_wrapper(bad, 1, 2, None, device="cpu", bypass_fail=True) is None


# ---- the real operator on CPU (config 1: plumbing) ---------------------------------------
def test_fp8_gemm_rowwise_operator_cpu_plumbing():
    from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name

    assert "fp8_gemm_rowwise" in list_operators()
    Op = load_opbench_by_name("FP8_gemm_rowwise")  # case-insensitive
    assert Op.name == "fp8_gemm_rowwise"
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_rowwise", "--device", "cpu", "--m", "128", "--n", "256", "--k", "512",
         "--metrics", "latency,tflops,gbps", "--only", "_torch_dequant_cpu"])
    op = Op(tb_args=args, extra_args=extra)
    assert op.use_cuda_graphs is True and op.shapes == [(128, 256, 512)]
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["(M, N, K)", "torch_cpu_ref-latency", "torch_cpu_ref-tflops", "torch_cpu_ref-gbps"]
    assert table[0][0] == (128, 256, 512)
    lat = table[0][1].p50
    assert table[0][2] == pytest.approx(2 * 128 * 256 * 512 / lat / 1e12 * 1e3)
    assert table[0][3] == pytest.approx((128 * 512 + 256 * 512 + 2 * 128 * 256) / 1e9 / lat * 1e3)
    assert BASELINE_BENCHMARKS["fp8_gemm_rowwise"] == "_torch_dequant_cpu"
    assert REGISTERED_BENCHMARKS["fp8_gemm_rowwise"]["_hip_mi355x"].label == "hip_mi355x"


def test_operator_flags_and_shape_lists():
    from tritonbench_amd.operators.fp8_gemm_rowwise import operator as opmod

    a = opmod.parse_args([])
    assert a.use_tma is False and a.no_use_persistent is True and a.bias is False
    with pytest.raises(RuntimeError, match="TMA"):
        opmod.parse_args(["--use_tma"])
    assert len(opmod.BUILDIN_SHAPES) == 20 and (16, 13312, 13312) in opmod.BUILDIN_SHAPES
    args, extra = get_parser().parse_known_args(["--op", "fp8_gemm_rowwise", "--device", "cpu", "--llama", "--bias"])
    op = opmod.Operator(tb_args=args, extra_args=extra)
    assert len(op.shapes) == 12 and op.bias and (1, 57344, 8192) in op.shapes
    args, extra = get_parser().parse_known_args(["--op", "fp8_gemm_rowwise", "--device", "cpu", "--llama", "--prefill"])
    assert (4096, 8192, 28672) in opmod.Operator(tb_args=args, extra_args=extra).shapes


def test_operator_host_quantiser_matches_oracle_bitwise():
    from oracle import fp8_rowwise as orc
    from tritonbench_amd.operators.fp8_gemm_rowwise.operator import fp8_row_quantize

    x = orc.randn_f32(64, 272, 1.0, seed=5)
    xq, inv = fp8_row_quantize(x)
    oq, oinv = orc.fp8_row_quantize(x)
    assert torch.equal(xq.view(torch.uint8), oq.view(torch.uint8)) and torch.equal(inv, oinv)


def test_hip_backend_refuses_host_tensors():
    from tritonbench_amd import ops

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fp8_gemm_rowwise(
            torch.zeros(16, 16).to(torch.float8_e4m3fn), torch.zeros(16, 16).to(torch.float8_e4m3fn),
            torch.ones(16), torch.ones(16))


def test_grouped_operator_cpu_plumbing():
    from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name

    assert "fp8_gemm_rowwise_grouped" in list_operators()
    Op = load_opbench_by_name("fp8_gemm_rowwise_grouped")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_rowwise_grouped", "--device", "cpu", "--m", "96", "--n", "64", "--k", "128",
         "--group_size", "3", "--metrics", "latency,tflops,gbps", "--only", "_torch_dequant_cpu"])
    op = Op(tb_args=args, extra_args=extra)
    assert op.shapes == [(96, 64, 128)] and op.group_sizes == [3]
    group_A, group_B, m_sizes, a_scale, b_scale = next(op.get_input_iter())
    assert group_A.shape == (96, 128) and group_B.shape == (3 * 64, 128)
    assert m_sizes.dtype == torch.int32 and m_sizes.tolist() == [32, 32, 32]
    assert a_scale.shape == (96,) and b_scale.shape == (192,)
    # the host baseline is the oracle's grouped product
    from oracle import fp8_rowwise as orc
    want = orc.grouped_dequant_matmul(group_A, group_B, m_sizes, a_scale, b_scale)
    assert torch.equal(op._torch_dequant_cpu(group_A, group_B, m_sizes, a_scale, b_scale)(), want)
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["(group_size, M, N, K)", "torch_cpu_ref-latency", "torch_cpu_ref-tflops", "torch_cpu_ref-gbps"]
    assert table[0][0] == (3, 96, 64, 128)
    lat = table[0][1].p50
    assert table[0][2] == pytest.approx(2 * 96 * 64 * 128 / lat / 1e12 * 1e3)
    assert table[0][3] == pytest.approx((96 * 128 + 3 * 64 * 128 + 2 * 96 * 64) / 1e9 / lat * 1e3)
    assert REGISTERED_BENCHMARKS["fp8_gemm_rowwise_grouped"]["_hip_mi355x"].label == "hip_mi355x"
    with pytest.raises((RuntimeError, NotImplementedError)):
        op._hip_mi355x(group_A, group_B, m_sizes, a_scale, b_scale)()


def test_blockwise_operator_cpu_plumbing():
    from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name
    from tritonbench_amd.operators.fp8_gemm_blockwise import operator as bw

    assert "fp8_gemm_blockwise" in list_operators()
    Op = load_opbench_by_name("fp8_gemm_blockwise")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_blockwise", "--device", "cpu", "--m", "130", "--n", "64", "--k", "272",
         "--metrics", "latency,tflops", "--only", "_torch_dequant_cpu"])
    op = Op(tb_args=args, extra_args=extra)
    xq, wq, x_scale, w_scale = next(op.get_input_iter())
    assert xq.shape == (130, 272) and x_scale.shape == (2, 3) and w_scale.shape == (1, 3)
    # the operator's quantiser (bf16 source, any device) is the oracle's, bit for bit
    from oracle import fp8_rowwise as orc
    x = orc.randn_f32(130, 272, 1.0, seed=5).to(torch.bfloat16)
    q1, s1 = bw.fp8_block_quantize(x)
    q2, s2 = orc.fp8_block_quantize(x)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1, s2)
    want = orc.blockwise_dequant_matmul(xq, wq, x_scale, w_scale)
    assert torch.equal(op._torch_dequant_cpu(xq, wq, x_scale, w_scale)(), want)
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["(M, N, K)", "torch_cpu_ref-latency", "torch_cpu_ref-tflops"]
    assert table[0][0] == (130, 64, 272)
    assert REGISTERED_BENCHMARKS["fp8_gemm_blockwise"]["_hip_mi355x"].label == "hip_mi355x"


def test_tensorwise_operator_cpu_plumbing():
    from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name

    assert "fp8_gemm" in list_operators()
    Op = load_opbench_by_name("fp8_gemm")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm", "--device", "cpu", "--m", "64", "--n", "48", "--k", "32",
         "--metrics", "latency,tflops,gbps", "--only", "_torch_dequant_cpu"])
    op = Op(tb_args=args, extra_args=extra)
    a, b = next(op.get_input_iter())
    assert a.shape == (64, 32) and b.shape == (32, 48) and b.stride(0) == 1  # b column-major as _scaled_mm wants it
    out = op._torch_dequant_cpu(a, b)()
    assert out.dtype == torch.float16
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["(M, N, K)", "torch_cpu_ref-tflops", "torch_cpu_ref-gbps", "torch_cpu_ref-latency"] or \
        headers == ["(M, N, K)", "torch_cpu_ref-latency", "torch_cpu_ref-tflops", "torch_cpu_ref-gbps"]
    assert table[0][0] == (64, 48, 32)
    # default sweep: 2^10 .. 2^14 in quarter steps, square
    args, extra = get_parser().parse_known_args(["--op", "fp8_gemm", "--device", "cpu"])
    shapes = Op(tb_args=args, extra_args=extra)._shapes()
    assert len(shapes) == 20 and shapes[0] == (1024, 1024, 1024) and shapes[1] == (1280, 1280, 1280) and shapes[-1] == (28672, 28672, 28672)
    args, extra = get_parser().parse_known_args(["--op", "fp8_gemm", "--device", "cpu", "--m", "8", "--n", "8", "--k", "16", "--scaling_rowwise"])
    assert Op(tb_args=args, extra_args=extra)._torch_dequant_cpu(*next(Op(tb_args=args, extra_args=extra).get_input_iter()))().dtype == torch.bfloat16


def test_export_dumps_inputs_and_outputs(tmp_path):
    from tritonbench_amd.harness.loader import load_opbench_by_name

    Op = load_opbench_by_name("fp8_gemm_rowwise")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_rowwise", "--device", "cpu", "--m", "32", "--n", "48", "--k", "64", "--metrics", "latency",
         "--only", "_torch_dequant_cpu", "--export", "both", "--export-dir", str(tmp_path)])
    op = Op(tb_args=args, extra_args=extra)
    op.run(1, 1)
    files = sorted(f.name for f in tmp_path.iterdir())
    assert files == ["x_(32,48,64)-_torch_dequant_cpu-fwd-output.pt", "x_(32,48,64)-input.pt"]
    xq, wq, xs, ws, bias = torch.load(tmp_path / "x_(32,48,64)-input.pt", weights_only=True)
    out = torch.load(tmp_path / "x_(32,48,64)-_torch_dequant_cpu-fwd-output.pt", weights_only=True)
    assert xq.dtype == torch.float8_e4m3fn and xq.shape == (32, 64) and bias is None and out.shape == (32, 48)
    from oracle import fp8_rowwise as orc
    assert torch.equal(out, orc.dequant_matmul(xq, wq, xs, ws))
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_rowwise", "--device", "cpu", "--m", "32", "--n", "48", "--k", "64", "--only", "_torch_dequant_cpu",
         "--export", "input", "--export-dir", str(tmp_path / "missing")])
    with pytest.raises(RuntimeError, match="must exist"):
        Op(tb_args=args, extra_args=extra).run(1, 1)


def test_cuda_time_groups_kernels_between_flush_fills():
    # per call: everything between two cache-clearing fills, whatever the number of kernels
    # (upstream cuda_time.py:15-49 requires every kernel name to occur equally often instead)
    from tritonbench_amd.harness.cuda_time import split_calls

    fill = "void at::native::vectorized_elementwise_kernel<4, at::native::FillFunctor<int>, std::array<char*, 1ul> >(int)"
    events = [
        (5.0, 99.0, "stray kernel before the first fill"),
        (10.0, 70.0, fill), (90.0, 20.0, "gemm"), (111.0, 6.0, "finalize"),
        (120.0, 70.0, fill), (200.0, 22.0, "gemm"), (223.0, 5.0, "finalize"),
        (230.0, 70.0, fill), (310.0, 14.0, "skinny"),
    ]
    assert split_calls(reversed(events)) == pytest.approx([0.026, 0.027, 0.014])
    assert split_calls([]) == []
    # a backend that zero-fills its own bf16 output inside the call is not taken for the flush
    own_fill = fill.replace("FillFunctor<int>", "FillFunctor<c10::BFloat16>")
    events = [(10.0, 70.0, fill), (90.0, 3.0, own_fill), (95.0, 20.0, "grouped gemm"),
              (120.0, 70.0, fill), (200.0, 3.0, own_fill), (205.0, 21.0, "grouped gemm")]
    assert split_calls(events) == pytest.approx([0.023, 0.024])


def test_cuda_time_metric_needs_a_gpu_backend():
    out = _run("--only", "ref", "--metrics", "cuda_time")
    headers, table = out._table()
    assert table[0][headers.index("ref-cuda_time")] == "not supported"


@pytest.mark.gpu
def test_cuda_time_metric_on_the_gpu(gpu_device):
    from tritonbench_amd.harness.loader import load_opbench_by_name

    Op = load_opbench_by_name("fp8_gemm_rowwise")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_gemm_rowwise", "--m", "128", "--n", "8192", "--k", "8192", "--only", "_hip_mi355x",
         "--metrics", "latency,cuda_time"])
    op = Op(tb_args=args, extra_args=extra)
    op.run(5, 20)
    headers, table = op.output._table()
    lat = table[0][headers.index("hip_mi355x-latency")]
    dev = table[0][headers.index("hip_mi355x-cuda_time")]
    # kernel time only (one kernel per call for this shape), operands evicted before each call, no launch gaps counted
    assert 0.010 < dev.p50 < 0.100 and 0.010 < lat.p50 < 0.100


def test_fused_quant_operator_cpu_plumbing():
    from oracle import fp8_rowwise as orc
    from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name
    from tritonbench_amd.operators.fp8_fused_quant_gemm_rowwise import operator as fq

    assert "fp8_fused_quant_gemm_rowwise" in list_operators()
    assert len(fq.BUILDIN_SHAPES) == 20 and fq.BUILDIN_SHAPES[0] == (1, 2304, 2048) and fq.BUILDIN_SHAPES[-1] == (16384, 8192, 13312)
    Op = load_opbench_by_name("fp8_fused_quant_gemm_rowwise")
    args, extra = get_parser().parse_known_args(
        ["--op", "fp8_fused_quant_gemm_rowwise", "--device", "cpu", "--m", "5", "--n", "48", "--k", "272",
         "--metrics", "latency,tflops", "--only", "_rms_norm_dequant_cpu"])
    op = Op(tb_args=args, extra_args=extra)
    x1, x2, wq, w_scale, wd = next(op.get_input_iter())
    assert x1.dtype == torch.bfloat16 and x1.shape == (5, 272) and x2.shape == (5, 272)
    assert wq.shape == (48, 272) and w_scale.shape == (48,) and wd.shape == (272,)
    # the operator's CPU chain is the oracle's: front end, row quantiser, dequantised product
    xq, xs = orc.rms_norm_fp8_rowwise_quant(x1, wd, fq.RMS_NORM_EPS)
    want = orc.dequant_matmul(xq, wq, xs, w_scale, None)
    # (a code that falls the other way on a rounding tie moves single terms of the sums by one e4m3 step)
    got = op._rms_norm_dequant_cpu(x1, x2, wq, w_scale, wd)().double()
    assert (got - want.double()).norm() / want.double().norm() <= 1e-2
    op.run(1, 2)
    headers, table = op.output._table()
    assert headers == ["(M, N, K)", "rms_norm_cpu_ref-latency", "rms_norm_cpu_ref-tflops"]
    assert table[0][0] == (5, 48, 272)
    assert table[0][2] == pytest.approx(2 * 5 * 48 * 272 / table[0][1].p50 / 1e12 * 1e3)
    for name in ("rms_norm_fused", "rms_norm_quant", "silu_mul_fused", "silu_mul_quant"):
        assert name in REGISTERED_BENCHMARKS["fp8_fused_quant_gemm_rowwise"]
    with pytest.raises((RuntimeError, NotImplementedError)):
        op.rms_norm_fused(x1, x2, wq, w_scale, wd)()
