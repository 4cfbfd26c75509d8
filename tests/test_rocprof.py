"""The `rocprof` metric: command lines, counter-pass limits and CSV parsing on the CPU; one
real profiled child process on the GPU."""
import os
import sys
import types

import pytest

from tritonbench_amd.harness import rocprof

KERNEL_STATS = '''"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"
"void (anonymous namespace)::gemm_tiled_kernel<256, 256, 2, 2, false, 0, false, false, 2, false>((anonymous namespace)::GemmParams)",887,323890240,365152.468997,44.66,351435,508375,15510.049166
"void (anonymous namespace)::splitk_finalize_kernel((anonymous namespace)::GemmParams)",10,30000,3000.0,0.01,2900,3100,50.0
'''

TRACE_HEAD = ('"Kind","Agent_Id","Queue_Id","Stream_Id","Thread_Id","Dispatch_Id","Kernel_Id","Kernel_Name",'
              '"Correlation_Id","Start_Timestamp","End_Timestamp","LDS_Block_Size","Scratch_Size","VGPR_Count",'
              '"Accum_VGPR_Count","SGPR_Count","Workgroup_Size_X","Workgroup_Size_Y","Workgroup_Size_Z",'
              '"Grid_Size_X","Grid_Size_Y","Grid_Size_Z"\n')


def _trace_row(i, name, start, end):
    return f'"KERNEL_DISPATCH","Agent 1",1,0,9,{i},7,"{name}",{i},{start},{end},0,0,8,0,16,256,1,1,256,1,1\n'


def test_child_and_profiler_command_lines(tmp_path):
    tb = types.SimpleNamespace(device="cuda", precision="fp8")
    child = rocprof.child_argv("fp8_gemm_rowwise", "_hip_mi355x", 3, tb, ["--m", "16", "--n", "32", "--k", "64"], python="/usr/bin/python3")
    assert child[:2] == ["/usr/bin/python3", rocprof.RUN_PY] and os.path.basename(rocprof.RUN_PY) == "run.py"
    for flag, value in (("--op", "fp8_gemm_rowwise"), ("--only", "_hip_mi355x"), ("--input-id", "3"), ("--num-inputs", "1"),
                        ("--metrics", rocprof.IN_TASK_METRIC), ("--device", "cuda"), ("--precision", "fp8"), ("--k", "64")):
        assert child[child.index(flag) + 1] == value
    cmd = rocprof.profiler_argv(child, str(tmp_path))
    sep = cmd.index("--")
    assert os.path.basename(cmd[0]) == "rocprofv3"
    assert "--kernel-trace" in cmd[:sep] and "--stats" in cmd[:sep] and "--pmc" not in cmd
    # the interpreter itself follows the separator: nothing that would exec again in between
    assert cmd[sep + 1] == "/usr/bin/python3" and cmd[sep + 2] == rocprof.RUN_PY
    pmc = rocprof.profiler_argv(child, str(tmp_path), pmc=["FETCH_SIZE"])
    sep = pmc.index("--")
    assert pmc[pmc.index("--pmc") + 1] == "FETCH_SIZE"
    assert not {"--kernel-trace", "--stats", "--sys-trace", "-s", "-r"} & set(pmc[:sep])  # a counter pass is its own run
    with pytest.raises(ValueError, match="interpreter"):
        rocprof.profiler_argv(["env", "python3", "run.py"], str(tmp_path))
    with pytest.raises(ValueError, match="interpreter"):
        rocprof.profiler_argv(["bash", "-c", "python3 run.py"], str(tmp_path))


def test_counter_pass_limits():
    rocprof.check_pmc_fits(["FETCH_SIZE"])
    rocprof.check_pmc_fits(["WRITE_SIZE", "TCC_HIT_sum", "TCC_MISS_sum"])
    rocprof.check_pmc_fits([f"SQ_COUNTER_{i}" for i in range(8)])
    rocprof.check_pmc_fits(["SQ_WAVES", "SQ_WAVES_sum"])  # reductions of one counter count once
    with pytest.raises(ValueError, match="TCC_"):
        rocprof.check_pmc_fits(["FETCH_SIZE", "WRITE_SIZE"])  # 3 + 2 TCC counters
    with pytest.raises(ValueError, match="SQ_"):
        rocprof.check_pmc_fits([f"SQ_COUNTER_{i}" for i in range(9)])
    with pytest.raises(ValueError, match="TA_"):
        rocprof.check_pmc_fits(["TA_A", "TA_B", "TA_C"])


def test_kernel_stats_and_names(tmp_path):
    path = tmp_path / "run_kernel_stats.csv"
    path.write_text(KERNEL_STATS)
    rows = rocprof.parse_kernel_stats(str(path))
    assert [r["calls"] for r in rows] == [887, 10]
    assert rows[0]["avg_us"] == pytest.approx(365.152468997)
    assert rows[1]["min_us"] == pytest.approx(2.9) and rows[1]["percent"] == pytest.approx(0.01)
    assert rocprof.short_kernel_name(rows[0]["name"]) == "gemm_tiled_kernel<256, 256, 2, 2, false, 0, false, false, 2, false>"
    assert rocprof.short_kernel_name(rows[1]["name"]) == "splitk_finalize_kernel"
    assert rocprof.matching(rows, ["splitk"]) == [rows[1]]
    assert rocprof._find(str(tmp_path), "_kernel_stats.csv") == str(path)


def test_window_between_markers(tmp_path):
    fill = "void at::native::vectorized_elementwise_kernel<8, at::native::FillFunctor<short>, std::array<char*, 1ul> >(int)"
    gemm = "void (anonymous namespace)::gemm_tiled_kernel<128, 128, 2, 2, false, 2, false, false, 2, true>((anonymous namespace)::GemmParams)"
    fin = "void (anonymous namespace)::splitk_finalize_kernel((anonymous namespace)::GemmParams)"
    rows = [_trace_row(1, "randn", 100, 900), _trace_row(2, gemm, 1000, 21000), _trace_row(3, fin, 21500, 24500)]  # warm-up
    t = 30000
    rows.append(_trace_row(4, fill, t, t + 500))
    i = 5
    for c in range(rocprof.IN_TASK_CALLS):
        rows.append(_trace_row(i, gemm, t + 1000, t + 1000 + 20000 + 1000 * c)); i += 1
        rows.append(_trace_row(i, fin, t + 30000, t + 33000)); i += 1
        t += 40000
    rows.append(_trace_row(i, fill, t, t + 500))
    rows.append(_trace_row(i + 1, "later", t + 1000, t + 2000))
    path = tmp_path / "run_kernel_trace.csv"
    path.write_text(TRACE_HEAD + "".join(reversed(rows)))  # order in the file does not matter
    stats = rocprof.window_stats(rocprof.parse_kernel_trace(str(path)))
    assert [s["kernel"] for s in stats] == ["gemm_tiled_kernel<128, 128, 2, 2, false, 2, false, false, 2, true>", "splitk_finalize_kernel"]
    assert stats[0]["launches_per_call"] == 1 and stats[0]["avg_us"] == pytest.approx(22.0) and stats[0]["min_us"] == pytest.approx(20.0)
    assert stats[1]["us_per_call"] == pytest.approx(3.0)
    cell = rocprof.format_rows(stats)
    assert cell.startswith("gemm_tiled_kernel<128") and "22.0 us x1" in cell and "splitk_finalize_kernel: 3.0 us x1" in cell
    with pytest.raises(RuntimeError, match="marker"):
        rocprof.window_stats(rocprof.parse_kernel_trace(str(path)), marker="NoSuchKernel")


def test_traffic_summary_scales_by_the_copy_kernel(tmp_path):
    head = ('"Correlation_Id","Dispatch_Id","Agent_Id","Queue_Id","Process_Id","Thread_Id","Grid_Size","Kernel_Id","Kernel_Name",'
            '"Workgroup_Size","LDS_Block_Size","Scratch_Size","VGPR_Count","Accum_VGPR_Count","SGPR_Count","Counter_Name",'
            '"Counter_Value","Start_Timestamp","End_Timestamp"\n')

    def row(i, name, counter, value):
        return f'{i},{i},"Agent 1",1,9,9,1024,5,"{name}",256,0,0,8,0,16,"{counter}",{value},1,2\n'

    copy = "void at::native::vectorized_elementwise_kernel<4, at::native::AUnaryFunctor<float, float, float, at::native::binary_internal::MulFunctor<float> >, x>(int)"
    gemm = "void (anonymous namespace)::gemm_tiled_kernel<256, 256, 2, 2, false, 0, false, false, 2, false>((anonymous namespace)::GemmParams)"
    f = tmp_path / "f.csv"
    w = tmp_path / "w.csv"
    f.write_text(head + row(1, copy, "FETCH_SIZE", 131072.0) + row(2, gemm, "FETCH_SIZE", 400000.0) + row(3, gemm, "FETCH_SIZE", 390000.0))
    w.write_text(head + row(1, copy, "WRITE_SIZE", 262144.0) + row(2, gemm, "WRITE_SIZE", 131072.0) + row(3, gemm, "WRITE_SIZE", 131072.0))
    out = rocprof.traffic_summary(str(f), str(w), "gemm_tiled_kernel<256, 256", "MulFunctor", 256 << 20, 256 << 20)
    assert out["fetch_factor"] == pytest.approx(2.0) and out["write_factor"] == pytest.approx(1.0)
    assert out["dispatches"] == 2
    assert out["fetch_bytes"] == 395000 * 1024 * 2 and out["write_bytes"] == 131072 * 1024
    assert out["traffic_bytes"] == out["fetch_bytes"] + out["write_bytes"]
    assert out["kernel"].startswith("gemm_tiled_kernel<256, 256")


@pytest.mark.gpu
def test_rocprof_metric_profiles_a_child_process(gpu_device):
    import run as run_py

    out = run_py.run(["--op", "fp8_gemm_rowwise", "--m", "320", "--n", "1024", "--k", "8192", "--only", "_hip_mi355x",
                      "--metrics", "rocprof,rocprof_us"])
    (x_val, per_backend), = out.result
    rec = per_backend["_hip_mi355x"]
    assert rec.error_msg is None
    cell = rec.extra_metrics["rocprof"]
    print(cell, flush=True)
    # this shape runs a split-K plan: two kernels per call, the tiled one first
    assert cell.startswith("gemm_tiled_kernel<") and "splitk_finalize_kernel" in cell and " us x1" in cell
    assert 1.0 < rec.extra_metrics["rocprof_us"] < 500.0
    assert "hip_mi355x-rocprof" in str(out)


def test_counter_cell_format():
    cell = rocprof.format_counters({"gemm_tiled_kernel<128, 128>": {"WRITE_SIZE": 2048.0, "FETCH_SIZE": 35628.66},
                                    "splitk_finalize_kernel": {"FETCH_SIZE": 8240.0}})
    assert cell == ("gemm_tiled_kernel<128, 128>: FETCH_SIZE=35628.7, WRITE_SIZE=2048; "
                    "splitk_finalize_kernel: FETCH_SIZE=8240")


@pytest.mark.gpu
def test_rocprof_metric_collects_counters_in_a_second_child(gpu_device):
    """--rocprof-pmc: one counter pass in a child run of its own; the split-K plan of this shape
    writes its fp32 partial sums and the finalize pass reads them."""
    import run as run_py

    out = run_py.run(["--op", "fp8_gemm_rowwise", "--m", "320", "--n", "1024", "--k", "8192", "--only", "_hip_mi355x",
                      "--metrics", "rocprof", "--rocprof-pmc", "WRITE_SIZE"])
    (x_val, per_backend), = out.result
    rec = per_backend["_hip_mi355x"]
    assert rec.error_msg is None
    cell = rec.extra_metrics["rocprof_counters"]
    print(cell, flush=True)
    assert "gemm_tiled_kernel<" in cell and "splitk_finalize_kernel: WRITE_SIZE=" in cell
    # the finalize pass writes the bf16 output: 320 x 1024 x 2 B = 640 KiB (the counter is in KiB)
    written = float(cell.split("splitk_finalize_kernel: WRITE_SIZE=")[1].split(";")[0].split(",")[0])
    assert 500.0 <= written <= 900.0
    assert "hip_mi355x-rocprof_counters" in str(out)
