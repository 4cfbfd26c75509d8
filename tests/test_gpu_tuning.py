"""The measured choice of plan (tritonbench_amd/tuning.py) and the operator backend built on it:
candidates per shape, cache, and that whatever it picks computes the same product. No timing is
asserted here. Needs an MI355X."""
import pytest
import torch

from oracle import fp8_rowwise as orc
from tritonbench_amd import _lib, ops, tuning


def test_candidate_plans_follow_the_shape_rules():
    c = tuning.candidates(16, 8192, 8192)
    assert set(c) == {f"tiled config {i}" for i in range(_lib.NUM_TILE_CONFIGS)} | {
        "skinny", "skinny, one tile per workgroup", "skinny, narrow tiles"}
    assert c["tiled config 2"] == _lib.tiled_variant(2, 0) and c["skinny"] == _lib.VARIANT_SKINNY
    assert "skinny" not in tuning.candidates(128, 8192, 8192) and "skinny, narrow tiles" in tuning.candidates(128, 8192, 8192)
    assert set(tuning.candidates(4096, 8192, 8192)) == {f"tiled config {i}" for i in range(_lib.NUM_TILE_CONFIGS)}
    assert tuning.candidates(64, 64, 24) == {"generic": _lib.VARIANT_GENERIC}  # K no multiple of 16: one family takes it


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,bias", [(16, 2048, 2048, False), (100, 1024, 1024, True), (8, 64, 40, False)])
def test_autotuned_plan_is_a_candidate_and_computes_the_product(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    dev = gpu_device
    tuning.clear_cache()
    sets = tuning.make_operand_sets(m, n, k, bias, dev, max_sets=4, min_bytes=1)
    variant, us, times = tuning.autotune(m, n, k, dev, bias=bias, sets=sets, rounds=1)
    assert variant in tuning.candidates(m, n, k).values() and us == min(times.values()) and us > 0
    assert tuning.autotune(m, n, k, dev, bias=bias) == (variant, us, times)  # cached: nothing is timed again
    xq, wq, xs, ws, b = orc.make_inputs(m, n, k, 1.0, bias)
    want = orc.dequant_matmul(xq, wq, xs, ws, b)
    got = ops.fp8_gemm_rowwise(xq.to(dev), wq.to(dev), xs.to(dev), ws.to(dev), bias=None if b is None else b.to(dev), variant=variant)
    torch.cuda.synchronize()
    torch.testing.assert_close(got.cpu(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
def test_autotuned_backend_runs_through_the_harness(gpu_device):
    """Disabled by default (like upstream's optional backends), selected with --only; its accuracy cell
    compares it with the CPU baseline like any other backend."""
    import run as run_py

    tuning.clear_cache()
    out = run_py.run(["--op", "fp8_gemm_rowwise", "--m", "64", "--n", "1024", "--k", "512", "--metrics", "latency,accuracy",
                      "--only", "_torch_dequant_cpu,_hip_mi355x,_hip_mi355x_autotuned"])
    (x_val, per_backend), = out.result
    assert x_val == (64, 1024, 512)
    for name in ("_hip_mi355x", "_hip_mi355x_autotuned"):
        assert per_backend[name].error_msg is None and per_backend[name].accuracy is True
    assert "hip_mi355x_autotuned-latency" in str(out)
    default = run_py.run(["--op", "fp8_gemm_rowwise", "--m", "64", "--n", "1024", "--k", "512", "--metrics", "latency"])
    assert "_hip_mi355x_autotuned" not in default.result[0][1]
