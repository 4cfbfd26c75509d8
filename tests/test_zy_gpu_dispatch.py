"""The automatic choice of kernel family, tile configuration and split factor against the pinned
alternatives, timed on the device: the cost estimates behind the choice are tables of measured
constants, and a table that has drifted away from the kernels shows here as a choice that is
clearly slower than one of its alternatives. Needs an MI355X.

Timing (tritonbench_amd/tuning.py, the module behind the autotuned backend): a captured graph of
16 launches over rotating operand sets (cold weights, as a model's are), sustained bursts, the
median of three. The bar is 25 %: repeated measurements of one and the same plan on the shorter of
these shapes (10-30 us) differ by up to 8 % within a run (1 x 8192 x 16384 and 2048^3 have both shown
the automatic choice and the identical pinned plan that far apart), and plans of two launches move
more than that from run to run: 1024 x 1024 x 8192 in four splits has measured 19.7 to 26.8 us over
eight runs (its second kernel alone 4.9 to 7.1) with the unsplit plans beside it steady to 0.1 us.
A table that has drifted shows well beyond the bar (the 128x256 constants once put nineteen small
shapes 30-45 % off).

These are wall-clock assertions, not parity: they carry the `perf` marker beside `gpu`
(`-m "gpu and not perf"` leaves them out), every shape prints its margin, and the file sorts behind
every parity file so that a noisy replay cannot keep `pytest -x` from reaching those."""
import pytest
import torch

from tritonbench_amd import _lib, tuning

pytestmark = [pytest.mark.gpu, pytest.mark.perf]

TOLERANCE = 1.25
# decode- and small-prefill-sized rows of the Llama-3-70B projection sweep, and the small ragged shape with bias
SHAPES = [(32, 8192, 8192, False), (64, 8192, 8192, False), (128, 8192, 8192, False), (128, 10240, 8192, False),
          (32, 10240, 8192, False), (256, 8192, 8192, False), (1000, 3000, 4112, True),
          (128, 8192, 4096, False), (128, 8192, 28672, False), (256, 4096, 8192, False),
          (64, 4096, 8192, False), (128, 2048, 8192, False),
          # the rest of the decode rows (M = 1, 32, 128) of the Llama-3-70B sweep
          (1, 8192, 8192, False), (1, 10240, 8192, False), (1, 57344, 8192, False), (1, 8192, 28672, False),
          (32, 57344, 8192, False), (32, 8192, 28672, False), (128, 57344, 8192, False),
          # one tile row of 256x256 tiles with streamed B; several tile rows of the smaller configurations
          (256, 57344, 8192, False), (512, 16384, 16384, False),
          # decode-sized rows of the reference operator's own default sweep (operator.py:107-128); the
          # first is the shape of its stored run configuration
          (16, 13312, 13312, False), (1, 8192, 16384, False), (4, 13312, 2048, False), (8, 8192, 6656, False),
          (16, 4096, 6656, False), (32, 2304, 16384, False), (32, 8192, 13312, False), (64, 13312, 2048, False),
          (128, 2304, 6656, False), (128, 8192, 2304, False),
          # at most one 128x128 work item per CU: the deep-ring configuration, unsplit and split
          (1024, 2048, 4096, False), (2048, 2048, 2048, False), (1024, 1024, 8192, False), (1024, 2048, 16384, False),
          (768, 2048, 2048, False),
          # narrow panels with long rows: a few workgroups that each stream a long tile
          (1, 2048, 28672, False), (8, 1024, 28672, False), (16, 1024, 16384, False),
          # a vocabulary-wide panel with short rows (the output projection of a small model)
          (1, 128256, 2048, False), (8, 128256, 2048, False), (1, 151936, 1536, False)]


@pytest.mark.parametrize("m,n,k,bias", SHAPES)
def test_automatic_choice_is_close_to_the_best_alternative(gpu_device, m, n, k, bias):
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    dev = gpu_device
    # operand sets to rotate through: more than twice the 256 MB memory-side cache in total, as the
    # cost tables are calibrated on operands that come from HBM
    sets = tuning.make_operand_sets(m, n, k, bias, dev)
    alternatives = tuning.candidates(m, n, k)
    # two rounds over all candidates, the automatic choice first and last: whatever is timed first
    # runs on a colder clock
    # (further rounds, up to five in all, only if the bound does not hold after two: one noisy replay must not
    # fail the suite; every timing call runs on a fresh stream, so the rounds also see different hardware queues)
    times, auto = {name: float("inf") for name in alternatives}, float("inf")
    for rnd in range(5):
        auto = min(auto, tuning.time_variant_us(sets, _lib.VARIANT_AUTO))
        for name, v in alternatives.items():
            times[name] = min(times[name], tuning.time_variant_us(sets, v))
        auto = min(auto, tuning.time_variant_us(sets, _lib.VARIANT_AUTO))
        if rnd >= 1 and auto <= TOLERANCE * min(times.values()):
            break
    best_name = min(times, key=times.get)
    print(f"  automatic {auto:.1f} us = {auto / times[best_name]:.3f} x best ('{best_name}' {times[best_name]:.1f} us; "
          f"bar {TOLERANCE:.2f}); " + ", ".join(f"{nm} {t:.1f}" for nm, t in times.items()), flush=True)
    assert auto <= TOLERANCE * times[best_name], (
        f"automatic choice takes {auto:.1f} us, '{best_name}' {times[best_name]:.1f} us: the cost tables need recalibrating")
