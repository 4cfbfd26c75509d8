"""Host-side arithmetic the kernels rely on, restated and checked without a GPU.

The tiled kernel's tile walk divides work-item and tile numbers by two run-time constants (the
number of tiles, and the tiles in a group of tile rows). The launch code replaces both divisions by
a multiply and a shift with constants it prepares per launch (make_fast_div / fast_div in
tritonbench_amd/csrc/fp8_rowwise_gemm.hip): shift = 31 + ceil(log2 d), mul = ceil(2^shift / d),
n / d = (n * mul) >> shift for every 0 <= n < 2^31. The launch code admits at most 2^31 - 1 work
items, so that range is the whole domain. This file pins the formula; the GPU parity tests run the
walk itself on every tile configuration."""
import random


def make_fast_div(d):
    l = 0
    while (1 << l) < d:
        l += 1
    shift = 31 + l
    mul = ((1 << shift) + d - 1) // d
    return mul, shift


def fast_div(n, mul, shift):
    return ((n * mul) & ((1 << 64) - 1)) >> shift  # the kernel's product is a 64-bit unsigned multiply


def test_reciprocal_fits_32_bits_and_the_product_64():
    for d in list(range(1, 5000)) + [2 ** k + o for k in range(12, 31) for o in (-1, 0, 1)] + [2 ** 31 - 1]:
        mul, shift = make_fast_div(d)
        assert 0 < mul < 2 ** 32 and 31 <= shift <= 62
        assert (2 ** 31 - 1) * mul < 2 ** 64


def test_quotients_are_exact_over_the_whole_domain():
    rng = random.Random(1337)
    divisors = list(range(1, 300)) + [1024, 1025, 4095, 4096, 4097, 65535, 65536, 65537, 10 ** 6 + 3, 2 ** 24 - 1, 2 ** 30 + 1,
                                      2 ** 31 - 1] + [rng.randrange(1, 2 ** 31) for _ in range(300)]
    top = 2 ** 31 - 1
    for d in divisors:
        mul, shift = make_fast_div(d)
        edge = {0, 1, d - 1, d, d + 1, top, top - 1, (top // d) * d, (top // d) * d - 1}
        for q in (1, 2, 3, 7, 255, 256, 1023, 65535, top // d, max(top // d - 1, 0)):
            edge.update({q * d - 1, q * d, q * d + 1})
        samples = [n for n in edge if 0 <= n <= top] + [rng.randrange(0, 2 ** 31) for _ in range(200)]
        for n in samples:
            assert fast_div(n, mul, shift) == n // d, (n, d)


def test_exhaustive_for_small_divisors_and_numerators():
    for d in range(1, 130):
        mul, shift = make_fast_div(d)
        for n in range(0, 20000):
            assert fast_div(n, mul, shift) == n // d
