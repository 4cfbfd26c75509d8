"""Bit-level OCP e4m3fn codec in numpy. TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Written from the format definition, independently of torch's cast, so the two can be
checked against each other:
    sign(1) | exponent(4, bias 7) | mantissa(3)
    exponent 0      : subnormal, value = m/8 * 2^-6            (spacing 2^-9)
    exponent 1..15  : value = (1 + m/8) * 2^(e-7)
    0x7f / 0xff     : NaN (the only non-finite codes; there is no infinity)
    largest finite  : 0x7e = 1.75 * 2^8 = 448

The format is the one tritonbench's operator quantises to
(tritonbench/operators/fp8_gemm_rowwise/operator.py:130-131: FP8_DTYPE / E4M3_MAX_POS).

Pinned by tests/test_oracle_e4m3.py: closed-form values of named codes, monotonicity,
exhaustive round trip, exhaustive agreement with torch.float8_e4m3fn on all 256 codes and
on every midpoint / neighbour of midpoint between adjacent codes.
"""
import numpy as np

E4M3_MAX = 448.0
E4M3_MIN_SUBNORMAL = 2.0 ** -9
E4M3_MIN_NORMAL = 2.0 ** -6


def decode_table() -> np.ndarray:
    """float32[256]: value of every code (NaN at 0x7f and 0xff)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            out[code] = np.nan
        elif e == 0:
            out[code] = sign * (m / 8.0) * 2.0 ** -6
        else:
            out[code] = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


_TABLE = decode_table()


def decode(codes: np.ndarray) -> np.ndarray:
    """uint8 codes -> float32 values."""
    return _TABLE[np.asarray(codes, dtype=np.uint8)]


def encode_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn code, round to nearest, ties to even; no saturation:
    anything that rounds past 448 becomes NaN (0x7f | sign), as a plain cast does."""
    x = np.asarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    mag = np.abs(x).astype(np.float64)  # exact
    out = np.zeros(x.shape, dtype=np.uint8)

    nan = np.isnan(x)
    # subnormal range: multiples of 2^-9 up to 2^-6
    sub = mag < E4M3_MIN_NORMAL
    q_sub = np.rint(mag * 512.0)  # numpy rint is ties-to-even; result 0..8 (8 == first normal, code 0x08)
    # normal range
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(mag > 0, mag, 1.0)))
    e = np.clip(e, -6, 8)
    q = np.rint(mag / 2.0 ** e * 8.0)  # in [8, 16]
    carry = q >= 16
    e = np.where(carry, e + 1, e)
    q = np.where(carry, 8, q)
    code_norm = ((e + 7).astype(np.int64) << 3) | (q.astype(np.int64) - 8)
    overflow = (e > 8) | ((e == 8) & (q > 14)) | np.isinf(mag)
    code = np.where(sub, q_sub.astype(np.int64), code_norm)
    code = np.where(overflow | nan, 0x7F, code)
    out = (code.astype(np.uint8) | sign).astype(np.uint8)
    return out
