"""Pins the bit-level e4m3fn codec of the oracle (numpy and C) against the format's closed
form and against torch's cast, exhaustively where the domain is finite."""
import numpy as np
import torch

from oracle import cref, e4m3


def test_named_codes_closed_form():
    t = e4m3.decode_table()
    assert t[0x00] == 0.0 and t[0x80] == 0.0 and np.signbit(t[0x80])
    assert t[0x01] == 2.0 ** -9  # smallest subnormal
    assert t[0x07] == 7 * 2.0 ** -9
    assert t[0x08] == 2.0 ** -6  # smallest normal
    assert t[0x38] == 1.0
    assert t[0x3C] == 1.5
    assert t[0x40] == 2.0
    assert t[0x7E] == 448.0 and t[0xFE] == -448.0
    assert np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert np.isfinite(t).sum() == 254  # no infinities, two NaNs


def test_decode_monotone_and_symmetric():
    t = e4m3.decode_table()
    pos = t[:0x7F]
    assert np.all(np.diff(pos) > 0)
    assert np.array_equal(t[0x80:0xFF], -pos)


def test_decode_matches_torch_all_codes():
    t = e4m3.decode_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(t), np.isnan(tt))
    fin = ~np.isnan(t)
    assert np.array_equal(t[fin].view(np.uint32), tt[fin].view(np.uint32))


def test_c_decode_matches_numpy():
    lib = cref.load()
    t = e4m3.decode_table()
    for code in range(256):
        v = lib.oracle_e4m3_decode(code)
        if np.isnan(t[code]):
            assert np.isnan(v)
        else:
            assert np.float32(v) == t[code] and np.signbit(np.float32(v)) == np.signbit(t[code])


def _probe_points() -> np.ndarray:
    """Every code value, every midpoint between neighbours, and the floats just below and
    above each of them: the inputs where a wrong rounding rule shows."""
    t = e4m3.decode_table()[:0x7F].astype(np.float64)
    mids = (t[:-1] + t[1:]) / 2
    base = np.concatenate([t, mids, [464.0, 480.0, 1e-12, 2.0 ** -10, 3 * 2.0 ** -10]]).astype(np.float32)
    pts = np.concatenate([base, np.nextafter(base, np.float32(np.inf)), np.nextafter(base, np.float32(-np.inf))])
    return np.concatenate([pts, -pts]).astype(np.float32)


def test_encode_round_trip_all_codes():
    t = e4m3.decode_table()
    fin = ~np.isnan(t)
    codes = np.arange(256, dtype=np.uint8)[fin]
    assert np.array_equal(e4m3.encode_rne(t[fin]), codes)


def test_encode_ties_and_overflow_known_answers():
    enc = lambda v: int(e4m3.encode_rne(np.array([v], dtype=np.float32))[0])
    assert enc(448.0) == 0x7E
    assert enc(464.0) == 0x7E  # tie between 448 (even mantissa) and the NaN slot
    assert enc(np.nextafter(np.float32(464.0), np.float32(1e9))) == 0x7F
    assert enc(2.0 ** -10) == 0x00  # tie between 0 and 2^-9 -> even (0)
    assert enc(3 * 2.0 ** -10) == 0x02  # tie between 1 and 2 (x 2^-9) -> even (2)
    assert enc(np.nextafter(np.float32(2.0 ** -10), np.float32(1.0))) == 0x01
    assert enc(1.0625) == 0x38  # tie between 1.0 (m=0) and 1.125 (m=1) -> even
    assert enc(1.1875) == 0x3A  # tie between 1.125 (m=1) and 1.25 (m=2) -> even
    assert enc(-1.0) == 0xB8
    assert enc(7.5 * 2.0 ** -9) == 0x08  # rounds up into the first normal


def test_encode_matches_torch_on_probe_points_and_random():
    rng = np.random.default_rng(1337)
    x = np.concatenate([
        _probe_points(),
        rng.standard_normal(200000).astype(np.float32) * 100,
        rng.standard_normal(200000).astype(np.float32) * 0.01,
    ])
    mine = e4m3.encode_rne(x)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, ref)


def test_c_encode_matches_numpy_on_probe_points():
    lib = cref.load()
    x = _probe_points()
    mine = e4m3.encode_rne(x)
    for v, want in zip(x.tolist(), mine.tolist()):
        assert lib.oracle_e4m3_encode(v) == want, v
