"""Pins the oracle's (and the library's) fp16 conversions: exhaustive round trip, ties, numpy cross-check."""
import numpy as np


def test_f16_to_f32_all_patterns_match_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f64_to_f16_round_trip_is_identity(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float64)
    ok = ~np.isnan(vals)
    back = oracle.f64_to_f16(vals[ok])
    assert np.array_equal(back, bits[ok])


def test_f64_to_f16_ties_and_edges_by_hand(oracle):
    cases = [
        (2049.0, 0x6800),  # halfway 2048/2050 -> even (2048)
        (2051.0, 0x6802),  # halfway 2050/2052 -> even (2052)
        (1.0 + 2.0 ** -11, 0x3C00),  # halfway 1 / 1+2^-10 -> even (1)
        (1.0 + 3 * 2.0 ** -11, 0x3C02),
        (65504.0, 0x7BFF), (65519.999, 0x7BFF), (65520.0, 0x7C00), (1e9, 0x7C00), (-1e9, 0xFC00),
        (2.0 ** -24, 0x0001), (2.0 ** -25, 0x0000), (2.0 ** -25 * 1.0000001, 0x0001), (3 * 2.0 ** -25, 0x0002),
        (2.0 ** -14, 0x0400), (2.0 ** -14 - 2.0 ** -25, 0x0400), (0.0, 0x0000), (-0.0, 0x8000), (1e-30, 0x0000),
        # a double that rounds differently if first squeezed through float32 (double rounding)
        (1.0 + 2.0 ** -11 + 2.0 ** -40, 0x3C01),
    ]
    x = np.array([c[0] for c in cases], dtype=np.float64)
    assert oracle.f64_to_f16(x).tolist() == [c[1] for c in cases]


def test_f64_to_f16_random_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 1, 200000), rng.normal(0, 1e-5, 100000), rng.normal(0, 3e4, 100000)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f64_to_f16(x), want)
