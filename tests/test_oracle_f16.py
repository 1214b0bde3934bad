"""Pins the oracle's f16 codec (quantize.ts:22-60) against numpy's IEEE
binary16 routines and against closed forms derived independently of the bit
manipulation the reference uses."""
import struct

import numpy as np
import pytest

from oracle import quant_oracle as O


def test_f16_decode_all_patterns_match_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    got = O.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # the numpy restatement agrees too (signed zeros included)
    got64 = O.np_f16_bits_to_f64(bits)
    assert np.array_equal(got64[~nan].astype(np.float32).view(np.uint32),
                          want[~nan].view(np.uint32))


def test_f16_decode_known_values():
    f = O.lib().ref_f16_bits_to_f64
    assert f(0x3C00) == 1.0
    assert f(0xC000) == -2.0
    assert f(0x7BFF) == 65504.0
    assert f(0x0001) == 2.0 ** -24
    assert f(0x0400) == 2.0 ** -14
    assert f(0x7C00) == float("inf") and f(0xFC00) == float("-inf")
    assert np.isnan(f(0x7E00))
    assert struct.pack("<d", f(0x8000)) == struct.pack("<d", -0.0)


def _all_f32_with_exponent(e_lo, e_hi, stride=1):
    """Positive f32 bit patterns with biased exponent in [e_lo, e_hi)."""
    return np.arange(e_lo << 23, e_hi << 23, stride, dtype=np.uint32)


def test_f16_encode_normals_match_numpy_rne_exhaustive_strided():
    # every normal-result exponent (113..142); mantissas on a stride that is
    # coprime to 2^13 so that all rounding remainders occur, plus all exact
    # ties and their neighbours.
    u = _all_f32_with_exponent(113, 143, stride=37)
    ties = (np.arange(113 << 23, 143 << 23, 1 << 13, dtype=np.uint32) | 0x1000)
    u = np.concatenate([u, ties, ties - 1, ties + 1])
    for sign in (0, 0x80000000):
        x = (u | np.uint32(sign)).view(np.float32)
        got = O.f32_to_f16_bits(x)
        with np.errstate(over="ignore"):
            want = x.astype(np.float16).view(np.uint16)
        assert np.array_equal(got, want)


def test_f16_encode_top_binade_exhaustive():
    # exponent 142 is where rounding overflows into inf (65520 and above)
    u = _all_f32_with_exponent(142, 143)
    x = u.view(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), want)
    assert O.f32_to_f16_bits(np.float32(65519.99))[0] == 0x7BFF
    assert O.f32_to_f16_bits(np.float32(65520.0))[0] == 0x7C00


def test_f16_encode_subnormal_range_is_round_half_up():
    """For |x| < 2^-14 the reference truncates to 2^-37 units and then adds bit
    12: algebraically floor(|x|*2^24 + 1/2).  Checked on EVERY f32 in the
    range (exponents 102..112, 11 * 2^23 patterns) in chunks."""
    for e in range(102, 113):
        u = _all_f32_with_exponent(e, e + 1)
        x = u.view(np.float32)
        want = np.floor(x.astype(np.float64) * 2.0 ** 24 + 0.5).astype(np.uint16)
        got = O.f32_to_f16_bits(x)
        assert np.array_equal(got, want), e
        # and the negative side on a stride
        xn = (u[::257] | np.uint32(0x80000000)).view(np.float32)
        assert np.array_equal(O.f32_to_f16_bits(xn), want[::257] | 0x8000)


def test_f16_encode_deviations_from_ieee_are_exactly_the_ties_to_even_cases():
    """numpy rounds ties to even; the reference rounds them up.  The two differ
    exactly where |x|*2^24 has fraction 1/2 and an even integer part."""
    u = _all_f32_with_exponent(102, 113, stride=1 << 9)  # keeps all tie patterns of low exps
    x = u.view(np.float32)
    got = O.f32_to_f16_bits(x)
    want_ieee = x.astype(np.float16).view(np.uint16)
    t = x.astype(np.float64) * 2.0 ** 24
    is_even_tie = (t - np.floor(t) == 0.5) & (np.floor(t) % 2 == 0)
    assert np.array_equal(got != want_ieee, is_even_tie)
    assert is_even_tie.any()
    # smallest case: 2^-25 is a tie between 0 and the least subnormal
    assert O.f32_to_f16_bits(np.float32(2.0 ** -25))[0] == 1
    assert np.float32(2.0 ** -25).astype(np.float16).view(np.uint16) == 0


def test_f16_encode_special_values():
    f = lambda v: int(O.f32_to_f16_bits(np.float32(v))[0])
    assert f(0.0) == 0 and f(-0.0) == 0x8000
    assert f(1.0) == 0x3C00 and f(-2.0) == 0xC000
    assert f(65504.0) == 0x7BFF
    assert f(np.inf) == 0x7C00 and f(-np.inf) == 0xFC00
    assert f(1e10) == 0x7C00
    assert f(np.nan) & 0x7FFF == 0x7C00  # NaN collapses to the inf pattern (quantize.ts:38)
    below = np.nextafter(np.float32(2.0 ** -25), np.float32(0))
    assert f(below) == 0 and f(-below) == 0x8000  # exp < -10 -> signed zero (quantize.ts:32)
    assert f(2.0 ** -14) == 0x0400
    assert f(np.nextafter(np.float32(2.0 ** -14), np.float32(0))) == 0x0400  # rounds up into normal
    # f32 denormals have biased exponent 0 -> far below 2^-25
    assert f(np.float32(1e-40)) == 0


def test_numpy_restatement_of_encode_agrees_with_c():
    rng = np.random.default_rng(7)
    u = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    assert np.array_equal(O.f32_to_f16_bits(x), O.np_f32_to_f16_bits(x))
    # concentrate on the f16 range too
    x = (rng.standard_normal(1_000_000) * np.exp(rng.uniform(-20, 12, 1_000_000))).astype(np.float32)
    assert np.array_equal(O.f32_to_f16_bits(x), O.np_f32_to_f16_bits(x))


def test_round_trip_of_every_finite_f16():
    bits = np.arange(65536, dtype=np.uint16)
    finite = (bits & 0x7C00) != 0x7C00
    vals = O.f16_bits_to_f32(bits[finite])
    assert np.array_equal(O.f32_to_f16_bits(vals), bits[finite])
