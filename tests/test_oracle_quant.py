"""Pins the oracle's quantize / dequantize (quantize.ts:77-156 and the two
benchmark formats) by exact rational arithmetic, hand-worked cases, invariants
and brute force over the whole (q, scale) table."""
import json
import os
import struct
from fractions import Fraction

import numpy as np
import pytest

from oracle import quant_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def f32(x: float) -> float:
    return struct.unpack("<f", struct.pack("<f", x))[0]


def pack_bytes(qs):
    q = np.asarray(qs, np.int8).reshape(1, -1)
    return O.np_pack_int8(q)


# ------------------------------------------------------------------ packing

def test_int8_byte_lane_layout_is_little_endian_k_major():
    # word = q0 | q1<<8 | q2<<16 | q3<<24, lowest k in the lowest byte
    # (docs/quantization-design.md:57-60; quantize.ts:121-125)
    w = np.arange(1, 9, dtype=np.float32) / 8 * 127 / 127  # absmax 1.0 -> q = round(w*127)
    packed, scales = O.quantize_int8_grouped(w, 1, 8, 4)
    s0 = O.f16_bits_to_f32(scales)[0]
    q = np.floor(w[:4].astype(np.float64) * (127.0 / s0) + 0.5).astype(np.int64)
    assert packed[0] == (q[0] | q[1] << 8 | q[2] << 16 | q[3] << 24)
    assert packed.view(np.uint8)[:4].tolist() == q.tolist()


def test_int8_pack_unpack_round_trip_and_negative_bytes():
    q = np.array([[-128, -127, -1, 0, 1, 2, 126, 127]], np.int8)
    p = O.np_pack_int8(q)
    assert p.tolist() == [0x00FF8180, 0x7F7E0201]
    assert np.array_equal(O.np_unpack_int8(p, 1, 8), q)


def test_int4_nibble_layout():
    # nibble j of word holds k = 8*word + j (docs/quantization-design.md:69-75)
    q = np.array([[0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1]], np.int8)
    p = O.np_pack_int4(q)
    assert p.tolist() == [0x76543210, 0xFEDCBA98]
    assert np.array_equal(O.np_unpack_int4(p, 1, 16), q)
    s = np.full(1, 0x3C00, np.uint16)  # 1.0
    out = O.dequant_int4_grouped(p, s, 1, 16, 16)
    assert out.ravel().tolist() == q.ravel().astype(np.float32).tolist()


# ------------------------------------------------------------------ dequant

def _exact_f32_of_fraction(fr: Fraction) -> float:
    """Correctly rounded f32 of an exact rational via Python's correctly
    rounded int/int true division (then one more rounding to f32 — only used
    where the double is itself exact or far from an f32 tie)."""
    return f32(fr.numerator / fr.denominator)


def test_dequant_int8_grouped_hand_cases():
    one = 0x3C00
    out = O.dequant_int8_grouped(pack_bytes([127, -127, 0, 1]), np.array([one], np.uint16), 1, 4, 4)
    assert out.ravel().tolist() == [1.0, -1.0, 0.0, f32(1 / 127)]
    # -128 is not clamped (quantize.ts:149-150): -128/127
    out = O.dequant_int8_grouped(pack_bytes([-128, 64, 2, 3]), np.array([0x4000], np.uint16), 1, 4, 4)
    assert out.ravel().tolist() == [f32((-128 / 127) * 2.0), f32((64 / 127) * 2.0),
                                    f32((2 / 127) * 2.0), f32((3 / 127) * 2.0)]
    assert out.ravel()[0] < -2.0


def test_dequant_int8_grouped_is_double_arithmetic_not_f32():
    """The reference evaluates (qi / 127) * scale on JavaScript doubles and
    rounds once into the Float32Array (quantize.ts:152).  Doing the same two
    operations in f32 (what a GPU kernel would naively do) differs for many
    pairs; plain Python floats are the same IEEE doubles as JavaScript's, so
    they decide which one the oracle must equal."""
    rng = np.random.default_rng(3)
    found = 0
    for _ in range(20000):
        q = int(rng.integers(-127, 128))
        sb = int(rng.integers(0x0400, 0x7C00))
        s = float(np.uint16(sb).view(np.float16))
        as_double = f32((q / 127) * s)
        as_f32 = float(np.float32(np.float32(q) / np.float32(127)) * np.float32(s))
        if as_double != as_f32:
            got = O.dequant_int8_grouped(pack_bytes([q, 0, 0, 0]), np.array([sb], np.uint16), 1, 4, 4)
            assert got[0, 0] == as_double
            found += 1
    assert found >= 100


def test_dequant_int8_grouped_within_half_ulp_of_exact_rational():
    rng = np.random.default_rng(5)
    for _ in range(300):
        q = int(rng.integers(-128, 128))
        sb = int(rng.integers(1, 0x7C00))
        s = Fraction(float(np.uint16(sb).view(np.float16)))
        exact = Fraction(q, 127) * s
        got = float(O.dequant_int8_grouped(pack_bytes([q, 0, 0, 0]), np.array([sb], np.uint16), 1, 4, 4)[0, 0])
        if exact == 0:
            assert got == 0.0
            continue
        ulp = Fraction(float(np.spacing(np.float32(abs(got)))))
        # two double roundings then one f32 rounding: within 0.5 ulp(f32) + 2^-52 relative
        assert abs(Fraction(got) - exact) <= ulp / 2 + abs(exact) * Fraction(1, 2 ** 50)


def test_dequant_full_table_c_vs_numpy_float64():
    """Output depends only on (q, scale bits): all 256 x 65536 pairs."""
    sb = np.arange(65536, dtype=np.uint16)
    for q in range(-128, 128):
        packed = np.repeat(pack_bytes([q, q, q, q]), 65536 // 4)
        # one row per scale would be slow; use n=65536 rows of k=4, G=4
        packed = np.full(65536, pack_bytes([q, q, q, q])[0], np.uint32)
        c = O.dequant_int8_grouped(packed, sb, 65536, 4, 4)
        n = O.np_dequant_int8_grouped(packed, sb, 65536, 4, 4)
        cn, nn = np.isnan(c), np.isnan(n)
        assert np.array_equal(cn, nn)
        assert np.array_equal(c[~cn].view(np.uint32), n[~nn].view(np.uint32)), q


def test_dequant_int8_grouped_structure():
    rng = np.random.default_rng(11)
    n, k, g = 6, 256, 64
    q = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = O.f32_to_f16_bits(rng.uniform(0.01, 2.0, n * k // g).astype(np.float32))
    out = O.dequant_int8_grouped(O.np_pack_int8(q), sb, n, k, g)
    s = O.f16_bits_to_f32(sb).reshape(n, k // g)
    # group structure: element (r, c) uses scale (r, c // g)
    srep = np.repeat(s, g, axis=1)
    assert np.array_equal(out[q == 127], srep[q == 127])
    assert np.array_equal(out[q == -127], -srep[q == -127])
    assert np.all(out[q == 0] == 0)
    # odd symmetry and monotonicity in q for a positive scale
    neg = O.dequant_int8_grouped(O.np_pack_int8((-q).astype(np.int8)), sb, n, k, g)
    assert np.array_equal(neg, -out)
    assert np.array_equal(out, O.np_dequant_int8_grouped(O.np_pack_int8(q), sb, n, k, g))


def test_dequant_int8_row_is_the_exact_product():
    rng = np.random.default_rng(13)
    n, k = 64, 128
    q = rng.integers(-128, 128, (n, k)).astype(np.int8)
    s = rng.uniform(0.002, 0.02, n).astype(np.float32)
    out = O.dequant_int8_row(O.np_pack_int8(q), s, n, k)
    # q (8 bits) * s (24 bits) is exact in double; f32 product is its correct rounding
    want = (q.astype(np.float32) * s[:, None]).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    for r, c in [(0, 0), (5, 77), (63, 127)]:
        exact = Fraction(int(q[r, c])) * Fraction(float(s[r]))
        assert float(out[r, c]) == f32(exact.numerator / exact.denominator)
    assert np.array_equal(out, O.np_dequant_int8_row(O.np_pack_int8(q), s, n, k))


def test_dequant_int4_grouped_is_exact_in_f32_for_all_pairs():
    """q in [-8,7] times an 11-bit significand needs at most 15 bits: exact in
    f32.  All 16 x 65536 pairs against exact rationals (sampled) and numpy."""
    sb = np.arange(65536, dtype=np.uint16)
    sv = sb.view(np.float16).astype(np.float64)
    for q in range(-8, 8):
        word = np.uint32(sum(((q & 0xF) << (4 * j)) for j in range(8)))
        packed = np.full(65536, word, np.uint32)
        out = O.dequant_int4_grouped(packed, sb, 65536, 8, 8)
        with np.errstate(invalid="ignore"):
            want = (q * sv).astype(np.float32)
        ok = ~np.isnan(want)
        assert np.array_equal(np.isnan(out[:, 0]), ~ok)
        assert np.array_equal(out[ok, 0].view(np.uint32), want[ok].view(np.uint32))
        # exactness: f32 result equals the real product wherever it is a normal f32
        fin = ok & np.isfinite(sv) & (np.abs(want) >= 2.0 ** -126)
        assert np.array_equal(out[fin, 0].astype(np.float64), q * sv[fin])
        assert np.array_equal(out[:, 3], out[:, 0], equal_nan=True)
    rng = np.random.default_rng(17)
    for _ in range(100):
        q, b = int(rng.integers(-8, 8)), int(rng.integers(0x0400, 0x7C00))
        exact = Fraction(q) * Fraction(float(np.uint16(b).view(np.float16)))
        word = np.array([(q & 0xF)], np.uint32)
        got = O.dequant_int4_grouped(word, np.array([b], np.uint16), 1, 8, 8)[0, 0]
        assert Fraction(float(got)) == exact


# ----------------------------------------------------------------- quantize

def test_quantize_argument_errors_match_reference_messages():
    w = np.zeros(16, np.float32)
    with pytest.raises(ValueError, match="expected 32 elements, got 16"):
        O.quantize_int8_grouped(w, 4, 8, 4)
    with pytest.raises(ValueError, match="K=6 must be divisible by 4"):
        O.quantize_int8_grouped(np.zeros(12, np.float32), 2, 6, 2)
    with pytest.raises(ValueError, match="K=8 must be divisible by groupSize=3"):
        O.quantize_int8_grouped(w, 2, 8, 3)


def test_quantize_hand_worked_group():
    # absmax 2.0 (f16 exact) -> inv = 63.5; values chosen to land on half-integers
    w = np.array([2.0, -2.0, 0.5 / 63.5, -0.5 / 63.5], np.float64)
    w32 = w.astype(np.float32)
    packed, scales = O.quantize_int8_grouped(w32, 1, 4, 4)
    assert scales[0] == 0x4000
    t = w32.astype(np.float64) * 63.5
    want = [127, -127] + [int(np.floor(v + 0.5)) for v in t[2:]]
    assert O.np_unpack_int8(packed, 1, 4).ravel().tolist() == want


def test_quantize_math_round_ties_go_toward_plus_infinity():
    """Math.round(2.5)=3, Math.round(-2.5)=-2, Math.round(-0.5)=-0 -> 0
    (quantize.ts:116-119).  With absmax 127 the multiplier is exactly 1."""
    w = np.array([127.0, 2.5, -2.5, -0.5, 0.5, 1.5, -1.5, -126.5], np.float32)
    packed, scales = O.quantize_int8_grouped(w, 1, 8, 8)
    assert O.f16_bits_to_f32(scales)[0] == 127.0
    assert O.np_unpack_int8(packed, 1, 8).ravel().tolist() == [127, 3, -2, 0, 1, 2, -1, -126]


def test_quantize_zero_group_nan_and_inf():
    w = np.zeros(12, np.float32)
    w[4:8] = [np.nan, 1.0, -0.25, np.nan]      # NaN ignored by absmax, quantizes to 0
    w[8:12] = [np.inf, 1.0, -1.0, 0.0]         # scale inf -> inv 0 -> inf*0 = NaN -> 0
    packed, scales = O.quantize_int8_grouped(w, 1, 12, 4)
    q = O.np_unpack_int8(packed, 1, 12).ravel().tolist()
    assert scales.tolist() == [0, 0x3C00, 0x7C00]
    assert q == [0, 0, 0, 0, 0, 127, -32, 0, 0, 0, 0, 0]
    # -0.25*127 = -31.75 -> -32
    deq = O.dequant_int8_grouped(packed, scales, 1, 12, 4).ravel()
    assert np.all(deq[:4] == 0) and np.isnan(deq[8:]).all()  # 0 * inf = NaN, as in JS


def test_quantize_clamps_when_f16_scale_rounds_below_absmax():
    # absmax 1.0004 rounds down to f16 1.0 -> w*127 = 127.05 -> clamp to 127
    w = np.array([1.0004, -1.0004, 0.5, 0.0], np.float32)
    packed, scales = O.quantize_int8_grouped(w, 1, 4, 4)
    assert scales[0] == 0x3C00
    assert O.np_unpack_int8(packed, 1, 4).ravel().tolist() == [127, -127, 64, 0]


@pytest.mark.parametrize("g", [64, 128])
def test_quantize_invariants_on_probe_style_weights(g):
    cases = json.load(open(os.path.join(GOLD, "quant_probe_cases.json")))["gemv_probe"]
    draw = O.make_lcg(cases["seed"])
    n, k = 512, 1024
    w = draw(n * k).astype(np.float32).reshape(n, k)
    packed, scales = O.quantize_int8_grouped(w, n, k, g)
    q = O.np_unpack_int8(packed, n, k)
    assert q.min() >= -127 and q.max() <= 127
    s = O.f16_bits_to_f32(scales).reshape(n, k // g)
    absmax = np.abs(w.reshape(n, k // g, g)).max(-1)
    # stored scale is the f16 rounding of the group's abs-max (file header of quantize.ts)
    assert np.array_equal(scales.reshape(n, k // g), O.f32_to_f16_bits(absmax).reshape(n, k // g))
    # the arg-max element maps to +-127
    am = np.abs(w.reshape(n, k // g, g)).argmax(-1)
    qam = np.take_along_axis(q.reshape(n, k // g, g), am[..., None], -1)[..., 0]
    assert np.all(np.abs(qam) == 127)
    # reconstruction error bounded by half a step (plus f16 scale rounding on clamped maxima)
    deq = O.dequant_int8_grouped(packed, scales, n, k, g)
    step = np.repeat(s, g, axis=1) / 127.0
    err = np.abs(deq.astype(np.float64) - w.astype(np.float64))
    assert np.all(err <= 0.5 * step + np.abs(w) * 2.0 ** -11 + 1e-9)
    # idempotence: re-quantizing the dequantized weight reproduces the same integers
    p2, s2 = O.quantize_int8_grouped(deq, n, k, g)
    assert np.array_equal(s2, scales) and np.array_equal(p2, packed)
    # numpy restatement agrees bit for bit
    p3, s3 = O.np_quantize_int8_grouped(w, n, k, g)
    assert np.array_equal(s3, scales) and np.array_equal(p3, packed)


def test_quantize_c_vs_numpy_on_adversarial_half_integers():
    rng = np.random.default_rng(23)
    n, k, g = 64, 256, 64
    # weights that are exact multiples of absmax/254 land on .5 after scaling
    base = rng.integers(-254, 255, (n, k)).astype(np.float64) / 254.0
    base[:, ::g] = 1.0
    amp = np.exp2(rng.integers(-6, 4, (n, 1)).astype(np.float64))
    w = (base * amp).astype(np.float32)
    a = O.quantize_int8_grouped(w, n, k, g)
    b = O.np_quantize_int8_grouped(w, n, k, g)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
