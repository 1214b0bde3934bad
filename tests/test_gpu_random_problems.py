"""Seeded random problems through the seam call with NO configuration named: whatever the
library's routing picks for a shape (VALU or matrix-core GEMV, rows in one or several
launches, K slices of equal or unequal length, tiled launches with or without K slices
across workgroups, the f32 routes) must give the oracle's result; a third of the problems
end their epilogue with a binary step on an [M,N] input, which has to move with every slice
of rows a route makes.

Tolerances: rel-L2 <= 1e-3 (the stated bar) everywhere; f16 activations with f32 output on
at most 16 rows <= 2e-6 (exact products, f32 accumulate: order noise only)."""
import os
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from helpers import f16_round, fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu

FORMATS = [("int4-grouped", 32), ("int4-grouped", 128), ("int8-grouped", 64), ("int8-grouped", 128), ("int8-row", 0)]
ROWS = [1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 17, 24, 31, 32, 33, 48, 63, 64, 65, 80, 100, 128, 130, 200, 256, 300, 513,
        1024, 2100]
ACTS = [None, "relu", "silu", "gelu"]


def draw(seed):
    rng = np.random.default_rng(seed)
    fmt, g = FORMATS[rng.integers(len(FORMATS))]
    m = int(ROWS[rng.integers(len(ROWS))])
    # K: a multiple of the group size; half of the draws of the 128 the matrix-core kernels take
    unit = 128 if rng.random() < 0.5 else max(g, 32)
    k = int(unit * rng.integers(1, 9216 // unit + 1))
    if rng.random() < 0.15:
        k = int(rng.choice([11008, 5504, 13696, 4096, 12288]))   # steps that no power of two divides, and the benchmark's own
    n = int(rng.choice([1, 15, 16, 17, 100, 256, 333, 515, 768, 1000, 1024, 2048, 4096, 8192, 12288]))
    if m * n * k > 6e9:   # keep the oracle to a second or two: a shorter K first (many tiles stay many)
        k = int(max(unit, (6e9 / (m * n)) // unit * unit))
    if m * n * k > 6e9:
        n = 256
    xdt = "f16" if rng.random() < 0.7 else "f32"
    ydt = "f16" if (xdt == "f16" and rng.random() < 0.5) else "f32"
    bias = rng.random() < 0.5
    act = ACTS[rng.integers(len(ACTS))]
    return rng, fmt, g, m, n, k, xdt, ydt, bias, act


def draw_binary(rng):
    """A third of the problems close their chain with a binary step on an [M,N] input (a
    residual add, or a gate), drawn after everything else so that the other draws stay."""
    return [None, None, "add", "mul", None, None][rng.integers(6)]


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


# TLHIP_TEST_RANDOM_PROBLEMS=<count> widens the sweep for a one-off run
@pytest.mark.parametrize("seed", range(int(os.environ.get("TLHIP_TEST_RANDOM_PROBLEMS", "160"))))
def test_whatever_the_routing_picks_matches_the_oracle(be, seed):
    rng, fmt, g, m, n, k, xdt, ydt, has_bias, act = draw(zlib.crc32(b"route-%d" % seed))
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, xdt, rng, std=0.5)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), ydt))
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    bias = f16_round(rng.standard_normal(n) * 0.1).astype(np.float32) if has_bias else None
    bt = be.ops.tensorFromArray(bias, [n], "f32") if has_bias else None
    sel = be.selectedConfig(w, xdt, m, ydt).as_tuple()
    binary = draw_binary(rng)
    other = f16_round(rng.standard_normal((m, n))).astype(np.float32) if binary else None
    ot = be.ops.tensorFromArray(other, [m, n], "f32") if binary else None

    def linear():
        ep = be.makeEpilogue(bt, act, (binary, ot) if binary else None)
        return be._matmulQuantizedB(xt, be.ops.transpose(w), ep, None)

    y = linear()
    got = y.numpy()
    want = O.linear(x.astype(np.float32), deq, bias, act or "none", threads=8)
    if binary:
        want = (want + other if binary == "add" else want * other).astype(np.float32)
    what = (fmt, g, m, n, k, xdt, ydt, has_bias, act, binary, sel)
    assert got.shape == (m, n), what
    assert got.dtype == (np.float16 if ydt == "f16" else np.float32), what
    assert np.isfinite(got).all(), what
    err = rel_l2(got, want)
    assert err <= 1e-3, (err, what)
    if xdt == "f16" and ydt == "f32" and m <= 16:
        assert err <= 2e-6, (err, what)
    # the same call again gives the same bits (no route depends on arrival order)
    y2 = linear()
    assert np.array_equal(y2.numpy(), got), what
    for t in (y, y2, xt, w) + ((bt,) if bt is not None else ()) + ((ot,) if ot is not None else ()):
        t.destroy()


# Launches of many tiles, which the draws above (kept small for the oracle) rarely reach: the
# default takes the kernel that keeps the weights packed up to the operand registers, on
# its 256-row tiles, for every format.
@pytest.mark.parametrize("fmt,g,m,n,k", [
    ("int8-grouped", 64, 1024, 12288, 256),
    ("int8-grouped", 128, 2100, 4096, 384),
    ("int8-row", 0, 513, 8192, 512),
    ("int8-row", 0, 2100, 4096, 256),
    ("int4-grouped", 32, 2100, 8192, 256),
    ("int4-grouped", 128, 4100, 8192, 128),
])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_many_tile_launches_on_the_default_route(be, fmt, g, m, n, k, ydt):
    rng = np.random.default_rng(m + n + k + g)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), ydt))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bias = f16_round(rng.standard_normal(n) * 0.1).astype(np.float32)
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    sel = be.selectedConfig(w, "f16", m, ydt).as_tuple()
    assert sel[0] == 3 and sel[1] == 256 or (fmt == "int4-grouped" and sel[:3] == (3, 128, 256)), sel
    y = be.linear(xt, w, bt, "silu", fused=True)
    got = y.numpy()
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    assert got.shape == (m, n) and np.isfinite(got).all()
    # per block of 256 x 256, so that one wrong tile cannot hide in the whole
    for r0 in range(0, m, 256):
        for c0 in range(0, n, 256):
            e = rel_l2(got[r0:r0 + 256, c0:c0 + 256], want[r0:r0 + 256, c0:c0 + 256])
            assert e <= 1e-3, (r0, c0, e, sel)
    for t in (y, xt, w, bt):
        t.destroy()
