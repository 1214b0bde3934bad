"""Pins for the oracle's rmsnorm / gated-activation restatements (CPU only).

The rows and the closed form are those of the reference's own RMSNorm test
(test/nn-rmsnorm.spec.ts:10-41, tolerance 1e-4 there); the remaining checks are
what the mathematics fixes: unit RMS of the output, invariance under scaling of
x when eps = 0, constant rows, and the role of each of the five f32 stores.
"""
import math

import numpy as np
import pytest

from oracle import quant_oracle as O

SPEC_ROWS = [
    [0.5, -1.2, 2.0, 0.1, -0.7, 1.5, -2.2, 0.9],
    [3.0, 0.0, -1.0, 0.25, 1.1, -0.4, 0.8, -1.6],
]


def closed_form(rows, w, eps):
    out = []
    for row in rows:
        ms = sum(v * v for v in row) / len(row)
        inv = 1.0 / math.sqrt(ms + eps)
        out.append([v * inv * w[j] for j, v in enumerate(row)])
    return np.array(out, np.float64)


def test_rmsnorm_reference_spec_rows():
    x = np.array(SPEC_ROWS, np.float32)
    got = O.rmsnorm(x, np.ones(8, np.float32), 1e-6)
    want = closed_form(SPEC_ROWS, [1.0] * 8, 1e-6)
    assert np.max(np.abs(got - want)) < 1e-6  # the reference asserts 1e-4


def test_rmsnorm_weight_is_applied_per_column():
    x = np.array(SPEC_ROWS, np.float32)
    w = np.array([1.5, -2.0, 0.25, 3.0, 0.0, 1.0, -0.5, 4.0], np.float32)
    got = O.rmsnorm(x, w, 1e-6)
    want = closed_form(SPEC_ROWS, [float(v) for v in w], 1e-6)
    assert np.max(np.abs(got - want)) < 2e-6
    assert np.all(got[:, 4] == 0.0)


def test_rmsnorm_unit_rms_and_scale_invariance():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 1024)).astype(np.float32)
    ones = np.ones(1024, np.float32)
    y = O.rmsnorm(x, ones, 0.0)
    rms = np.sqrt(np.mean(y.astype(np.float64) ** 2, axis=1))
    assert np.max(np.abs(rms - 1.0)) < 1e-5  # sequential f32 sum of 1024 squares
    # powers of two scale x exactly, so the output is bit-identical
    assert np.array_equal(O.rmsnorm(x * np.float32(8.0), ones, 0.0), y)
    y3 = O.rmsnorm(x * np.float32(3.0), ones, 0.0)
    assert np.max(np.abs(y3 - y)) < 1e-5


def test_rmsnorm_constant_rows_and_eps():
    d = 64
    x = np.full((1, d), -2.5, np.float32)
    w = np.linspace(-1, 1, d).astype(np.float32)
    y = O.rmsnorm(x, w, 0.0)
    assert np.max(np.abs(y + w)) < 1e-7  # x / |x| = -1
    # eps enters under the root: a zero row stays zero, a tiny row is damped
    assert np.all(O.rmsnorm(np.zeros((2, d), np.float32), w, 1e-6) == 0.0)
    tiny = np.full((1, d), 1e-4, np.float32)
    got = O.rmsnorm(tiny, np.ones(d, np.float32), 1e-6)
    assert np.max(np.abs(got - 1e-4 / math.sqrt(1e-8 + 1e-6))) < 1e-8


def test_rmsnorm_running_sum_rounds_to_f32_every_step():
    # 2^24 + 1 is not an f32: a sequential f32 sum of ones stalls at 2^24, a
    # double sum does not.  d = 2^24 + 64 ones of value 1: sum = 2^24 exactly.
    d = (1 << 24) + 64
    x = np.ones((1, d), np.float32)
    y = O.rmsnorm(x, np.ones(d, np.float32), 0.0)
    mean = np.float32(np.float32(1 << 24) / np.float64(d))
    inv = np.float32(1.0 / math.sqrt(float(mean)))
    assert y[0, 0] == inv and y[0, -1] == inv
    assert inv > 1.0  # a double-accumulated mean would be exactly 1


def test_rmsnorm_matches_numpy_f32_steps():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((5, 333)) * 3).astype(np.float32)
    w = rng.standard_normal(333).astype(np.float32)
    eps = 1e-5
    sq = x * x
    s = np.zeros(5, np.float32)
    for i in range(333):
        s = (s + sq[:, i]).astype(np.float32)
    mean = (s.astype(np.float64) / 333).astype(np.float32)
    t = (mean.astype(np.float64) + eps).astype(np.float32)
    inv = (1.0 / np.sqrt(t.astype(np.float64))).astype(np.float32)
    want = (x * inv[:, None]) * w[None, :]
    assert np.array_equal(O.rmsnorm(x, w, eps), want)


def test_mul_is_ieee_f32_product():
    rng = np.random.default_rng(2)
    a = rng.standard_normal(4096).astype(np.float32) * np.float32(1e3)
    b = rng.standard_normal(4096).astype(np.float32) * np.float32(1e-3)
    assert np.array_equal(O.mul(a, b), a * b)


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_gated_is_two_f32_ops(act):
    rng = np.random.default_rng(3)
    g = (rng.standard_normal(2048) * 4).astype(np.float32)
    u = rng.standard_normal(2048).astype(np.float32)
    want = O.np_unary(act, g) * u
    got = O.gated(g, u, act)
    assert np.max(np.abs(got.astype(np.float64) - want)) <= 1e-6 * np.max(np.abs(want))
    # silu(0) = 0, gelu(0) = 0: a zero gate kills the product whatever `up` is
    assert np.all(O.gated(np.zeros(8, np.float32), u[:8], act) == 0.0)
