"""Pins the oracle's matmul and epilogue arithmetic (numeric.ts:510-595,
439-446; catalog.ts / composite.ts) against the reference's own known answers
and the formulas written out in its epilogue spec."""
import json
import math
import os

import numpy as np
import pytest

from oracle import quant_oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


@pytest.mark.parametrize("case", GOLD["matmul"], ids=lambda c: str(c["a_shape"]) + "x" + str(c["b_shape"]))
def test_matmul_reference_known_answers(case):
    a = np.array(case["a"], np.float32).reshape(case["a_shape"])
    b = np.array(case["b"], np.float32).reshape(case["b_shape"])
    out = O.matmul(a, b)
    assert list(out.shape) == case["out_shape"]
    assert out.ravel().tolist() == case["out"]


def test_matmul_mismatch_raises_reference_message():
    c = GOLD["matmul_mismatch"]
    with pytest.raises(ValueError, match=c["message"]):
        O.matmul(np.zeros(c["a_shape"], np.float32), np.zeros(c["b_shape"], np.float32))
    with pytest.raises(ValueError, match=c["message"]):
        O.matmul_nt(np.zeros((1, 4), np.float32), np.zeros((3, 8), np.float32))


def test_matmul_nt_equals_strided_matmul_on_transposed_view():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 96)).astype(np.float32)
    w = rng.standard_normal((17, 96)).astype(np.float32)
    a = O.matmul_nt(x, w)
    b = O.matmul(x, w.T)  # api.linear passes the transposed VIEW (torchlette.ts:887-891)
    assert np.array_equal(a, b)
    assert np.array_equal(O.matmul_nt(x, w, threads=4), a)


def test_matmul_accumulates_in_double_and_rounds_once():
    # 2^24 + 1 + 1 - 2^24: exact in double, lost in f32 sequential accumulation
    x = np.array([[2.0 ** 24, 1.0, 1.0, -(2.0 ** 24)]], np.float32)
    w = np.ones((1, 4), np.float32)
    assert O.matmul_nt(x, w)[0, 0] == 2.0
    acc = np.float32(0)
    for v in x[0]:
        acc = np.float32(acc + v)
    assert acc != 2.0
    # one rounding: result is the f32 nearest to the exact sum of exact products
    rng = np.random.default_rng(2)
    xs = rng.standard_normal((4, 257)).astype(np.float32)
    ws = rng.standard_normal((9, 257)).astype(np.float32)
    got = O.matmul_nt(xs, ws)
    for i in range(4):
        for j in range(9):
            exact = math.fsum(float(a) * float(b) for a, b in zip(xs[i], ws[j]))
            assert abs(float(got[i, j]) - exact) <= 0.5 * float(np.spacing(np.float32(abs(got[i, j])))) * 1.0001
    assert np.max(np.abs(got.astype(np.float64) - O.np_matmul_nt(xs, ws))) <= np.spacing(np.float32(np.abs(got).max()))


def _values(size, offset, scale):
    return ((np.arange(size) + offset) % 7 - 3).astype(np.float64) * scale


@pytest.mark.parametrize("case", GOLD["epilogue"]["cases"], ids=lambda c: c["name"])
def test_epilogue_matches_reference_spec_formulas(case):
    """Inputs and expected values are built exactly as the reference's epilogue
    spec builds them (matmul-epilogue.spec.ts:21-75); the oracle's per-op f32
    pipeline must satisfy that spec's closeness bound."""
    m, n, k, sc = case["m"], case["n"], case["k"], case["scale"]
    off = GOLD["epilogue"]["offsets"]
    a = _values(m * k, off["a"], sc).reshape(m, k)
    b = _values(k * n, off["b"], sc).reshape(k, n)
    bias = _values(n, off["bias"], sc)
    expected = np.zeros((m, n))
    for t in range(k):  # matmulReference: sum over t in increasing order
        expected += np.outer(a[:, t], b[t, :])
    got = O.matmul(a.astype(np.float32), b.astype(np.float32))
    for op in case["ops"]:
        if op == "bias":
            expected = expected + bias[None, :]
            got = O.bias_add(got, bias.astype(np.float32))
        elif op == "relu":
            expected = np.maximum(0, expected)
            got = O.unary("relu", got)
        elif op == "gelu":
            c = GOLD["epilogue"]["gelu_constants"]
            inner = c["sqrt_2_over_pi"] * (expected + c["cubic"] * expected * expected * expected)
            expected = 0.5 * expected * (1 + np.tanh(inner))
            got = O.unary("gelu", got)
        elif op == "silu":
            expected = expected / (1 + np.exp(-expected))
            got = O.unary("silu", got)
    bound = case["atol"] + case["rtol"] * np.abs(expected)
    assert np.all(np.abs(got.astype(np.float64) - expected) <= bound)
    # and far tighter than the spec's bound: only f32 storage error
    assert np.all(np.abs(got.astype(np.float64) - expected) <= 4e-6 * np.maximum(1.0, np.abs(expected)))


def test_unary_known_points_and_identities():
    u = lambda op, x: O.lib().ref_unary_scalar(O.UNARY[op], float(x))
    assert u("relu", -1.5) == 0.0 and u("relu", 2.5) == 2.5 and u("relu", 0.0) == 0.0
    assert u("silu", 0.0) == 0.0 and u("sigmoid", 0.0) == 0.5
    assert u("gelu", 0.0) == 0.0 and u("gelu_erf", 0.0) == 0.0
    for x in (-4.0, -1.0, -0.3, 0.7, 2.0, 5.0):
        # silu(x) = x * sigmoid(x);  silu(x) - silu(-x) = x
        assert abs(u("silu", x) - x * u("sigmoid", x)) <= 1e-15 * max(1, abs(x))
        assert abs(u("silu", x) - u("silu", -x) - x) <= 1e-15 * max(1, abs(x))
        # gelu(x) - gelu(-x) = x for both forms (odd inner function)
        assert abs(u("gelu", x) - u("gelu", -x) - x) <= 1e-15 * max(1, abs(x))
        assert abs(u("gelu_erf", x) - u("gelu_erf", -x) - x) <= 1e-15 * max(1, abs(x))
        # A-S 7.1.26 is within 1.5e-7 of erf
        exact = 0.5 * x * (1 + math.erf(x / math.sqrt(2)))
        assert abs(u("gelu_erf", x) - exact) <= 2e-7 * max(1, abs(x))
        # tanh form stays within 1e-3 of the exact GELU (a different function, loosely)
        assert abs(u("gelu", x) - exact) <= 1e-3
    assert abs(u("gelu", 1.0) - 0.8411919906082768) < 1e-12  # 0.5*(1+tanh(0.7978845608*1.044715))
    assert u("gelu", 1.0) == 0.5 * (1 + math.tanh(0.7978845608 * (1.0 + 0.044715)))
    assert u("silu", 1.0) == 1.0 / (1.0 + math.exp(-1.0))


def test_unary_c_vs_numpy():
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(100000) * 4).astype(np.float32)
    for op in ("relu", "silu", "gelu", "sigmoid", "tanh"):
        a, b = O.unary(op, x), O.np_unary(op, x)
        # libm vs numpy exp/tanh may differ in the last double bit -> rarely 1 f32 ulp.
        # gelu's 1 + tanh(.) cancels for x << 0, where that last bit is all that is
        # left (values ~1e-16): compare those absolutely.
        ulps = np.abs(a.view(np.int32).astype(np.int64) - b.view(np.int32).astype(np.int64))
        close_abs = np.abs(a.astype(np.float64) - b.astype(np.float64)) <= 1e-14
        assert np.all((ulps <= 1) | close_abs)
        assert np.mean((a != b) & ~close_abs) < 1e-3


def test_linear_is_three_f32_ops():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 64)).astype(np.float32)
    w = rng.standard_normal((8, 64)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    y = O.linear(x, w, b, "silu")
    step1 = O.matmul_nt(x, w)
    step2 = (step1.astype(np.float64) + b.astype(np.float64)[None, :]).astype(np.float32)
    step3 = O.np_unary("silu", step2)
    assert np.max(np.abs(y.view(np.int32).astype(np.int64) - step3.view(np.int32).astype(np.int64))) <= 1


def test_lcg_matches_probe_recurrence():
    draw = O.make_lcg(0x51A7EE)
    v = np.concatenate([draw(3), draw(70000), draw(5)])
    s = 0x51A7EE
    for i in (0, 1, 2):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        assert v[i] == s / 2 ** 31 - 1
    s = 0x51A7EE
    for i in range(len(v)):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
    assert v[-1] == s / 2 ** 31 - 1
    assert -1.0 <= v.min() and v.max() < 1.0
