"""GPU parity: device top-k (the LM-head consumer, src/backend/webgpu/topk-kernel.ts)
against a numpy sort by (value descending, index ascending) -- exact."""
import ctypes as C

import numpy as np
import pytest

import torchlette_amd as T
from torchlette_amd import _lib as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def reference_topk(v, k):
    """first-maximum linear scan, k rounds == stable sort by (-value, index); NaN last"""
    key = np.where(np.isnan(v), -np.inf, v).astype(np.float64)
    nan = np.isnan(v)
    order = np.lexsort((np.arange(v.size), nan, -key))
    idx = order[:k].astype(np.int32)
    vals = v[idx].astype(np.float32)
    if idx.size < k:
        vals = np.concatenate([vals, np.full(k - idx.size, -3.4028234e38, np.float32)])
        idx = np.concatenate([idx, np.full(k - idx.size, -1, np.int32)])
    return vals, idx


@pytest.mark.parametrize("n", [1, 5, 64, 4095, 4096, 4097, 151936, 256000, 262145, 700001])
@pytest.mark.parametrize("k", [1, 8, 64])
def test_topk_matches_a_stable_sort(be, n, k):
    rng = np.random.default_rng(n * 7 + k)
    v = rng.standard_normal(n).astype(np.float32)
    t = be.ops.tensorFromArray(v, [n], "f32")
    vals, idx = be.readTopK(t, k)
    want_v, want_i = reference_topk(v, k)
    assert np.array_equal(idx, want_i)
    assert np.array_equal(vals.view(np.uint32), want_v.view(np.uint32))


def test_topk_ties_signs_infinities_nan(be):
    rng = np.random.default_rng(3)
    n = 20000
    v = rng.integers(-3, 4, n).astype(np.float32)          # many ties: the smaller index must win
    v[100] = np.inf
    v[7000] = np.inf
    v[5] = -np.inf
    v[17] = np.nan
    v[18] = -0.0
    v[19] = 0.0
    t = be.ops.tensorFromArray(v, [n], "f32")
    for k in (1, 2, 3, 64, 200):
        vals, idx = be.readTopK(t, k)
        want_v, want_i = reference_topk(v, k)
        assert np.array_equal(idx, want_i), k
        assert np.array_equal(vals, want_v), k
    # all NaN but two: the numbers come first, then NaN by index
    w = np.full(50, np.nan, np.float32)
    w[30] = -5.0
    w[40] = -7.0
    vals, idx = be.readTopK(be.ops.tensorFromArray(w, [50], "f32"), 4)
    assert list(idx) == [30, 40, 0, 1] and vals[0] == -5.0 and vals[1] == -7.0 and np.isnan(vals[2:]).all()


def test_topk_window_and_packed_form(be):
    rng = np.random.default_rng(9)
    v = rng.standard_normal(3 * 50000).astype(np.float32)
    t = be.ops.tensorFromArray(v, [3, 50000], "f32")
    vals, idx = be.readTopK(t, 16, offset=50000, length=50000)   # the middle row
    want_v, want_i = reference_topk(v[50000:100000], 16)
    assert np.array_equal(idx, want_i) and np.array_equal(vals, want_v)
    row = be.ops.tensorFromArray(v[:50000], [1, 1, 50000], "f32")
    packed = be.deviceTopK(row, 64).numpy()
    want_v, want_i = reference_topk(v[:50000], 64)
    assert packed.shape == (1, 2, 64)
    assert np.array_equal(packed[0, 0], want_v) and np.array_equal(packed[0, 1], want_i.astype(np.float32))


def test_topk_after_the_lm_head_gemv(be):
    """argmax of the logits the packed LM head produces == argmax of the oracle's logits
    when the margin is above the GEMV tolerance (greedy decoding reads 2 numbers back)."""
    from oracle import quant_oracle as O
    from helpers import make_weight, make_x
    rng = np.random.default_rng(21)
    n, k = 8192, 512
    packed, scales, deq = make_weight("int8-row", n, k, 0, rng)
    x = make_x(1, k, "f16", rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int8-row", "f32"))
    y = be.linear(be.ops.tensorFromArray(x, [1, k], "f16"), w)
    vals, idx = be.readTopK(y, 8)
    want = O.linear(x.astype(np.float32), deq)[0]
    order = np.argsort(-want, kind="stable")
    assert idx[0] == order[0] or abs(want[order[0]] - want[order[1]]) < 1e-3 * abs(want[order[0]])
    assert np.allclose(vals, np.sort(want)[::-1][:8], rtol=1e-4, atol=1e-5)


def test_topk_errors(be):
    t = be.ops.tensorFromArray(np.zeros(10, np.float32), [10], "f32")
    with pytest.raises(L.TlhipError, match="k="):
        be.readTopK(t, 0)
    with pytest.raises(ValueError, match="range"):
        be.readTopK(t, 2, offset=8, length=5)
