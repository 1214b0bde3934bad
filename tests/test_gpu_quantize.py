"""GPU parity: the device quantizer (quantizeLinearWeight of
src/backend/quantize.ts:77-131 for weights already in HBM) against the oracle,
bit for bit, including the ties of Math.round, the round-half-up subnormal
scales of f32ToF16Bits, zero groups, NaN and infinities."""
import ctypes as C

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def device_quantize(be, w, g):
    n, k = w.shape
    wt = be.ops.tensorFromArray(w, [n, k], "f32")
    q = be.quantizeLinearWeightOnDevice(wt, g)
    packed = np.empty(n * k // 4, np.uint32)
    scales = np.empty(n * (k // g), np.uint16)
    L.call("tlhip_memcpy_d2h", packed.ctypes.data, q.ptr, packed.nbytes, None)
    L.call("tlhip_memcpy_d2h", scales.ctypes.data, q.scales.ptr, scales.nbytes, None)
    be.synchronize()
    return q, packed, scales


@pytest.mark.parametrize("n,k,g", [(7, 64, 64), (33, 256, 64), (128, 1024, 128), (5, 96, 32), (3, 4096, 64),
                                   (600, 512, 4), (2, 12, 12)])
def test_device_quantizer_matches_the_oracle_bit_for_bit(be, n, k, g):
    rng = np.random.default_rng(n * 131 + k + g)
    w = (rng.standard_normal((n, k)) * rng.uniform(1e-3, 3.0, (n, 1))).astype(np.float32)
    _, packed, scales = device_quantize(be, w, g)
    want_packed, want_scales = O.quantize_int8_grouped(w.ravel(), n, k, g)
    assert np.array_equal(scales, want_scales)
    assert np.array_equal(packed, want_packed)


def test_device_quantizer_edge_values(be):
    n, k, g = 8, 64, 16
    w = np.zeros((n, k), np.float32)
    rng = np.random.default_rng(11)
    # row 0: exact half-integer products of both signs (scale 127/127 = 1 -> inv = 127/amax)
    w[0, :16] = np.array([127, 2.5, -2.5, 0.5, -0.5, 1.5, -1.5, 126.5, -126.5, 3, -3, 0, 63.5, -63.5, 100, -100],
                         np.float32)
    # row 1: a zero group next to a non-zero one
    w[1, 16:32] = rng.standard_normal(16)
    # row 2: NaN and infinities
    w[2, :16] = rng.standard_normal(16)
    w[2, 3] = np.nan
    w[2, 20] = np.inf
    w[2, 21] = -np.inf
    w[2, 22] = 1.0
    # row 3: group maximum in the f16 subnormal range, on a rounding tie (round-half-up there)
    w[3, :16] = np.float32(2.0 ** -24 * 1.5) * np.linspace(-1, 1, 16, dtype=np.float32)
    w[3, 5] = np.float32(2.0 ** -24 * 1.5)
    # row 4: maximum above the f16 range -> infinite scale, everything quantizes to 0
    w[4, :16] = np.float32(1e6) * rng.standard_normal(16).astype(np.float32)
    # row 5: all NaN group
    w[5, :16] = np.nan
    # rows 6, 7: ordinary
    w[6:] = rng.standard_normal((2, k)).astype(np.float32) * 0.02
    _, packed, scales = device_quantize(be, w, g)
    want_packed, want_scales = O.quantize_int8_grouped(w.ravel(), n, k, g)
    assert np.array_equal(scales, want_scales)
    assert np.array_equal(packed, want_packed)


def test_quantized_on_device_weight_runs_through_the_matmul_seam(be):
    rng = np.random.default_rng(5)
    n, k, g = 256, 512, 64
    w = rng.standard_normal((n, k)).astype(np.float32) * 0.05
    q, packed, scales = device_quantize(be, w, g)
    deq = be.dequantizeToF32(q).numpy()
    assert np.array_equal(deq.view(np.uint32), O.dequant_int8_grouped(packed, scales, n, k, g).view(np.uint32))
    x = rng.standard_normal((1, k)).astype(np.float32)
    xt = be.ops.tensorFromArray(x, [1, k], "f32")
    y = be.ops.matmul(xt, be.ops.transpose(q)).numpy()
    want = O.linear(x, deq)
    assert np.linalg.norm(y - want) / np.linalg.norm(want) <= 1e-5


def test_device_quantizer_errors(be):
    wt = be.ops.tensorFromArray(np.zeros((2, 6), np.float32), [2, 6], "f32")
    with pytest.raises(ValueError, match="divisible by 4"):
        be.quantizeLinearWeightOnDevice(wt, 6)
    wt2 = be.ops.tensorFromArray(np.zeros((2, 16), np.float32), [2, 16], "f32")
    with pytest.raises(ValueError, match="divisible by groupSize"):
        be.quantizeLinearWeightOnDevice(wt2, 12)
    p = C.c_void_p(16)
    with pytest.raises(L.TlhipError, match="multiple of 4"):
        L.call("tlhip_quantize_int8_grouped_device", p, 2, 12, 6, p, p, None)


@pytest.mark.parametrize("on_device", [False, True])
def test_loader_branch_quantizes_once_and_then_hits_the_cache(be, tmp_path, on_device):
    """browser-loader.ts:654-699: miss -> fetch f32, quantize, store; hit -> the tensor's
    bytes are never fetched.  Either way the weight equals the oracle's bit for bit."""
    n, k, g = 48, 512, 64
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((n, k)) * 0.2).astype(np.float32)
    cache = T.PackedWeightCache(str(tmp_path / "packed"))
    fetched = []

    def fetch():
        fetched.append(1)
        return w

    want_packed, want_scales = O.quantize_int8_grouped(w.ravel(), n, k, g)
    want = O.dequant_int8_grouped(want_packed, want_scales, n, k, g)
    url, name = "https://host/model.safetensors", "model.layers.0.self_attn.q_proj.weight"
    for expect_fetches in (1, 1):
        q = T.loadQuantizedWeight(be, cache, url, name, n, k, "int8-64", fetch, "f32", onDevice=on_device)
        assert len(fetched) == expect_fetches
        got = be.dequantizeToF32(q).numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    rec = cache.getCachedPacked(T.packedKey(url, name, "int8-grouped", g))
    assert np.array_equal(rec["packed"], want_packed.ravel()) and np.array_equal(rec["scales"], want_scales.ravel())
    # another group size is another key: quantized again
    T.loadQuantizedWeight(be, cache, url, name, n, k, "int8-128", fetch, "f32", onDevice=on_device)
    assert len(fetched) == 2
    # no cache at all still works
    T.loadQuantizedWeight(be, None, url, name, n, k, "int8-64", fetch, "f32", onDevice=on_device)
    assert len(fetched) == 3
