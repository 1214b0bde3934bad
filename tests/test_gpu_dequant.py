"""GPU parity: the HIP dequant kernel is bit-exact against the oracle
(quantize.ts:138-156 for int8-grouped; f32(q*s) for the other two formats)."""
import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from helpers import make_weight, fmt_name

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def assert_bits_equal(got, want):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape
    gn, wn = np.isnan(got), np.isnan(want)
    assert np.array_equal(gn, wn)
    assert np.array_equal(got[~gn].view(np.uint32), want[~wn].view(np.uint32))


def gpu_dequant(be, fmt, packed, scales, n, k, g, element="f16"):
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element))
    before = T.getDequantI8DispatchCount()
    out = be.dequantizeToF32(w)
    res = out.numpy()
    if n and k:
        assert T.getDequantI8DispatchCount() == before + 1
    out.destroy()
    return res


def test_int8_grouped_full_table(be):
    """Every (byte, f16 scale) pair: 256 x 65536, -128 and inf/NaN scales included."""
    n, k, g = 65536, 256, 256
    q = np.tile(np.arange(256, dtype=np.uint8).view(np.int8), (n, 1))
    packed = O.np_pack_int8(q)
    scales = np.arange(65536, dtype=np.uint16)
    want = O.dequant_int8_grouped(packed, scales, n, k, g)
    assert_bits_equal(gpu_dequant(be, "int8-grouped", packed, scales, n, k, g), want)


def test_int4_grouped_full_table(be):
    n, k, g = 65536, 32, 32
    q = np.tile(np.concatenate([np.arange(-8, 8), np.arange(7, -9, -1)]).astype(np.int8), (n, 1))
    packed = O.np_pack_int4(q)
    scales = np.arange(65536, dtype=np.uint16)
    want = O.dequant_int4_grouped(packed, scales, n, k, g)
    assert_bits_equal(gpu_dequant(be, "int4-grouped", packed, scales, n, k, g), want)


def test_int8_row_all_bytes_times_sampled_scales(be):
    rng = np.random.default_rng(5)
    n, k = 8192, 256
    q = np.tile(np.arange(256, dtype=np.uint8).view(np.int8), (n, 1))
    packed = O.np_pack_int8(q)
    scales = rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32).copy()
    scales[:4] = [0.0, -0.0, np.float32(1e-42), np.float32(3e38)]
    want = O.dequant_int8_row(packed, scales, n, k)
    assert_bits_equal(gpu_dequant(be, "int8-row", packed, scales, n, k, 0), want)


@pytest.mark.parametrize("fmt,n,k,g", [
    ("int8-grouped", 512, 1024, 64), ("int8-grouped", 1024, 2048, 128), ("int8-grouped", 130, 192, 64),
    ("int8-row", 1024, 1024, 0), ("int8-row", 1000, 2304, 0),
    ("int4-grouped", 2048, 1024, 32), ("int4-grouped", 1024, 3072, 32), ("int4-grouped", 4096, 4096, 32),
    ("int4-grouped", 100, 12288, 32), ("int4-grouped", 64, 256, 64), ("int4-grouped", 33, 128, 128),
])
def test_config_shaped_tensors(be, fmt, n, k, g):
    rng = np.random.default_rng(n + k)
    packed, scales, want = make_weight(fmt, n, k, g, rng)
    assert_bits_equal(gpu_dequant(be, fmt, packed, scales, n, k, g), want)


@pytest.mark.parametrize("fmt,n,k,g", [
    ("int8-grouped", 7, 8, 4), ("int8-grouped", 5, 24, 8), ("int8-row", 3, 4, 0), ("int8-row", 9, 20, 0),
    ("int4-grouped", 5, 8, 8), ("int4-grouped", 4, 48, 16), ("int4-grouped", 3, 16, 4),
])
def test_rows_that_are_not_whole_16_byte_chunks(be, fmt, n, k, g):
    rng = np.random.default_rng(n * 31 + k)
    if fmt == "int8-grouped":
        q = rng.integers(-128, 128, (n, k)).astype(np.int8)
        packed = O.np_pack_int8(q)
        scales = rng.integers(0, 0x7C00, n * k // g).astype(np.uint16)
    elif fmt == "int8-row":
        q = rng.integers(-128, 128, (n, k)).astype(np.int8)
        packed = O.np_pack_int8(q)
        scales = rng.uniform(0.001, 1, n).astype(np.float32)
    else:
        q = rng.integers(-8, 8, (n, k)).astype(np.int8)
        packed = O.np_pack_int4(q)
        scales = rng.integers(0, 0x7C00, n * k // g).astype(np.uint16)
    want = O.dequant(fmt, packed, scales, n, k, g)
    assert_bits_equal(gpu_dequant(be, fmt, packed, scales, n, k, g), want)


def test_empty_weight(be):
    out = gpu_dequant(be, "int4-grouped", np.zeros(0, np.uint32), np.zeros(0, np.uint16), 0, 64, 32)
    assert out.shape == (0, 64)


def test_dequant_of_native_quantizer_output_round_trips(be):
    """quantize (native host) -> upload -> dequant (GPU) == oracle dequant of oracle quantize."""
    rng = np.random.default_rng(77)
    n, k, g = 256, 1024, 64
    w = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    packed, scales = T.quantizeLinearWeight(w, n, k, g)
    want = O.dequant_int8_grouped(*O.quantize_int8_grouped(w, n, k, g), n, k, g)
    assert_bits_equal(gpu_dequant(be, "int8-grouped", packed, scales, n, k, g), want)
