"""GPU parity of the per-wave pipelined skinny GEMV (configuration variant 5, int4 weights
in groups of 32, f16 activations, 1..16 rows) against the oracle.

f32 output: the products are exact and accumulate in f32, so only the order of the sums
differs from the oracle (rel-L2 <= 2e-6 asserted); f16 output: the stated bar, 1e-3."""
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def run(be, packed, scales, n, k, x, element, cfg, bias=None, act=None):
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", element))
    xt = be.ops.tensorFromArray(x, list(x.shape), "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f32") if bias is not None else None
    y = be.linear(xt, w, bt, act, fused=True, config=L.KernelConfig.of(*cfg))
    out = y.numpy()
    y.destroy()
    xt.destroy()
    return out


# (n, k): ragged row blocks, K that the waves do not divide, several passes (n / 16 row
# blocks over 256 workgroups x 3 blocks per pass), a single row block
SHAPES = [(2048, 1024), (1000, 2048), (4096, 4096), (12288, 1024), (13000, 640), (16, 128), (24, 3200), (16000, 256), (520, 768), (4096, 11008)]


@pytest.mark.parametrize("cfg", [(5, 8, 2, 1), (5, 8, 4, 1), (5, 4, 3, 2), (5, 8, 2, 1, 2), (5, 4, 2, 2, 2), (5, 8, 2, 1, 2, 0, 1), (5, 4, 3, 2, 2, 0, 1)])
@pytest.mark.parametrize("m", [1, 3, 4, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k", SHAPES)
def test_wave_gemv_matches_oracle(be, n, k, m, cfg):
    rng = np.random.default_rng(zlib.crc32(repr((n, k, m, cfg)).encode()))
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    if len(cfg) > 4 and cfg[4] == 2 and k % 256:
        pytest.skip("two iterations per step take K in multiples of 256")
    before = T.getQuantGemvDispatchCount()
    try:
        got = run(be, packed, scales, n, k, x, "f32", cfg, bias=bias, act="silu")
    except L.TlhipError as e:
        if "more registers than a lane has" in str(e):
            pytest.skip("no instance: this depth does not fit the register file for these rows and row blocks")
        if "more than 4 row blocks" in str(e) and n > 256 * cfg[3] * 64:
            pytest.skip("more rows than one pass over the chip covers")
        raise
    assert T.getQuantGemvDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    assert got.shape == (m, n) and got.dtype == np.float32
    assert rel_l2(got, want) <= 2e-6, rel_l2(got, want)
    again = run(be, packed, scales, n, k, x, "f32", cfg, bias=bias, act="silu")
    assert np.array_equal(got, again)  # the sums are formed in a fixed order
    got16 = run(be, packed, scales, n, k, x, "f16", cfg)
    assert got16.dtype == np.float16
    assert rel_l2(got16, O.linear(x.astype(np.float32), deq, threads=8)) <= 1e-3


def test_wave_gemv_refuses_what_it_is_not_built_for(be):
    rng = np.random.default_rng(3)
    packed, scales, _ = make_weight("int4-grouped", 256, 1024, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 256, 1024, T.resolveWeightFormat("int4-32", "f32"))
    x17 = be.ops.tensorFromArray(make_x(17, 1024, "f16", rng), [17, 1024], "f16")
    with pytest.raises(L.TlhipError, match="M must be 1..16"):
        be.linear(x17, w, config=L.KernelConfig.of(5, 8, 2, 1))
    x = be.ops.tensorFromArray(make_x(4, 1024, "f16", rng), [4, 1024], "f16")
    with pytest.raises(L.TlhipError, match="steps in flight"):
        be.linear(x, w, config=L.KernelConfig.of(5, 8, 7, 1))
    p8, s8, _ = make_weight("int8-row", 256, 1024, 0, rng)
    w8 = be.createQuantizedWeight(p8, s8, 256, 1024, T.resolveWeightFormat("int8-row", "f32"))
    with pytest.raises(L.TlhipError, match="int4 weights with group size 32"):
        be.linear(x, w8, config=L.KernelConfig.of(5, 8, 2, 1))
