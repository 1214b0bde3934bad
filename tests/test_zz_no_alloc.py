"""GPU parity of tlhip_gemv_noalloc, the decode GEMV that allocates nothing.

It runs the same kernels as tlhip_gemv with the K-slice workspace in a fixed
device array of the library.  Checked through the C ABI: bit-identical to
tlhip_gemv (same configuration, and the slices are summed in slice order
whoever arrives last) and within the stated rel-L2 bar of the oracle, on two
calls in a row that share the array, the second smaller than the first."""
import ctypes as C
import os

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
REL_L2_TOL = 1e-3


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def _case(be, n, k, m, seed, act):
    rng = np.random.default_rng(seed)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    want = O.linear(x.astype(np.float32), deq, bias, act, threads=8)
    return w, xt, bt, want


def _run(be, entry, w, xt, bt, act, m, n):
    out = be._alloc([m, n], "f32")
    L.call("tlhip_memset", out.ptr, 0xFF, out.nbytes, None)  # a NaN pattern: every element must be written
    ep = be.makeEpilogue(bt, act)
    qw = be._qweight(w, False)
    L.call(entry, C.byref(qw), xt.ptr, L.F16, m, out.ptr, L.F32, 1.0, C.byref(ep), None)
    got = out.numpy()
    out.destroy()
    return got


def test_noalloc_matches_gemv_on_two_calls_sharing_the_scratch(be):
    # both shapes are too long for one workgroup's LDS at their M, so the selected
    # configurations slice K across workgroups and go through the scratch
    first = (2048, 12288, 16, 11, "silu")
    second = (528, 12288, 8, 12, "gelu")  # smaller, ragged N: stale tiles and counters of the first call lie behind it
    cases = [(_case(be, *c), c) for c in (first, second)]
    for (w, xt, bt, want), (n, k, m, _, act) in cases:
        cfg = be.selectedConfig(w, "f16", m, "f32")
        assert cfg.variant in (L.VARIANT_GEMV_MFMA, L.VARIANT_GEMV_XREG) and cfg.p3 > 1, cfg.as_tuple()
    results = []
    for (w, xt, bt, want), (n, k, m, _, act) in cases:  # the two no-alloc calls in a row
        results.append(_run(be, "tlhip_gemv_noalloc", w, xt, bt, act, m, n))
    for got, ((w, xt, bt, want), (n, k, m, _, act)) in zip(results, cases):
        ref = _run(be, "tlhip_gemv", w, xt, bt, act, m, n)
        assert not np.isnan(got).any()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (n, k, m)
        assert rel_l2(got, want) <= REL_L2_TOL
        assert rel_l2(got, want) <= 2e-5
    # and once more in the other order: the counters are cleared per call
    (w, xt, bt, want), (n, k, m, _, act) = cases[0]
    again = _run(be, "tlhip_gemv_noalloc", w, xt, bt, act, m, n)
    assert np.array_equal(again.view(np.uint32), results[0].view(np.uint32))


def test_noalloc_without_k_slices_and_m1(be):
    # a configuration that needs no scratch goes straight through
    w, xt, bt, want = _case(be, 1024, 2048, 1, 13, "relu")
    got = _run(be, "tlhip_gemv_noalloc", w, xt, bt, "relu", 1, 1024)
    ref = _run(be, "tlhip_gemv", w, xt, bt, "relu", 1, 1024)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert rel_l2(got, want) <= 2e-5


@pytest.mark.parametrize("n,k,m", [(640, 28672, 12), (520, 4000 * 4, 9), (1000, 11008, 16), (256, 20480, 13), (300, 8192, 10)])
def test_noalloc_takes_the_route_gemv_takes(be, n, k, m):
    """9..16 rows on shapes where the default is not one launch of the matrix-core kernel
    (K too long for LDS at these rows, K slices of unequal length, the VALU kernel with the
    rows in chunks of 8 on the matrix cores): both entry points select and route alike, so
    the results are the same bits whatever the route is."""
    w, xt, bt, want = _case(be, n, k, m, 100 + m, "silu")
    got = _run(be, "tlhip_gemv_noalloc", w, xt, bt, "silu", m, n)
    ref = _run(be, "tlhip_gemv", w, xt, bt, "silu", m, n)
    assert not np.isnan(got).any()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert rel_l2(got, want) <= 2e-5
    again = _run(be, "tlhip_gemv_noalloc", w, xt, bt, "silu", m, n)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))


def test_noalloc_rejects_more_scratch_than_it_holds(be):
    # 8192 rows x 16 K slices x 1 KiB of partial tiles = 8 MiB, above the fixed 4 MiB
    n, k, m = 8192, 4096, 16
    rng = np.random.default_rng(5)
    packed = rng.integers(0, 2 ** 32, n * k // 8, dtype=np.uint64).astype(np.uint32)
    scales = np.full(n * k // 32, 0x2000, np.uint16)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    be.seedPerShapeMatmulChoice(w, "f16", m, "f32", L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 1, 1, 16))
    try:
        assert be.selectedConfig(w, "f16", m, "f32").p3 == 16
        xt = be.ops.tensorFromArray(make_x(m, k, "f16", rng), [m, k], "f16")
        out = be._alloc([m, n], "f32")
        qw = be._qweight(w, False)
        rc = L.load().tlhip_gemv_noalloc(C.byref(qw), xt.ptr, L.F16, m, out.ptr, L.F32, 1.0, None, None)
        assert rc == L.ERR_INVALID
        assert "fixed scratch holds" in L.last_error()
        # the allocating entry point serves the same problem
        L.call("tlhip_gemv", C.byref(qw), xt.ptr, L.F16, m, out.ptr, L.F32, 1.0, None, None)
        be.synchronize()
    finally:
        # the seed made an entry of this exact problem: drop it with the whole cache and
        # bring the shipped tuning file back, so that later tests select as a fresh process does
        T.clearTuningCache()
        tuning = os.path.join(os.path.dirname(T.__file__), "tuning", "mi355x.json")
        T.importTuningCache(open(tuning).read())
