"""GPU parity: decode GEMV / skinny GEMM over packed weights vs the oracle
(bit-exact dequant -> CPU-backend matmul -> add -> activation).

Tolerance: rel-L2 <= 1e-3 (the stated bar), and for the reference's own format
the probe's bar max |d|/max(1,|ref|) <= 5e-4 (probe-quant-gemv.ts:182-187)."""
import json
import os
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import f16_round, fmt_name, make_weight, make_x, per_row_err, rel_l2

pytestmark = pytest.mark.gpu
REL_L2_TOL = 1e-3
PROBE_TOL = 5e-4
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def run_linear(be, fmt, packed, scales, n, k, g, x, element, bias=None, act=None, fused=False, config=None):
    xdt = "f16" if x.dtype == np.float16 else "f32"
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element))
    xt = be.ops.tensorFromArray(x, list(x.shape), xdt)
    bt = None
    if bias is not None:
        bt = be.ops.tensorFromArray(bias, [n], "f16" if bias.dtype == np.float16 else "f32")
    y = be.linear(xt, w, bt, act, fused=fused, config=config)
    out = y.numpy()
    y.destroy()
    xt.destroy()
    return out


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("fmt,n,k,g,xdt,element", [
    ("int4-grouped", 2048, 1024, 32, "f16", "f16"),
    ("int4-grouped", 1024, 3072, 32, "f16", "f16"),
    ("int8-row", 1024, 1024, 0, "f32", "f32"),
    ("int8-row", 1536, 2304, 0, "f16", "f32"),
    ("int8-grouped", 512, 1024, 64, "f32", "f32"),
    ("int8-grouped", 768, 2048, 128, "f16", "f16"),
])
def test_gemv_matches_oracle(be, fmt, n, k, g, xdt, element, m):
    rng = np.random.default_rng(zlib.crc32(repr((fmt, n, k, m)).encode()))
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, xdt, rng)
    before = T.getQuantGemvDispatchCount()
    got = run_linear(be, fmt, packed, scales, n, k, g, x, element)
    assert T.getQuantGemvDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq)
    assert got.shape == (m, n)
    assert got.dtype == (np.float16 if (xdt == "f16" and element == "f16") else np.float32)
    tol = REL_L2_TOL
    assert rel_l2(got, want) <= tol, rel_l2(got, want)
    if got.dtype == np.float32:
        assert rel_l2(got, want) <= 2e-6  # f32 accumulate of exact products: order noise only


@pytest.mark.parametrize("m", [17, 24, 32, 33, 48, 64])
@pytest.mark.parametrize("fmt,g,n,k,cfg", [
    ("int4-grouped", 32, 1000, 2048, (1, 8, 2, 8, 1)),            # K split over the waves of a workgroup
    ("int4-grouped", 32, 1536, 2048, (1, 8, 2, 4, 2, 0, 1)),      # ... and over two workgroups, whole-line loads
    ("int4-grouped", 128, 520, 1024, (1, 4, 1, 1, 1)),            # a wave owns its row blocks
    ("int4-grouped", 32, 2048, 4096, (1, 8, 1, 2, 4)),            # four K slices
    ("int8-row", 0, 1000, 2304, (1, 8, 2, 1, 2, 0, 1)),
    ("int8-grouped", 64, 768, 2048, (1, 4, 2, 4, 2)),
])
def test_seventeen_to_64_rows_in_one_launch_of_the_matrix_core_gemv(be, fmt, g, n, k, cfg, m):
    """Two or four tiles of 16 activation rows per weight row block: the weights stream once
    for all rows.  Against the oracle (f32 out: exact products, order noise only), and
    bit-identical to the same configuration run on the first 16 rows alone wherever the
    launch geometry does not enter the arithmetic (every row's sum is formed in the same
    order whatever the number of tiles)."""
    rng = np.random.default_rng(zlib.crc32(repr((fmt, n, k, m, cfg)).encode()))
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    c = L.KernelConfig.of(*cfg)
    before = T.getQuantGemvDispatchCount()
    try:
        got = run_linear(be, fmt, packed, scales, n, k, g, x, "f32", bias=bias, act="silu", fused=True, config=c)
    except L.TlhipError as e:
        if "do not fit LDS" in str(e) and m > 32:
            pytest.skip("four tiles of rows: this geometry's activations and parked tiles exceed LDS")
        raise
    assert T.getQuantGemvDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    assert got.shape == (m, n)
    assert rel_l2(got, want) <= 2e-6, rel_l2(got, want)
    first = run_linear(be, fmt, packed, scales, n, k, g, x[:16].copy(), "f32", bias=bias, act="silu", fused=True, config=c)
    assert np.array_equal(got[:16], first)
    got16 = run_linear(be, fmt, packed, scales, n, k, g, x, "f16", config=c)
    assert got16.dtype == np.float16
    assert rel_l2(got16, O.linear(x.astype(np.float32), deq, threads=8)) <= REL_L2_TOL


def test_more_than_16_rows_reject_what_the_matrix_core_gemv_does_not_cover(be):
    rng = np.random.default_rng(5)
    packed, scales, _ = make_weight("int4-grouped", 256, 1024, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 256, 1024, T.resolveWeightFormat("int4-32", "f32"))
    x = be.ops.tensorFromArray(make_x(40, 1024, "f16", rng), [40, 1024], "f16")
    with pytest.raises(L.TlhipError, match="at most 8 waves"):
        be.linear(x, w, config=L.KernelConfig.of(1, 16, 1, 16, 1))
    with pytest.raises(L.TlhipError, match="1 or 2 above 32 rows"):
        be.linear(x, w, config=L.KernelConfig.of(1, 8, 4, 8, 1))
    x65 = be.ops.tensorFromArray(make_x(65, 1024, "f16", rng), [65, 1024], "f16")
    with pytest.raises(L.TlhipError, match="M must be"):
        be.linear(x65, w, config=L.KernelConfig.of(1, 8, 1, 8, 1))


@pytest.mark.parametrize("m", [5, 9, 15, 16, 40])
@pytest.mark.parametrize("k", [11008, 13696])
def test_k_whose_steps_do_not_divide_over_the_slices(be, m, k):
    """K = 11008 is 86 steps of 128 and K = 13696 is 107: two equal slices of 16 rows do not
    fit LDS and four do not divide the steps.  The matrix-core kernel then takes slices of
    unequal length (22, 22, 21, 21), one launch, instead of falling to the VALU kernel's
    pass per four rows.  Heuristic defaults; against the oracle, and every explicit
    configuration with unequal slices gives the same bits from launch to launch."""
    n = 768
    rng = np.random.default_rng(k + m)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    saved = T.exportTuningCache()
    T.clearTuningCache()
    try:
        before = T.getQuantGemvDispatchCount()
        got = run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32")
        launches = T.getQuantGemvDispatchCount() - before
    finally:
        T.importTuningCache(saved)
    assert launches == 1, launches
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert rel_l2(got, want) <= 2e-6, rel_l2(got, want)
    if m <= 16:
        for cfg in ((1, 8, 1, 8, 4), (1, 8, 1, 2, 8), (1, 4, 1, 1, 16)):
            a = run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=L.KernelConfig.of(*cfg))
            b = run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=L.KernelConfig.of(*cfg))
            assert rel_l2(a, want) <= 2e-6 and np.array_equal(a, b), cfg
        with pytest.raises(L.TlhipError, match="slices of unequal length"):
            run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=L.KernelConfig.of(1, 8, 2, 8, 4))


@pytest.mark.parametrize("fmt,n,k,g", [
    ("int4-grouped", 4096, 4096, 32), ("int4-grouped", 12288, 4096, 32), ("int4-grouped", 4096, 12288, 32),
])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_qwen3_8b_shapes(be, fmt, n, k, g, m):
    rng = np.random.default_rng(n + k + m)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    got = run_linear(be, fmt, packed, scales, n, k, g, x, "f16")
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert rel_l2(got, want) <= REL_L2_TOL
    # f16 output rounding only: within one f16 ulp of the oracle
    assert per_row_err(got, want) <= 2e-3


def test_every_candidate_config_gives_the_same_answer(be):
    rng = np.random.default_rng(42)
    n, k, g, m = 777, 2048, 32, 3   # ragged N: every tail path is exercised
    packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    want = O.linear(x.astype(np.float32), deq)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    cands = be.candidates(w, "f16", m, "f32")
    assert len(cands) >= 20
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    for c in cands:
        y = be.linear(xt, w, config=c)
        got = y.numpy()
        y.destroy()
        assert rel_l2(got, want) <= 2e-6, c.as_tuple()


@pytest.mark.parametrize("fmt,n,k,g", [
    ("int4-grouped", 4096, 12288, 32), ("int4-grouped", 1000, 4096, 64),
    ("int8-grouped", 520, 4096, 128), ("int8-row", 1031, 2304, 0),
])
@pytest.mark.parametrize("m", [5, 8, 13, 16])
def test_matrix_core_kernel_with_k_slices_across_workgroups(be, fmt, n, k, g, m):
    """Slices of K on different workgroups, combined by the last arriver: same
    answer for every slice count, bit-identical on repeated launches (the sum
    runs in slice order whoever arrives last), counters back at zero each time."""
    rng = np.random.default_rng(n + k + m)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    ran = 0
    for ks in (2, 4, 8, 16):
        for waves, unroll, kw in ((8, 2, 8), (4, 1, 1), (8, 4, 2)):
            c = L.KernelConfig.of(1, waves, unroll, kw, ks)
            if c.as_tuple() not in [d.as_tuple() for d in be.candidates(w, "f16", m, "f32")] and ks != 16:
                continue
            try:
                first = None
                for _ in range(3):
                    y = be.linear(xt, w, bt, "silu", fused=True, config=c)
                    got = y.numpy()
                    y.destroy()
                    if first is None:
                        first = got
                    assert np.array_equal(got, first), c.as_tuple()
            except L.TlhipError as e:
                assert "not applicable" in str(e), str(e)
                continue
            ran += 1
            assert rel_l2(first, want) <= 5e-6, (c.as_tuple(), rel_l2(first, want))
    assert ran >= 3


@pytest.mark.parametrize("fmt,n,k,g", [
    ("int4-grouped", 200, 256, 32),     # a row shorter than a workgroup: several rows per staging step
    ("int4-grouped", 130, 768, 64),     # 96 units per row: not a divisor of any workgroup size
    ("int4-grouped", 96, 5120, 128),    # more than one staging round at M = 16
    ("int8-row", 150, 1344, 0),
    ("int8-grouped", 64, 640, 64),
])
@pytest.mark.parametrize("m", [5, 9, 16])
def test_matrix_core_kernel_activation_staging_geometries(be, fmt, n, k, g, m):
    """The flat (row, unit) staging of the 16x16x32 kernel: every workgroup size, K split
    and slice count the kernel takes for these shapes, rows longer and shorter than a
    workgroup, M below a full tile (the rows past M alias the last row)."""
    rng = np.random.default_rng(7 * n + k + m)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    want = O.linear(x.astype(np.float32), deq, threads=8)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    cands = [c for c in be.candidates(w, "f16", m, "f32") if c.variant == L.VARIANT_GEMV_MFMA]
    assert len(cands) >= 4
    for c in cands:
        y = be.linear(xt, w, config=c)
        got = y.numpy()
        y.destroy()
        assert rel_l2(got, want) <= 5e-6, (c.as_tuple(), rel_l2(got, want))


def test_k_slices_reject_what_the_workspace_cannot_hold(be):
    rng = np.random.default_rng(5)
    n, k, m = 256, 1024, 8
    packed, scales, _ = make_weight("int4-grouped", n, k, 32, rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(make_x(m, k, "f16", rng), [m, k], "f16")
    for ks in (3, 16, 32):   # not a power of two / does not divide K/128 = 8 / too many
        with pytest.raises(L.TlhipError, match="config not applicable"):
            be.linear(xt, w, config=L.KernelConfig.of(1, 8, 2, 8, ks))


@pytest.mark.parametrize("fmt,g,xdt", [("int8-grouped", 64, "f32"), ("int8-row", 0, "f16"), ("int4-grouped", 64, "f32")])
def test_candidates_other_formats(be, fmt, g, xdt):
    rng = np.random.default_rng(43)
    n, k, m = 515, 1280, 2
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, xdt, rng)
    want = O.linear(x.astype(np.float32), deq)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    for c in be.candidates(w, xdt, m, "f32")[::3]:
        y = be.linear(xt, w, config=c)
        got = y.numpy()
        y.destroy()
        assert rel_l2(got, want) <= 2e-6, c.as_tuple()


@pytest.mark.parametrize("act", [None, "relu", "silu", "gelu", "gelu_erf", "sigmoid", "tanh"])
@pytest.mark.parametrize("fused", [False, True])
def test_bias_and_activation_fused_and_unfused(be, act, fused):
    rng = np.random.default_rng(7)
    n, k, g, m = 1024, 1024, 32, 4
    packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    got = run_linear(be, "int4-grouped", packed, scales, n, k, g, x, "f16", bias=bias, act=act, fused=fused)
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), act or "none")
    assert got.dtype == np.float16
    assert rel_l2(got, want) <= REL_L2_TOL
    # f32 output shows the epilogue arithmetic without the f16 store
    got32 = run_linear(be, "int4-grouped", packed, scales, n, k, g, x, "f32", bias=bias, act=act, fused=fused)
    assert rel_l2(got32, want) <= 1e-5


def test_reference_probe_shapes_int8_grouped(be):
    """The quant GEMV probe's generator, shapes and bar (probe-quant-gemv.ts),
    minus its lm_head-sized case which is covered below at full N."""
    cases = json.load(open(os.path.join(GOLD, "quant_probe_cases.json")))["gemv_probe"]
    draw = O.make_lcg(cases["seed"])
    for g in cases["group_sizes"]:
        for n, k in cases["shapes_nk"]:
            w = draw(n * k).astype(np.float32)
            a = draw(k).astype(np.float32)
            if n > 4096:
                continue  # keeps the LCG stream in step with the probe; big case tested separately
            packed, scales = T.quantizeLinearWeight(w, n, k, g)
            deq = O.dequant_int8_grouped(packed, scales, n, k, g)
            ref = deq.astype(np.float64) @ a.astype(np.float64)
            before = T.getQuantGemvDispatchCount()
            got = run_linear(be, "int8-grouped", packed, scales, n, k, g, a.reshape(1, k), "f32")
            assert T.getQuantGemvDispatchCount() - before == 1
            assert per_row_err(got, ref) <= cases["per_row_tol"], (n, k, g)
            assert per_row_err(got, O.linear(a.reshape(1, k), deq)) <= cases["per_row_tol"]


@pytest.mark.parametrize("waves,unroll", [(4, 4), (4, 2), (8, 4), (8, 2), (16, 2)])
@pytest.mark.parametrize("n,k,m", [(515, 1280, 2), (100, 256, 16), (4103, 2304, 8), (16, 128, 1), (9000, 512, 5)])
def test_matrix_core_gemv_with_whole_line_weight_loads(be, n, k, m, waves, unroll):
    """int8 with one scale per row, the form whose loads take 128-byte lines (8 lanes to a
    row) and pass through a wave-private LDS patch: ragged N (rows past the end alias the
    last row), one to many 128-k pairs per batch, several row blocks per wave; bias +
    activation; against the oracle and against the same kernel with operand-layout loads."""
    rng = np.random.default_rng(n + k + m + waves + unroll)
    packed, scales, deq = make_weight("int8-row", n, k, 0, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    cfg = L.KernelConfig.of(1, waves, unroll, 1, 1, 0, 1)
    if (k // 64) % unroll != 0:
        with pytest.raises(L.TlhipError, match="config not applicable"):
            run_linear(be, "int8-row", packed, scales, n, k, 0, x, "f32", config=cfg)
        return
    got = run_linear(be, "int8-row", packed, scales, n, k, 0, x, "f32", bias=bias, act="silu", fused=True, config=cfg)
    want = O.linear(x.astype(np.float32), deq, bias, "silu")
    assert got.shape == (m, n)
    assert rel_l2(got, want) <= 2e-6, rel_l2(got, want)
    plain = run_linear(be, "int8-row", packed, scales, n, k, 0, x, "f32", bias=bias, act="silu", fused=True,
                       config=L.KernelConfig.of(1, waves, unroll, 1, 1))
    assert np.array_equal(got, plain)


@pytest.mark.parametrize("waves,unroll,kw,ks", [(8, 2, 8, 1), (8, 4, 4, 1), (8, 2, 1, 1), (4, 4, 2, 2), (8, 2, 8, 4), (16, 2, 16, 1),
                                                (8, 2, 2, 8)])
@pytest.mark.parametrize("n,k,m", [(515, 2048, 3), (100, 4096, 16), (4103, 2048, 8), (16, 4096, 1)])
def test_whole_line_weight_loads_int4_with_k_splits(be, n, k, m, waves, unroll, kw, ks):
    """The same load shape for int4 with group size 32 (a pair of iterations = 256 k), with
    the K splits across waves and across workgroups the decode shapes use: the patches then
    lie behind the parked tiles in LDS.  Bit-equal to the operand-layout loads."""
    rng = np.random.default_rng(n + k + m + waves + unroll + kw + ks)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    cfg = L.KernelConfig.of(1, waves, unroll, kw, ks, 0, 1)
    base = L.KernelConfig.of(1, waves, unroll, kw, ks)
    try:
        plain = run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=base)
    except L.TlhipError:
        with pytest.raises(L.TlhipError, match="config not applicable"):
            run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=cfg)
        return
    try:
        got = run_linear(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=cfg)
    except L.TlhipError as e:   # the patches can push a launch that just fitted over the LDS budget
        assert "do not fit LDS" in str(e)
        return
    assert rel_l2(got, O.linear(x.astype(np.float32), deq)) <= 2e-6
    assert np.array_equal(got, plain)


def test_whole_line_weight_loads_reject_what_they_do_not_cover(be):
    rng = np.random.default_rng(9)
    x = make_x(2, 192, "f16", rng)
    packed, scales, _ = make_weight("int8-row", 64, 192, 0, rng)
    with pytest.raises(L.TlhipError, match="whole-line weight loads"):   # K = 192 is not a multiple of 128
        run_linear(be, "int8-row", packed, scales, 64, 192, 0, x, "f32", config=L.KernelConfig.of(1, 4, 1, 1, 1, 0, 1))
    x = make_x(2, 256, "f16", rng)
    packed, scales, _ = make_weight("int8-row", 64, 256, 0, rng)
    with pytest.raises(L.TlhipError, match="whole-line weight loads"):   # one iteration in flight
        run_linear(be, "int8-row", packed, scales, 64, 256, 0, x, "f32", config=L.KernelConfig.of(1, 4, 1, 1, 1, 0, 1))
    packed4, scales4, _ = make_weight("int4-grouped", 64, 256, 64, rng)
    with pytest.raises(L.TlhipError, match="whole-line weight loads"):   # int4 with another group size
        run_linear(be, "int4-grouped", packed4, scales4, 64, 256, 64, x, "f32", config=L.KernelConfig.of(1, 4, 2, 1, 1, 0, 1))
    x = make_x(2, 192, "f16", rng)
    packed8, scales8, _ = make_weight("int8-grouped", 64, 192, 64, rng)
    with pytest.raises(L.TlhipError, match="whole-line weight loads"):   # K = 192 again, grouped
        run_linear(be, "int8-grouped", packed8, scales8, 64, 192, 64, x, "f32", config=L.KernelConfig.of(1, 4, 1, 1, 1, 0, 1))


@pytest.mark.parametrize("g", [64, 128])
@pytest.mark.parametrize("waves,unroll,kw,ks", [(4, 4, 1, 1), (8, 2, 8, 1), (8, 2, 2, 2), (16, 2, 1, 1)])
@pytest.mark.parametrize("n,k,m", [(515, 1024, 2), (4103, 2048, 8), (100, 512, 16)])
def test_whole_line_weight_loads_int8_grouped(be, n, k, m, waves, unroll, kw, ks, g):
    """The reference's own format (int8, f16 absmax per group of 64 or 128) through the same
    load shape; bit-equal to the operand-layout loads."""
    rng = np.random.default_rng(n + k + m + waves + unroll + kw + ks + g)
    packed, scales, deq = make_weight("int8-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    try:
        plain = run_linear(be, "int8-grouped", packed, scales, n, k, g, x, "f32", config=L.KernelConfig.of(1, waves, unroll, kw, ks))
        got = run_linear(be, "int8-grouped", packed, scales, n, k, g, x, "f32", config=L.KernelConfig.of(1, waves, unroll, kw, ks, 0, 1))
    except L.TlhipError as e:
        assert "config not applicable" in str(e)
        return
    assert rel_l2(got, O.linear(x.astype(np.float32), deq)) <= 2e-6
    assert np.array_equal(got, plain)


def test_lm_head_sized_n(be):
    """N = 151936 (the probe's lm_head case) and the Gemma-shaped 256000 x 2304 int8-row."""
    rng = np.random.default_rng(3)
    n, k, g = 151936, 2048, 64
    q = rng.integers(-127, 128, (n, k)).astype(np.int8)
    packed = O.np_pack_int8(q)
    scales = f16_round(rng.uniform(0.5, 1.0, n * k // g)).view(np.uint16)
    a = make_x(1, k, "f32", rng)
    got = run_linear(be, "int8-grouped", packed, scales, n, k, g, a, "f32")
    deq = O.dequant_int8_grouped(packed, scales, n, k, g)
    want = O.linear(a, deq, threads=8)
    assert per_row_err(got, want) <= PROBE_TOL
    del deq
    n, k = 256000, 2304
    q = rng.integers(-127, 128, (n, k)).astype(np.int8)
    packed = O.np_pack_int8(q)
    rs = rng.uniform(0.002, 0.01, n).astype(np.float32)
    for m in (1, 8):
        x = make_x(m, k, "f16", rng)
        got = run_linear(be, "int8-row", packed, rs, n, k, 0, x, "f32")
        want = O.linear(x.astype(np.float32), O.dequant_int8_row(packed, rs, n, k), threads=8)
        assert rel_l2(got, want) <= 1e-5


def test_linearity_and_row_permutation_at_full_size(be):
    """Size-independent properties at a config-3 shape: y(x1+x2) = y(x1)+y(x2)
    for f16-exact sums, and permuting weight rows permutes outputs."""
    rng = np.random.default_rng(11)
    n, k, g = 12288, 4096, 32
    packed, scales, _ = make_weight("int4-grouped", n, k, g, rng)
    x1 = f16_round(rng.integers(-8, 9, (1, k)) / 8.0)
    x2 = f16_round(rng.integers(-8, 9, (1, k)) / 8.0)
    y1 = run_linear(be, "int4-grouped", packed, scales, n, k, g, x1, "f32")
    y2 = run_linear(be, "int4-grouped", packed, scales, n, k, g, x2, "f32")
    y12 = run_linear(be, "int4-grouped", packed, scales, n, k, g, f16_round(x1.astype(np.float32) + x2), "f32")
    assert rel_l2(y12, y1 + y2) <= 1e-6
    perm = rng.permutation(n)
    pp = packed.reshape(n, k // 8)[perm].reshape(-1)
    sp = scales.reshape(n, k // g)[perm].reshape(-1)
    yp = run_linear(be, "int4-grouped", pp, sp, n, k, g, x1, "f32")
    assert np.array_equal(yp[0], y1[0][perm])


def test_alpha_zero_weights_and_extreme_values(be):
    rng = np.random.default_rng(5)
    n, k, g = 256, 512, 32
    q = np.zeros((n, k), np.int8)
    q[::2] = -8
    q[1::2] = 7
    packed = O.np_pack_int4(q)
    scales = f16_round(np.full(n * k // g, 0.05)).view(np.uint16)
    x = f16_round(np.ones((2, k)))
    got = run_linear(be, "int4-grouped", packed, scales, n, k, g, x, "f32")
    want = O.linear(x.astype(np.float32), O.dequant_int4_grouped(packed, scales, n, k, g))
    assert rel_l2(got, want) <= 1e-6
    # int8 extremes incl. -128 (never produced by the quantizer, representable in the byte)
    q8 = rng.choice(np.array([-128, -127, 127, 0], np.int8), (n, k))
    p8 = O.np_pack_int8(q8)
    s8 = f16_round(rng.uniform(0.5, 2, n * k // 64)).view(np.uint16)
    x = make_x(1, k, "f32", rng)
    got = run_linear(be, "int8-grouped", p8, s8, n, k, 64, x, "f32")
    want = O.linear(x, O.dequant_int8_grouped(p8, s8, n, k, 64))
    assert rel_l2(got, want) <= 2e-6


def test_seam_errors(be):
    rng = np.random.default_rng(1)
    packed, scales, _ = make_weight("int4-grouped", 64, 128, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 64, 128, T.resolveWeightFormat("int4-32"))
    x = be.ops.tensorFromArray(np.zeros((1, 96), np.float16), [1, 96], "f16")
    with pytest.raises(ValueError, match="matmul dimension mismatch"):
        be.linear(x, w)
    with pytest.raises(ValueError, match="packed length"):
        be.createQuantizedWeight(packed[:-1], scales, 64, 128, T.resolveWeightFormat("int4-32"))
    with pytest.raises(ValueError, match="scales length"):
        be.createQuantizedWeight(packed, scales[:-1], 64, 128, T.resolveWeightFormat("int4-32"))
    with pytest.raises(ValueError, match="format.packing is required"):
        be.createQuantizedWeight(packed, scales, 64, 128, T.StorageFormat("f16"))
    bad = T.HipTensor(be, [64, 128], "f16", w.ptr, w.nbytes, False, None, w.format, None)
    with pytest.raises(ValueError, match="missing packing/scales"):
        be.ops.matmul(x, be.ops.transpose(bad))
    with pytest.raises(L.TlhipError, match="config not applicable"):
        x2 = be.ops.tensorFromArray(np.zeros((1, 128), np.float16), [1, 128], "f16")
        be.linear(x2, w, config=L.KernelConfig.of(0, 48, 1, 4, 1))
    with pytest.raises(ValueError, match="explicitly"):
        w.numpy()


def test_transpose_view_carries_format_and_scales(be):
    rng = np.random.default_rng(2)
    packed, scales, _ = make_weight("int8-grouped", 32, 64, 64, rng)
    w = be.createQuantizedWeight(packed, scales, 32, 64, T.resolveWeightFormat("int8-64"))
    assert w.shape == [32, 64] and w.dtype == "f16" and w.strides == [64, 1]
    wt = be.ops.transpose(w)
    assert wt.shape == [64, 32] and wt.strides == [1, 64]
    assert wt.format is w.format and wt.scales is w.scales and wt.ownsBuffer is False


@pytest.mark.parametrize("fmt,g,k,ns", [
    ("int4-grouped", 32, 1024, [2048, 1024, 1024]),       # q, k, v of the 0.6B decode step
    ("int4-grouped", 32, 1024, [3072, 3072]),              # gate, up
    ("int4-grouped", 64, 3072, [1024]),                    # a group of one
    ("int8-row", 0, 2304, [1000, 37, 515, 2048]),          # ragged N, four problems
    ("int8-grouped", 64, 2048, [4096, 512]),
])
def test_grouped_decode_gemvs_equal_separate_launches(be, fmt, g, k, ns):
    """q/k/v (or gate/up) in one launch: bit-identical to the separate calls with
    the same kernel configuration, and within tolerance of the oracle."""
    rng = np.random.default_rng(sum(ns) + k)
    x = make_x(1, k, "f16", rng)
    xt = be.ops.tensorFromArray(x, [1, k], "f16")
    ws, deqs, biases, bts = [], [], [], []
    for n in ns:
        packed, scales, deq = make_weight(fmt, n, k, g, rng)
        ws.append(be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32")))
        deqs.append(deq)
        b = rng.standard_normal(n).astype(np.float32)
        biases.append(b)
        bts.append(be.ops.tensorFromArray(b, [n], "f32"))
    before = T.getQuantGemvDispatchCount()
    outs = be.linearGrouped(xt, ws, bts, "silu")
    assert T.getQuantGemvDispatchCount() == before + len(ns)
    for w, bt, b, deq, o in zip(ws, bts, biases, deqs, outs):
        got = o.numpy()
        want = O.linear(x.astype(np.float32), deq, b, "silu")
        assert rel_l2(got, want) <= 2e-6
        c = be.selectedConfig(ws[int(np.argmax(ns))], "f16", 1, "f32")
        if c.variant == 0:
            c.p4 = 2
            c.p1 = min(c.p1, 2)
            sep = be.linear(xt, w, bt, "silu", fused=True, config=c).numpy()
            assert np.array_equal(got, sep)


def test_grouped_gemv_rejects_mixed_shapes(be):
    rng = np.random.default_rng(1)
    x = be.ops.tensorFromArray(make_x(1, 256, "f16", rng), [1, 256], "f16")
    p1, s1, _ = make_weight("int4-grouped", 64, 256, 32, rng)
    p2, s2, _ = make_weight("int4-grouped", 64, 512, 32, rng)
    w1 = be.createQuantizedWeight(p1, s1, 64, 256, T.resolveWeightFormat("int4-32", "f32"))
    w2 = be.createQuantizedWeight(p2, s2, 64, 512, T.resolveWeightFormat("int4-32", "f32"))
    # different K cannot share the activation row: the second problem's K does not match x
    outs = be.linearGrouped(x, [w1], None, None)
    assert outs[0].numpy().shape == (1, 64)
    with pytest.raises(ValueError, match="1..4"):
        be.linearGrouped(x, [w1] * 5)
    x17 = be.ops.tensorFromArray(make_x(17, 256, "f16", rng), [17, 256], "f16")
    with pytest.raises(ValueError, match="1..16 rows"):
        be.linearGrouped(x17, [w1])
    del w2


@pytest.mark.parametrize("m", [2, 4, 8, 16])
@pytest.mark.parametrize("fmt,g,k,ns,cfg", [
    ("int4-grouped", 32, 4096, [1024, 256, 256], None),                 # q, k, v: whatever is selected for their sum
    ("int4-grouped", 32, 2048, [1000, 37, 515, 2048], (1, 8, 2, 8, 1)),    # ragged N, four problems, LDS-staged matrix-core kernel
    ("int4-grouped", 32, 2048, [3072, 3072], (1, 8, 2, 4, 2, 0, 1)),        # gate, up: K slices across workgroups, whole-line loads
    ("int4-grouped", 32, 2048, [1536, 512], (4, 8, 2, 1, 1)),           # activations in registers
    ("int4-grouped", 32, 2048, [1536, 520], (4, 8, 1, 1, 2, 1, 1)),     # ... every load upfront, K slices, barrier
    ("int8-row", 0, 2304, [1000, 515], (1, 8, 2, 1, 1, 0, 1)),
    ("int8-grouped", 64, 2048, [768, 512], (1, 4, 2, 4, 1)),
])
def test_grouped_batched_decode_equals_the_oracle_and_separate_launches(be, fmt, g, k, ns, cfg, m):
    """q/k/v (or gate/up) of a batched decode step (M <= 16 rows on the same activations)
    in one launch of a matrix-core kernel: per problem within tolerance of the oracle, and
    bit-identical to the same configuration launched on that problem alone wherever the
    per-row-block arithmetic does not depend on the launch geometry (no K split across
    waves of different workgroups)."""
    rng = np.random.default_rng(sum(ns) + k + m)
    x = make_x(m, k, "f16", rng)
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    ws, deqs, biases, bts = [], [], [], []
    for n in ns:
        packed, scales, deq = make_weight(fmt, n, k, g, rng)
        ws.append(be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32")))
        deqs.append(deq)
        b = rng.standard_normal(n).astype(np.float32)
        biases.append(b)
        bts.append(be.ops.tensorFromArray(b, [n], "f32"))
    # the group is chosen like ONE problem with all the rows: seed that problem's winner
    total = be.createQuantizedWeight(np.zeros(sum(ns) * k // (8 if fmt.startswith("int4") else 4), np.uint32),
                                     np.zeros(sum(ns) * (k // g if g else 1), np.float32 if fmt == "int8-row" else np.uint16),
                                     sum(ns), k, T.resolveWeightFormat(fmt_name(fmt, g), "f32"))
    saved = T.exportTuningCache()
    try:
        if cfg is not None:
            be.seedPerShapeMatmulChoice(total, "f16", m, "f32", L.KernelConfig.of(*cfg))
        sel = be.selectedConfig(total, "f16", m, "f32")
        before = T.getQuantGemvDispatchCount()
        outs = be.linearGrouped(xt, ws, bts, "silu")
        assert T.getQuantGemvDispatchCount() == before + len(ns)
        for w, bt, b, deq, o in zip(ws, bts, biases, deqs, outs):
            got = o.numpy()
            want = O.linear(x.astype(np.float32), deq, b, "silu")
            assert got.shape == want.shape
            assert rel_l2(got, want) <= 2e-6, (sel.as_tuple(), rel_l2(got, want))
            if cfg is not None:
                try:
                    sep = be.linear(xt, w, bt, "silu", fused=True, config=L.KernelConfig.of(*cfg)).numpy()
                except L.TlhipError:
                    continue  # the configuration fits the group's rows but not this problem's alone
                assert np.array_equal(got, sep), sel.as_tuple()
    finally:
        T.clearTuningCache()
        T.importTuningCache(saved)


def test_k_slices_are_stable_over_many_back_to_back_launches(be):
    """The cross-workgroup combine relies on device-scope atomics for its tiles and
    counters: 300 back-to-back launches over rotating weights (so nothing stays in
    cache) must each reproduce, bit for bit, what the same weight gave the first time,
    and the unsliced kernel's answer to f32 accumulation order."""
    rng = np.random.default_rng(77)
    n, k, m, g = 4096, 12288, 16, 32
    x = make_x(m, k, "f16", rng)
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    ws = []
    for _ in range(3):
        packed = rng.integers(0, 2**32, n * k // 8, dtype=np.uint64).astype(np.uint32)
        scales = rng.uniform(0.01, 0.05, n * k // g).astype(np.float16).view(np.uint16)
        ws.append(be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32")))
    sliced = L.KernelConfig.of(1, 8, 2, 4, 4)
    firsts = [None] * 3
    outs = []
    for it in range(300):
        outs.append((it % 3, be.linear(xt, ws[it % 3], config=sliced)))
        if len(outs) == 30 or it == 299:
            for wi, y in outs:
                got = y.numpy()
                y.destroy()
                if firsts[wi] is None:
                    firsts[wi] = got
                assert np.array_equal(got, firsts[wi]), it
            outs = []
    valu = L.KernelConfig.of(0, 32, 1, 8, 1, 2)
    for wi in range(3):
        ref = be.linear(xt, ws[wi], config=valu).numpy()
        assert rel_l2(firsts[wi], ref) <= 2e-6


@pytest.mark.parametrize("n,k", [(4096, 12288), (1000, 4096), (12288, 4096), (40, 1024), (2049, 2048)])
@pytest.mark.parametrize("m", [1, 2, 7, 16])
def test_matrix_core_kernel_with_activations_in_registers(be, n, k, m):
    """Every configuration of the register-resident-activation kernel (waves, iterations
    in flight, workgroups per CU, K slices): the oracle's answer, and the same bits on a
    second launch (the K-slice sum runs in slice order whoever arrives last)."""
    rng = np.random.default_rng(n * 3 + k + m)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    cands = [c for c in be.candidates(w, "f16", m, "f32") if c.variant == L.VARIANT_GEMV_XREG]
    assert len(cands) >= 4, len(cands)
    seen_slices = set()
    for c in cands:
        seen_slices.add(max(1, c.p3))
        y1 = be.linear(xt, w, bt, "silu", fused=True, config=c)
        y2 = be.linear(xt, w, bt, "silu", fused=True, config=c)
        a, b = y1.numpy(), y2.numpy()
        y1.destroy()
        y2.destroy()
        assert np.array_equal(a, b), c.as_tuple()
        assert rel_l2(a, want) <= 5e-6, (c.as_tuple(), rel_l2(a, want))
    assert len(seen_slices) >= 2


def test_activations_in_registers_f16_out_and_rejections(be):
    rng = np.random.default_rng(91)
    n, k, m = 512, 2048, 9
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    y = be.linear(xt, w, config=L.KernelConfig.of(4, 8, 2, 1, 1))   # 16 iterations = 8 waves x 1 step x 2
    assert y.dtype == "f16"
    assert rel_l2(y.numpy().astype(np.float32), O.linear(x.astype(np.float32), deq)) <= REL_L2_TOL
    for bad in ((4, 8, 2, 1, 4),    # 4 slices: 4 iterations per slice cannot feed 8 waves x 2
                (4, 3, 1, 1, 1),    # waves
                (4, 8, 2, 3, 1),    # workgroups per CU
                (4, 4, 1, 1, 1)):   # 16 iterations / 4 waves = 4 steps... allowed: must run
        c = L.KernelConfig.of(*bad)
        if bad == (4, 4, 1, 1, 1):
            be.linear(xt, w, config=c).destroy()
            continue
        with pytest.raises(L.TlhipError, match="config not applicable"):
            be.linear(xt, w, config=c)
    # other formats, f32 activations, K not a multiple of 256: not this kernel's
    p8, s8, _ = make_weight("int8-row", 64, 1024, 0, rng)
    w8 = be.createQuantizedWeight(p8, s8, 64, 1024, T.resolveWeightFormat("int8-row", "f32"))
    x8 = be.ops.tensorFromArray(make_x(2, 1024, "f16", rng), [2, 1024], "f16")
    with pytest.raises(L.TlhipError, match="config not applicable"):
        be.linear(x8, w8, config=L.KernelConfig.of(4, 8, 1, 1, 1))


@pytest.mark.parametrize("n,k,g", [(4096, 4096, 32), (1001, 2048, 32), (520, 12288, 32), (96, 256, 64), (300, 1024, 128)])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_dot_products_on_the_4x4x4_matrix_core_instruction(be, n, k, g, m):
    """The form of the decode GEMV whose dot products go through v_mfma_f32_4x4x4_16b_f16
    (config field p5 = 1): every such configuration, every M it takes, ragged N, bias and
    activation in the epilogue; the products are exact, so the f32 bar applies."""
    rng = np.random.default_rng(n + k + g + m)
    packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng)
    bias = rng.standard_normal(n).astype(np.float32)
    want = O.linear(x.astype(np.float32), deq, bias, "silu", threads=8)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name("int4-grouped", g), "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    cands = [c for c in be.candidates(w, "f16", m, "f32") if c.variant == L.VARIANT_GEMV and c.p5 == 1]
    assert len(cands) >= 6
    for c in cands:
        y = be.linear(xt, w, bt, "silu", fused=True, config=c)
        got = y.numpy()
        y.destroy()
        assert rel_l2(got, want) <= 2e-6, (c.as_tuple(), rel_l2(got, want))


def test_the_4x4x4_form_rejects_what_it_does_not_cover(be):
    rng = np.random.default_rng(17)
    packed, scales, _ = make_weight("int4-grouped", 64, 1024, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 64, 1024, T.resolveWeightFormat("int4-32", "f32"))
    x5 = be.ops.tensorFromArray(make_x(5, 1024, "f16", rng), [5, 1024], "f16")
    x1 = be.ops.tensorFromArray(make_x(1, 1024, "f16", rng), [1, 1024], "f16")
    x32 = be.ops.tensorFromArray(make_x(1, 1024, "f32", rng), [1, 1024], "f32")
    for xt, cfg in ((x5, (0, 16, 1, 4, 1, 2, 1)),     # five rows
                    (x1, (0, 32, 1, 4, 1, 2, 1)),     # 32 lanes per row
                    (x1, (0, 16, 2, 4, 1, 2, 1)),     # two rows per lane group
                    (x32, (0, 16, 1, 4, 1, 2, 1)),    # f32 activations
                    (x1, (0, 16, 1, 4, 1, 2, 2))):    # unknown form
        with pytest.raises(L.TlhipError, match="config not applicable"):
            be.linear(xt, w, config=L.KernelConfig.of(*cfg))
    p8, s8, _ = make_weight("int8-row", 64, 1024, 0, rng)
    w8 = be.createQuantizedWeight(p8, s8, 64, 1024, T.resolveWeightFormat("int8-row", "f32"))
    with pytest.raises(L.TlhipError, match="config not applicable"):
        be.linear(x1, w8, config=L.KernelConfig.of(0, 16, 1, 4, 1, 2, 1))
