"""GPU parity: prefill GEMM with dequant fused into the LDS stage and a fused
epilogue, vs the oracle (bit-exact dequant -> CPU-backend matmul -> add ->
activation, each storing f32).

Tolerance: rel-L2 <= 1e-3.  The kernel rounds each dequantised weight once to
f16 before the MFMA (relative 2^-12 rms per weight), which by itself gives
about 2-3e-4; the f16 output store adds about 2e-4."""
import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import f16_round, fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
REL_L2_TOL = 1e-3
TILES = [(256, 256), (128, 256), (256, 128), (128, 128), (64, 128)]


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def tiled(bm, bn):
    return L.KernelConfig.of(L.VARIANT_TILED, bm, bn, 64, 2, 2)


def run(be, fmt, packed, scales, n, k, g, x, element, bias=None, act=None, fused=True, config=None):
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element))
    xt = be.ops.tensorFromArray(x, list(x.shape), "f16")
    bt = be.ops.tensorFromArray(bias, [n], "f16" if bias.dtype == np.float16 else "f32") if bias is not None else None
    y = be.linear(xt, w, bt, act, fused=fused, config=config)
    out = y.numpy()
    y.destroy()
    xt.destroy()
    return out


@pytest.mark.parametrize("bm,bn", TILES)
@pytest.mark.parametrize("fmt,g", [("int4-grouped", 32), ("int4-grouped", 128), ("int8-grouped", 64), ("int8-row", 0)])
def test_every_tile_config_ragged_shapes(be, fmt, g, bm, bn):
    rng = np.random.default_rng(bm * 7 + bn + g)
    m, n, k = 300, 333, 256          # neither M nor N a multiple of any tile
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    if (bm, bn) == (256, 256) and fmt != "int4-grouped":
        # not built: the int8 dequantisation would spill registers at this tile
        with pytest.raises(L.TlhipError, match="config not applicable"):
            run(be, fmt, packed, scales, n, k, g, x, "f32", config=tiled(bm, bn))
        return
    before = T.getQuantGemmDispatchCount()
    got = run(be, fmt, packed, scales, n, k, g, x, "f32", config=tiled(bm, bn))
    assert T.getQuantGemmDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert got.shape == (m, n) and got.dtype == np.float32
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)


DIRECT_TILES = [(256, 256, 2, 4), (256, 128, 2, 4), (128, 256, 2, 4), (256, 128, 4, 2), (128, 128, 2, 2), (256, 256, 2, 2),
                (128, 256, 1, 4), (128, 192, 2, 2)]


@pytest.mark.parametrize("bm,bn,wm,wn", DIRECT_TILES)
@pytest.mark.parametrize("g,m,n,k", [(32, 300, 333, 256), (128, 300, 333, 384), (32, 520, 777, 1152), (64, 64, 256, 128)])
def test_direct_weight_operand_gemm_every_tile_ragged_shapes(be, g, m, n, k, bm, bn, wm, wn):
    """The int4 GEMM whose weights are dequantised in registers (no LDS for W):
    ragged M and N, odd and even numbers of 128-k steps, bias + activation fused."""
    rng = np.random.default_rng(bm + bn + wm + g + k)
    packed, scales, deq = make_weight("int4-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = rng.standard_normal(n).astype(np.float32)
    cfg = L.KernelConfig.of(3, bm, bn, 128, wm, wn)
    before = T.getQuantGemmDispatchCount()
    got = run(be, "int4-grouped", packed, scales, n, k, g, x, "f32", bias=bias, act="gelu", config=cfg)
    assert T.getQuantGemmDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, bias, "gelu", threads=8)
    assert got.shape == (m, n) and got.dtype == np.float32
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)
    # and against the LDS-staged GEMM: same roundings of the weights, f32 accumulate
    other = run(be, "int4-grouped", packed, scales, n, k, g, x, "f32", bias=bias, act="gelu", config=tiled(128, 128))
    assert rel_l2(got, other) <= 2e-6


INT8_DIRECT_TILES = [(128, 128, 2, 2), (128, 256, 2, 4), (256, 128, 2, 4), (256, 256, 2, 4)]


@pytest.mark.parametrize("bm,bn,wm,wn", INT8_DIRECT_TILES)
@pytest.mark.parametrize("g,m,n,k,ks", [(64, 300, 333, 256, 0), (128, 300, 333, 384, 0), (64, 520, 777, 1152, 0),
                                        (256, 64, 256, 512, 2), (64, 130, 300, 2048, 4), (1024, 200, 136, 1024, 8)])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_direct_weight_operand_gemm_on_int8_groups(be, g, m, n, k, ks, bm, bn, wm, wn, ydt):
    """The same kernel on int8 weights in groups of 64 or more (one f16 scale per group,
    the format's 1/127 folded into alpha): ragged M and N, odd and even numbers of 128-k
    steps, one group per step up to one per row, K slices across workgroups, bias +
    activation fused.  Against the oracle, and against the LDS-staged kernel, which rounds
    the same products to f16 and sums in f32 too."""
    rng = np.random.default_rng(bm + bn + g + k + ks)
    packed, scales, deq = make_weight("int8-grouped", n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    cfg = L.KernelConfig.of(3, bm, bn, 128, wm, wn, ks)
    before = T.getQuantGemmDispatchCount()
    got = run(be, "int8-grouped", packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=cfg)
    assert T.getQuantGemmDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), "silu", threads=8)
    assert got.shape == (m, n) and got.dtype == (np.float16 if ydt == "f16" else np.float32)
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)
    if ydt == "f32":
        # and against the LDS-staged GEMM: the same rounding of q * scale to f16 (the format's
        # 1/127 multiplies the sums in both), f32 accumulate
        other = run(be, "int8-grouped", packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=tiled(128, 128))
        assert rel_l2(got, other) <= 2e-6, rel_l2(got, other)
    again = run(be, "int8-grouped", packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=cfg)
    assert np.array_equal(again, got)


@pytest.mark.parametrize("m,n", [(1500, 2500), (600, 6500), (1100, 3600)])
@pytest.mark.parametrize("cfg", [(3, 128, 128, 128, 2, 2), (2, 128, 128, 64, 2, 2), (2, 64, 128, 64, 2, 2)])
def test_tile_counts_whose_edge_blocks_would_crowd_some_xcds(be, m, n, cfg):
    """12 x 20, 5 x 51 and 9 x 29 tiles of 128 x 128: with the largest blocks of tiles per
    XCD the partial blocks on the edges would all fall to the same XCDs, so the workgroup ->
    tile map takes smaller blocks there.  Every tile must still be computed exactly once."""
    rng = np.random.default_rng(m + n)
    k = 256
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    got = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f32", config=L.KernelConfig.of(*cfg))
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert got.shape == (m, n)
    # per 128 x 128 tile, so that one missing or doubled tile cannot hide in the whole
    for r0 in range(0, m, 128):
        for c0 in range(0, n, 128):
            e = rel_l2(got[r0:r0 + 128, c0:c0 + 128], want[r0:r0 + 128, c0:c0 + 128])
            assert e <= REL_L2_TOL, (r0, c0, e)


@pytest.mark.parametrize("bm,bn,wm,wn", INT8_DIRECT_TILES)
@pytest.mark.parametrize("m,n,k,ks", [(300, 333, 256, 0), (520, 777, 1152, 0), (64, 256, 512, 2), (130, 300, 2048, 8)])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_direct_weight_operand_gemm_on_int8_rows(be, m, n, k, ks, bm, bn, wm, wn, ydt):
    """int8 weights with one f32 scale per row: the MFMA operand is the bare integer (exact
    in f16) and the row's scale multiplies the sums in the epilogue (or in the launch that
    adds the K slices), so the f32 output differs from the oracle only by the order of the
    f32 sums: far closer than the 1e-3 bar, which the f16 output's rounding sets."""
    rng = np.random.default_rng(bm + bn + k + ks)
    packed, scales, deq = make_weight("int8-row", n, k, 0, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    cfg = L.KernelConfig.of(3, bm, bn, 128, wm, wn, ks)
    before = T.getQuantGemmDispatchCount()
    got = run(be, "int8-row", packed, scales, n, k, 0, x, ydt, bias=bias, act="gelu", config=cfg)
    assert T.getQuantGemmDispatchCount() == before + 1
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), "gelu", threads=8)
    assert got.shape == (m, n)
    assert rel_l2(got, want) <= (REL_L2_TOL if ydt == "f16" else 5e-6), rel_l2(got, want)
    again = run(be, "int8-row", packed, scales, n, k, 0, x, ydt, bias=bias, act="gelu", config=cfg)
    assert np.array_equal(again, got)


@pytest.mark.parametrize("cfg", [(3, 128, 128, 128, 2, 2), (3, 256, 128, 128, 2, 4, 2), (2, 128, 128, 64, 2, 2),
                                 (2, 64, 128, 64, 2, 2, 2), None])
def test_int8_rows_extreme_scales_above_16_rows(be, cfg):
    """Row scales from denormal to 3e38, zero and negative zero among them: both prefill
    kernels feed the bare integers to the matrix cores and apply the row's scale to the f32
    sums, so the scale never enters f16 (a dequantised f16 weight would overflow or vanish)."""
    rng = np.random.default_rng(11)
    m, n, k = 70, 256, 256
    packed, scales, _ = make_weight("int8-row", n, k, 0, rng)
    scales = scales.copy()
    scales[:8] = np.array([0.0, -0.0, 1e-40, 3e-39, 1e-30, 1e30, 3e38, 6.1e-5], np.float32)
    q = packed.view(np.int8).reshape(n, k).astype(np.float64)
    x = make_x(m, k, "f16", rng, std=0.01)
    got = run(be, "int8-row", packed, scales, n, k, 0, x, "f32", config=L.KernelConfig.of(*cfg) if cfg else None)
    with np.errstate(over="ignore", under="ignore"):
        want = ((x.astype(np.float64) @ q.T) * scales.astype(np.float64)[None, :]).astype(np.float32)
    assert np.all(np.isfinite(got[:, 8:]))
    for c in range(n):
        if np.any(np.isinf(want[:, c])) or scales[c] < 1e-37:
            continue  # past f32 on either side: the order of the multiplications decides
        assert rel_l2(got[:, c], want[:, c]) <= 1e-5, (c, scales[c])
    assert np.all(got[:, 0] == 0) and np.all(got[:, 1] == 0)


def test_direct_gemm_rejects_what_it_does_not_cover(be):
    rng = np.random.default_rng(3)
    x = be.ops.tensorFromArray(make_x(32, 192, "f16", rng), [32, 192], "f16")
    packed, scales, _ = make_weight("int4-grouped", 64, 192, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 64, 192, T.resolveWeightFormat("int4-32", "f32"))
    with pytest.raises(L.TlhipError, match="K must be a multiple of 128"):
        be.linear(x, w, config=L.KernelConfig.of(3, 256, 256, 128, 2, 4))
    packed8, scales8, _ = make_weight("int8-row", 64, 256, 0, rng)
    w8 = be.createQuantizedWeight(packed8, scales8, 64, 256, T.resolveWeightFormat("int8-row", "f32"))
    x8 = be.ops.tensorFromArray(make_x(32, 256, "f16", rng), [32, 256], "f16")
    with pytest.raises(L.TlhipError, match="int4-grouped"):
        be.linear(x8, w8, config=L.KernelConfig.of(3, 256, 256, 128, 2, 2))   # a tile not built for int8
    # int8 in groups: groups of 64 or more, and only the tiles built for it
    p32, s32, _ = make_weight("int8-grouped", 64, 256, 32, rng)
    w32 = be.createQuantizedWeight(p32, s32, 64, 256, T.resolveWeightFormat("int8-32", "f32"))
    with pytest.raises(L.TlhipError, match="multiple of 64"):
        be.linear(x8, w32, config=L.KernelConfig.of(3, 128, 128, 128, 2, 2))
    p64, s64, _ = make_weight("int8-grouped", 64, 256, 64, rng)
    w64 = be.createQuantizedWeight(p64, s64, 64, 256, T.resolveWeightFormat("int8-64", "f32"))
    with pytest.raises(L.TlhipError, match="multiple of 64"):
        be.linear(x8, w64, config=L.KernelConfig.of(3, 128, 256, 128, 1, 4))


@pytest.mark.parametrize("m,n,k,route", [(17, 128, 64, "gemm"), (64, 64, 128, "gemm"), (100, 512, 1024, "gemm"),
                                         (1000, 256, 2048, "gemm"), (33, 1000, 4096, "rows"), (80, 1000, 4096, "any"),
                                         (130, 1000, 4096, "any")])
def test_default_route_for_m_above_16_is_the_gemm(be, m, n, k, route):
    """One tiled launch (K-sliced or not), except where a few rows on a long K make the
    decode kernel cheaper by the library's cost model (33 rows, K = 4096: one launch of
    it); in between the model decides, and either way the result is the oracle's."""
    rng = np.random.default_rng(m + n + k)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    g0, v0 = T.getQuantGemmDispatchCount(), T.getQuantGemvDispatchCount()
    got = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f16", fused=False)
    gemms, gemvs = T.getQuantGemmDispatchCount() - g0, T.getQuantGemvDispatchCount() - v0
    assert (gemms, gemvs > 0) in ((1, False), (0, True))
    if route != "any":
        assert (gemms == 1) == (route == "gemm"), (gemms, gemvs)
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert got.dtype == np.float16
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)


@pytest.mark.parametrize("act", ["silu", "gelu", "relu", None])
def test_fused_epilogue_matches_unfused_ops_and_oracle(be, act):
    """Config-4 epilogue (f16 bias then silu / gelu-tanh, f16 out) at a reduced size."""
    rng = np.random.default_rng(21)
    m, n, k = 256, 768, 1024
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), act or "none", threads=8)
    fused = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f16", bias=bias, act=act, fused=True)
    unfused = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f16", bias=bias, act=act, fused=False)
    assert rel_l2(fused, want) <= REL_L2_TOL, rel_l2(fused, want)
    assert rel_l2(unfused, want) <= REL_L2_TOL
    # the fused path skips two f16 round trips; the two agree to f16 rounding
    assert rel_l2(fused, unfused) <= 6e-4


def test_gemm_against_gemv_on_the_same_rows(be):
    """The GEMM's first 16 rows vs the (exact-integer) GEMV kernels on the same rows."""
    rng = np.random.default_rng(31)
    m, n, k = 128, 1024, 2048
    packed, scales, _ = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    full = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f32")
    part = run(be, "int4-grouped", packed, scales, n, k, 32, x[:16].copy(), "f32")
    assert rel_l2(full[:16], part) <= 5e-4


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("m", [512, 2048])
def test_config4_full_size(be, m, act):
    """M x 4096 x 12288 int4-g32, bias + silu or gelu(tanh), f16 out: a row sample
    against the sequential-k oracle, the whole output against numpy float64 (same
    sums in a different order), and linearity in the activations."""
    rng = np.random.default_rng(m)
    n, k = 12288, 4096
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    got = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f16", bias=bias, act=act)
    rows = rng.choice(m, 32, replace=False)
    want_rows = O.linear(x[rows].astype(np.float32), deq, bias.astype(np.float32), act, threads=8)
    assert rel_l2(got[rows], want_rows) <= REL_L2_TOL, rel_l2(got[rows], want_rows)
    pre = O.np_matmul_nt(x.astype(np.float32), deq)
    want = O.np_unary(act, (pre.astype(np.float64) + bias.astype(np.float64)).astype(np.float32))
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)
    if act != "silu":
        return
    # no epilogue, f32 out: y(2*x) == 2*y(x) exactly (scaling by 2 is exact in f16 and f32)
    y1 = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f32")
    y2 = run(be, "int4-grouped", packed, scales, n, k, 32, f16_round(2 * x.astype(np.float32)), "f32")
    assert np.array_equal(y2, 2 * y1)
    assert rel_l2(y1, pre) <= 5e-4


def test_gemm_rejects_f32_activations_as_an_explicit_configuration(be):
    """A tiled configuration named by the caller takes f16 activations only; without one,
    f32 rows above 16 are rounded to f16 and take the tiled kernel (next test), up to 16
    rows stay on the VALU kernel's f32 arithmetic."""
    rng = np.random.default_rng(41)
    m, n, k = 40, 256, 512
    packed, scales, deq = make_weight("int8-grouped", n, k, 64, rng)
    x = make_x(m, k, "f32", rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int8-64", "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f32")
    with pytest.raises(L.TlhipError, match="activations must be f16"):
        be.linear(xt, w, config=tiled(128, 128))
    v0, g0 = T.getQuantGemvDispatchCount(), T.getQuantGemmDispatchCount()
    y = be.linear(xt, w).numpy()
    assert T.getQuantGemvDispatchCount() == v0 and T.getQuantGemmDispatchCount() == g0 + 1
    assert rel_l2(y, O.linear(x, deq)) <= REL_L2_TOL
    x16 = be.ops.tensorFromArray(x[:16].copy(), [16, k], "f32")
    v0 = T.getQuantGemvDispatchCount()
    y16 = be.linear(x16, w).numpy()
    assert T.getQuantGemvDispatchCount() == v0 + 1
    assert rel_l2(y16, O.linear(x[:16], deq)) <= 2e-6


@pytest.mark.parametrize("m,n,k,cfg", [
    (100, 384, 1024, (3, 128, 128, 128, 2, 2, 2)),
    (256, 512, 2048, (3, 128, 128, 128, 2, 2, 8)),
    (130, 300, 1024, (3, 256, 128, 128, 2, 4, 2)),     # ragged rows and columns
    (64, 256, 4096, (3, 128, 256, 128, 1, 4, 16)),
    (300, 520, 1536, (3, 128, 192, 128, 2, 2, 4)),     # three-tile-wide waves
])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_direct_gemm_with_k_slices_across_workgroups(be, m, n, k, cfg, ydt):
    """p5 workgroups share a tile, each walking a slice of K and leaving its partial sums
    in a plane of the workspace; a second launch adds the planes in slice order and runs
    the epilogue.  Against the oracle, bit-stable from launch to launch, and as close to
    the oracle as the unsplit kernel."""
    rng = np.random.default_rng(m + n + k)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), "gelu", threads=8)
    got = run(be, "int4-grouped", packed, scales, n, k, 32, x, ydt, bias=bias, act="gelu", config=L.KernelConfig.of(*cfg))
    assert got.shape == (m, n)
    err = rel_l2(got, want)
    assert err <= REL_L2_TOL, err
    for _ in range(3):
        again = run(be, "int4-grouped", packed, scales, n, k, 32, x, ydt, bias=bias, act="gelu", config=L.KernelConfig.of(*cfg))
        assert np.array_equal(again, got)
    unsplit = run(be, "int4-grouped", packed, scales, n, k, 32, x, ydt, bias=bias, act="gelu", config=L.KernelConfig.of(*cfg[:6]))
    assert abs(rel_l2(unsplit, want) - err) <= 2e-5


@pytest.mark.parametrize("fmt,g,m,n,k,cfg", [
    ("int8-grouped", 64, 100, 384, 1024, (2, 128, 128, 64, 2, 2, 2)),
    ("int8-row", 0, 130, 300, 2048, (2, 64, 128, 64, 2, 2, 8)),      # ragged rows and columns
    ("int8-grouped", 128, 256, 512, 4096, (2, 128, 128, 64, 2, 2, 16)),
    ("int4-grouped", 128, 70, 256, 2048, (2, 64, 128, 64, 2, 2, 4)),
])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_staged_gemm_with_k_slices_across_workgroups(be, fmt, g, m, n, k, cfg, ydt):
    """The LDS-staged GEMM (every format) with p5 workgroups per tile: against the oracle,
    bit-stable from launch to launch, as close to the oracle as the unsplit kernel."""
    rng = np.random.default_rng(m + n + k)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    bias = f16_round(rng.standard_normal(n) * 0.1)
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), "silu", threads=8)
    got = run(be, fmt, packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=L.KernelConfig.of(*cfg))
    err = rel_l2(got, want)
    assert got.shape == (m, n) and err <= REL_L2_TOL, err
    again = run(be, fmt, packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=L.KernelConfig.of(*cfg))
    assert np.array_equal(again, got)
    unsplit = run(be, fmt, packed, scales, n, k, g, x, ydt, bias=bias, act="silu", config=L.KernelConfig.of(*cfg[:6]))
    assert abs(rel_l2(unsplit, want) - err) <= 2e-5


def test_direct_gemm_k_slices_reject_what_they_do_not_cover(be):
    rng = np.random.default_rng(3)
    packed, scales, _ = make_weight("int4-grouped", 256, 1024, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 256, 1024, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(make_x(64, 1024, "f16", rng), [64, 1024], "f16")
    for ks in (3, 16, 32):   # not a power of two / does not divide K / 128 = 8 / too many
        with pytest.raises(L.TlhipError, match="K split across workgroups"):
            be.linear(xt, w, config=L.KernelConfig.of(3, 128, 128, 128, 2, 2, ks))


@pytest.mark.parametrize("m,passes", [(17, 1), (40, 1), (64, 1)])
@pytest.mark.parametrize("ydt", ["f16", "f32"])
def test_a_few_more_rows_than_16_go_through_the_decode_kernel(be, m, passes, ydt):
    """17..64 rows on a small matrix: far too few tiles to fill the chip, so the library
    runs the rows through the skinny matrix-core kernel (up to 64 rows per launch, one
    dispatch per launch) instead of a tiled launch.  Heuristic choice: no tuned entry for
    these problems."""
    n, k = 1024, 4096
    rng = np.random.default_rng(m)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng, std=0.5)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", ydt))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    bias = f16_round(rng.standard_normal(n) * 0.1)
    bt = be.ops.tensorFromArray(bias, [n], "f16")
    v0, g0 = T.getQuantGemvDispatchCount(), T.getQuantGemmDispatchCount()
    y = be.linear(xt, w, bt, "silu", fused=True)
    got = y.numpy()
    assert T.getQuantGemvDispatchCount() == v0 + passes and T.getQuantGemmDispatchCount() == g0
    want = O.linear(x.astype(np.float32), deq, bias.astype(np.float32), "silu", threads=8)
    assert got.shape == (m, n)
    assert rel_l2(got, want) <= (REL_L2_TOL if ydt == "f16" else 2e-6), rel_l2(got, want)
    for t in (y, xt, bt, w):
        t.destroy()


@pytest.mark.parametrize("fmt,g,m,n,k,ydt", [
    ("int4-grouped", 32, 17, 256, 512, "f32"),
    ("int4-grouped", 32, 64, 256, 512, "f32"),
    ("int4-grouped", 32, 300, 384, 1024, "f32"),       # ragged rows and tiles
    ("int4-grouped", 128, 4352, 256, 4096, "f32"),     # more rows than one workspace chunk holds (4096 at K = 4096)
    ("int8-grouped", 64, 96, 256, 512, "f32"),
    ("int8-row", 0, 130, 192, 768, "f32"),
    ("int4-grouped", 32, 64, 4096, 4096, "f32"),       # the f16 problem's tuned winner is the skinny kernel: the heuristic tile serves
])
def test_f32_activations_from_17_rows_take_the_matrix_cores(be, fmt, g, m, n, k, ydt):
    """f32 activations, 17 rows or more: rounded to f16 once, then the prefill GEMM of
    the f16 problem (no GEMV dispatch).  Checked against the oracle on the ORIGINAL f32
    activations at the stated bar (rel-L2 <= 1e-3: the rounding of x to f16 costs about
    3e-4), and against the oracle on the rounded activations at the prefill kernels' own
    accuracy."""
    rng = np.random.default_rng(m * 7 + k)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, "f32", rng, std=0.5)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f32")
    sel = be.selectedConfig(w, "f32", m, ydt)
    assert sel.variant in (2, 3), sel.as_tuple()        # a tiled kernel
    gemms = lambda: int(L.load().tlhip_counter(b"quant_gemm_dispatches"))
    v0, d0 = T.getQuantGemvDispatchCount(), gemms()
    y = be.linear(xt, w)
    got = y.numpy()
    assert T.getQuantGemvDispatchCount() == v0
    assert gemms() == d0 + (2 if m > 4096 else 1)      # one launch per workspace chunk
    want = O.linear(x, deq, threads=8)
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)
    want16 = O.linear(f16_round(x).astype(np.float32), deq, threads=8)
    assert rel_l2(got, want16) <= 4e-4, rel_l2(got, want16)
    # the f16 problem on the same rounded rows gives the same bits
    x16 = be.ops.tensorFromArray(f16_round(x), [m, k], "f16")
    y16 = be.linear(x16, w, config=sel)
    assert np.array_equal(y16.numpy(), got)
    for t in (y, y16, x16, xt):
        t.destroy()
    w.destroy()


@pytest.mark.parametrize("lo,hi", [(200.0, 4000.0), (2e-3, 8e-3)])
@pytest.mark.parametrize("cfg", [None, (2, 128, 128, 64, 2, 2)])
def test_prefill_scale_range(be, lo, hi, cfg):
    """The prefill GEMMs round q*s once to f16 before the matrix cores: inside the stated
    scale range (|q*s| within f16's normal range) the result keeps the 1e-3 bar."""
    rng = np.random.default_rng(int(hi))
    m, n, k = 64, 256, 512
    q = rng.integers(-8, 8, (n, k)).astype(np.int8)
    packed = O.np_pack_int4(q)
    scales = f16_round(rng.uniform(lo, hi, n * (k // 32))).view(np.uint16)
    deq = O.dequant_int4_grouped(packed, scales, n, k, 32)
    x = make_x(m, k, "f16", rng, std=0.5)
    got = run(be, "int4-grouped", packed, scales, n, k, 32, x, "f32",
              config=L.KernelConfig.of(*cfg) if cfg else None)
    want = O.linear(x.astype(np.float32), deq, threads=8)
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= REL_L2_TOL, rel_l2(got, want)


@pytest.mark.parametrize("m,cfg", [(300, None), (2100, None), (300, (3, 128, 128, 128, 2, 2)), (300, (2, 128, 128, 64, 2, 2))])
def test_lm_head_sized_prefill_on_sampled_columns(be, m, cfg):
    """256000 x 2304 int8-row (the Gemma-shaped LM head) above 16 rows: 2000 column tiles,
    up to 2.1 GB of f32 logits.  The oracle runs on sampled blocks of 256 columns (the first,
    the last, and six in between) of the first and the last 300 rows."""
    rng = np.random.default_rng(m)
    n, k = 256000, 2304
    q = rng.integers(-127, 128, (n, k), dtype=np.int8)
    packed = O.np_pack_int8(q)
    rs = rng.uniform(0.002, 0.01, n).astype(np.float32)
    x = make_x(m, k, "f16", rng, std=0.5)
    w = be.createQuantizedWeight(packed, rs, n, k, T.resolveWeightFormat("int8-row", "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    y = be.linear(xt, w, config=L.KernelConfig.of(*cfg) if cfg else None)
    got = y.numpy()
    assert got.shape == (m, n) and got.dtype == np.float32
    rows = np.unique(np.concatenate([np.arange(min(m, 300)), np.arange(max(0, m - 300), m)]))
    for c0 in [0, n - 256] + [int(c) * 256 for c in rng.integers(1, n // 256 - 1, 6)]:
        deq = O.dequant_int8_row(packed.reshape(n, k // 4)[c0:c0 + 256].reshape(-1), rs[c0:c0 + 256], 256, k)
        want = O.linear(x[rows].astype(np.float32), deq, threads=8)
        assert rel_l2(got[rows][:, c0:c0 + 256], want) <= 5e-6, c0
    for t in (y, xt, w):
        t.destroy()
