"""GPU parity: the two producers of a decode Linear's input — RMSNorm and the MLP's
act(gate) * up — as kernels of their own and fused into the GEMV that consumes
them, against the oracle's restatement of the CPU backend
(decomposed-ops.ts:221-233; qwen3-browser model.ts:357-361).

Tolerances.  f32 results: the device sums the squares in another order and takes
exp / reciprocal from the hardware approximations (about 1 ulp), so elementwise
results agree to a few f32 ulps: max |d| <= 4e-6 * max |ref| asserted.  A fused
GEMV on f32 activations inherits that on its inputs: rel-L2 <= 1e-5.  With f16
activations the fused kernels round f(x) to f16 once, like the kernel of its own
writing f16; a value that sits on a rounding boundary may fall to the other side,
so the stated bar rel-L2 <= 1e-3 applies."""
import ctypes as C
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import f16_round, fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
ELEMENTWISE_F32 = 4e-6
FUSED_F32 = 1e-5
F16_BAR = 1e-3


@pytest.fixture(scope="module")
def be():
    b = T.getBackend()
    b.fusedPrologueMaxRows = 4  # every row count the fused kernel takes, not only those where it is faster
    yield b
    del b.fusedPrologueMaxRows


def seeded(*key):
    return np.random.default_rng(zlib.crc32(repr(key).encode()))


def max_rel(got, want):
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(np.asarray(got, np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def norm_weight(k, rng):
    return (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float32)


# ----------------------------------------------------------------- standalone
@pytest.mark.parametrize("m,d", [(1, 4096), (3, 333), (16, 1000), (2, 8), (1, 12288), (300, 64)])
@pytest.mark.parametrize("xdt,ydt", [("f32", "f32"), ("f16", "f16"), ("f32", "f16"), ("f16", "f32")])
def test_rmsnorm_matches_oracle(be, m, d, xdt, ydt):
    rng = seeded("rmsnorm", m, d, xdt, ydt)
    x = make_x(m, d, xdt, rng, std=3.0)
    w = norm_weight(d, rng)
    eps = 1e-6
    xt = be.ops.tensorFromArray(x, [m, d], xdt)
    wt = be.ops.tensorFromArray(w, [d], "f32")
    y = be.ops.fusedRMSNormForward(xt, wt, {"numRows": m, "featureDim": d, "eps": eps}, outDtype=ydt)
    got = y.numpy().astype(np.float32)
    want = O.rmsnorm(x.astype(np.float32), w, eps)
    assert got.shape == (m, d)
    if ydt == "f32":
        assert max_rel(got, want) <= ELEMENTWISE_F32
    else:
        assert rel_l2(got, want) <= F16_BAR
    for t in (xt, wt, y):
        t.destroy()


def test_rmsnorm_reference_spec_rows(be):
    # the rows of test/nn-rmsnorm.spec.ts:31-41, unit weight, eps 1e-6, tolerance 1e-4 there
    rows = np.array([[0.5, -1.2, 2.0, 0.1, -0.7, 1.5, -2.2, 0.9],
                     [3.0, 0.0, -1.0, 0.25, 1.1, -0.4, 0.8, -1.6]], np.float32)
    xt = be.ops.tensorFromArray(rows, [2, 8], "f32")
    wt = be.ops.tensorFromArray(np.ones(8, np.float32), [8], "f32")
    y = be.ops.fusedRMSNormForward(xt, wt, {"numRows": 2, "featureDim": 8, "eps": 1e-6})
    ms = np.mean(rows.astype(np.float64) ** 2, axis=1, keepdims=True)
    want = rows / np.sqrt(ms + 1e-6)
    assert np.max(np.abs(y.numpy() - want)) < 1e-6
    for t in (xt, wt, y):
        t.destroy()


def test_rmsnorm_zero_rows_and_empty(be):
    xt = be.ops.tensorFromArray(np.zeros((2, 64), np.float32), [2, 64], "f32")
    wt = be.ops.tensorFromArray(np.ones(64, np.float32), [64], "f32")
    y = be.ops.fusedRMSNormForward(xt, wt, {"numRows": 2, "featureDim": 64, "eps": 1e-6})
    assert np.all(y.numpy() == 0.0)
    e = be.ops.zeros([0, 64], "f32")
    y0 = be.ops.fusedRMSNormForward(e, wt, {"numRows": 0, "featureDim": 64, "eps": 1e-6})
    assert y0.numpy().shape == (0, 64)
    with pytest.raises(ValueError):
        be.ops.fusedRMSNormForward(xt, wt, {"numRows": 3, "featureDim": 64, "eps": 1e-6})


@pytest.mark.parametrize("act", ["silu", "gelu_tanh", "none", "relu"])
@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("count", [1, 255, 12288, 4 * 12288 + 3])
def test_gated_mul_matches_oracle(be, act, dt, count):
    rng = seeded("gated", act, dt, count)
    g = make_x(1, count, dt, rng, std=3.0)[0]
    u = make_x(1, count, dt, rng)[0]
    gt = be.ops.tensorFromArray(g, [count], dt)
    ut = be.ops.tensorFromArray(u, [count], dt)
    y = be.ops.gatedMul(gt, ut, act)
    got = y.numpy().astype(np.float32)
    want = O.gated(g.astype(np.float32), u.astype(np.float32), act)
    if dt == "f32":
        # gelu's 1 + tanh(.) cancels for negative gates: the f32 error scales with |gate * up|
        scale = np.maximum(np.abs(want), np.abs(g * u))
        assert np.max(np.abs(got - want) / np.maximum(scale, 1e-3)) <= ELEMENTWISE_F32
    else:
        assert rel_l2(got, want) <= F16_BAR
    if act == "none" and dt == "f32":
        assert np.array_equal(got, g * u)  # api.mul: the IEEE product
    for t in (gt, ut, y):
        t.destroy()


# ---------------------------------------------------------------------- fused
SHAPES = [
    ("int4-grouped", 1024, 4096, 32, "f16", "f16"),
    ("int4-grouped", 768, 1024, 32, "f16", "f16"),
    ("int4-grouped", 512, 3072, 32, "f32", "f32"),
    ("int8-row", 512, 2304, 0, "f16", "f32"),
    ("int8-row", 640, 1024, 0, "f32", "f32"),
    ("int8-grouped", 512, 2048, 64, "f32", "f32"),
    ("int8-grouped", 384, 1024, 128, "f16", "f16"),
]


def fused_want(fx, deq, xdt):
    """f(x) as the kernel stages it (one f16 rounding for f16 activations), then the
    CPU-backend matmul."""
    if xdt == "f16":
        fx = f16_round(fx).astype(np.float32)
    return O.linear(fx, deq)


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("fmt,n,k,g,xdt,element", SHAPES)
def test_gemv_with_rmsnorm_prologue(be, fmt, n, k, g, xdt, element, m):
    rng = seeded("pro-rms", fmt, n, k, m)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(m, k, xdt, rng, std=2.5)
    nw = norm_weight(k, rng)
    eps = 1e-6
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element))
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    nwt = be.ops.tensorFromArray(nw, [k], "f32")
    before = T.getQuantGemvDispatchCount()
    y = be.linearAfterRMSNorm(xt, nwt, eps, w)
    assert T.getQuantGemvDispatchCount() == before + 1
    got = y.numpy().astype(np.float32)
    want = fused_want(O.rmsnorm(x.astype(np.float32), nw, eps), deq, xdt)
    assert got.shape == (m, n)
    assert rel_l2(got, want) <= (FUSED_F32 if xdt == "f32" else F16_BAR)
    for t in (xt, nwt, y):
        t.destroy()


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("fmt,n,k,g,xdt,element", SHAPES)
def test_gemv_with_gated_mul_prologue(be, fmt, n, k, g, xdt, element, m, act):
    rng = seeded("pro-gated", fmt, n, k, m, act)
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    gate = make_x(m, k, xdt, rng, std=2.0)
    up = make_x(m, k, xdt, rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element))
    gt = be.ops.tensorFromArray(gate, [m, k], xdt)
    ut = be.ops.tensorFromArray(up, [m, k], xdt)
    y = be.linearAfterGatedMul(gt, ut, act, w)
    got = y.numpy().astype(np.float32)
    want = fused_want(O.gated(gate.astype(np.float32), up.astype(np.float32), act), deq, xdt)
    assert rel_l2(got, want) <= (FUSED_F32 if xdt == "f32" else F16_BAR)
    for t in (gt, ut, y):
        t.destroy()


def test_prologue_with_bias_and_activation_epilogue(be):
    fmt, n, k, g = "int4-grouped", 1024, 2048, 32
    rng = seeded("pro-epi")
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(2, k, "f16", rng, std=2.0)
    nw = norm_weight(k, rng)
    bias = rng.standard_normal(n).astype(np.float32)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    xt = be.ops.tensorFromArray(x, [2, k], "f16")
    nwt = be.ops.tensorFromArray(nw, [k], "f32")
    bt = be.ops.tensorFromArray(bias, [n], "f32")
    y = be.linearAfterRMSNorm(xt, nwt, 1e-5, w, bt, "silu")
    fx = f16_round(O.rmsnorm(x.astype(np.float32), nw, 1e-5)).astype(np.float32)
    want = O.linear(fx, deq, bias, "silu")
    assert rel_l2(y.numpy().astype(np.float32), want) <= F16_BAR


def test_prologue_every_valu_config(be):
    """The staging code is shared by all VALU configurations: lanes per row, rows per
    lane group, waves, K-split waves and chunks in flight only change what follows."""
    fmt, n, k, g = "int4-grouped", 512, 2048, 32
    rng = seeded("pro-cfg")
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    x = make_x(3, k, "f16", rng, std=2.0)
    nw = norm_weight(k, rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    xt = be.ops.tensorFromArray(x, [3, k], "f16")
    nwt = be.ops.tensorFromArray(nw, [k], "f32")
    want = fused_want(O.rmsnorm(x.astype(np.float32), nw, 1e-6), deq, "f16")
    tried = 0
    for cfg in be.candidates(w, "f16", 3, "f16"):
        if cfg.variant != L.VARIANT_GEMV:
            continue
        be.seedPerShapeMatmulChoice(w, "f16", 3, "f16", cfg)
        y = be.linearAfterRMSNorm(xt, nwt, 1e-6, w)
        assert rel_l2(y.numpy().astype(np.float32), want) <= F16_BAR, cfg.as_tuple()
        y.destroy()
        tried += 1
    T.clearTuningCache()
    assert tried >= 20


def test_more_rows_than_the_fused_kernel_takes_fall_back(be):
    fmt, n, k, g = "int4-grouped", 512, 1024, 32
    rng = seeded("pro-fallback")
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    m = 7
    x = make_x(m, k, "f16", rng, std=2.0)
    nw = norm_weight(k, rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    nwt = be.ops.tensorFromArray(nw, [k], "f32")
    y = be.linearAfterRMSNorm(xt, nwt, 1e-6, w)
    want = fused_want(O.rmsnorm(x.astype(np.float32), nw, 1e-6), deq, "f16")
    assert rel_l2(y.numpy().astype(np.float32), want) <= F16_BAR
    # the C entry point itself says so, with its own code
    qw = be._qweight(w, transposed=False)
    pro = L.Prologue(L.PRO_RMSNORM, 0, 1e-6, 0, nwt.ptr)
    rc = L.load().tlhip_gemv_prologue(C.byref(qw), C.byref(pro), xt.ptr, L.F16, m, y.ptr, L.F16, 1.0, None,
                                      be.stream)
    assert rc == L.ERR_UNSUPPORTED
    assert "M <= 4" in L.last_error()


def test_prologue_rejects_bad_requests(be):
    fmt, n, k, g = "int4-grouped", 256, 1024, 32
    rng = seeded("pro-bad")
    packed, scales, _ = make_weight(fmt, n, k, g, rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    xt = be.ops.tensorFromArray(make_x(1, k, "f16", rng), [1, k], "f16")
    nwt = be.ops.tensorFromArray(norm_weight(k + 4, rng), [k + 4], "f32")
    y = be.ops.zeros([1, n], "f16")
    qw = be._qweight(w, transposed=False)

    def call(pro):
        return L.load().tlhip_gemv_prologue(C.byref(qw), C.byref(pro), xt.ptr, L.F16, 1, y.ptr, L.F16, 1.0, None,
                                            be.stream)

    assert call(L.Prologue(7, 0, 0.0, 0, nwt.ptr)) == L.ERR_INVALID
    assert call(L.Prologue(L.PRO_RMSNORM, 0, 1e-6, 0, None)) == L.ERR_INVALID
    assert call(L.Prologue(L.PRO_RMSNORM, 0, -1.0, 0, nwt.ptr)) == L.ERR_INVALID
    assert call(L.Prologue(L.PRO_RMSNORM, 0, 1e-6, 0, nwt.ptr + 4)) == L.ERR_INVALID  # not 16-byte aligned
    assert call(L.Prologue(L.PRO_GATED_MUL, 99, 0.0, 0, xt.ptr)) == L.ERR_INVALID
    with pytest.raises(ValueError):
        be.linearAfterRMSNorm(xt, nwt, 1e-6, w)  # norm weight of the wrong length


@pytest.mark.parametrize("fmt,k,g,ns", [
    ("int4-grouped", 4096, 32, (4096, 1024, 1024)),   # q / k / v of Qwen3-8B
    ("int4-grouped", 2048, 32, (3072, 3072)),         # gate / up
    ("int8-grouped", 1024, 64, (512, 256, 256, 128)),
])
def test_grouped_gemv_with_rmsnorm_prologue(be, fmt, k, g, ns):
    rng = seeded("pro-grouped", fmt, k, ns)
    x = make_x(1, k, "f16", rng, std=2.0)
    nw = norm_weight(k, rng)
    xt = be.ops.tensorFromArray(x, [1, k], "f16")
    nwt = be.ops.tensorFromArray(nw, [k], "f32")
    ws, deqs = [], []
    for n in ns:
        packed, scales, deq = make_weight(fmt, n, k, g, rng)
        ws.append(be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), "f16")))
        deqs.append(deq)
    outs = be.linearGroupedAfterRMSNorm(xt, nwt, 1e-6, ws)
    fx = O.rmsnorm(x.astype(np.float32), nw, 1e-6)
    for o, deq, wt in zip(outs, deqs, ws):
        want = fused_want(fx, deq, "f16")
        assert rel_l2(o.numpy().astype(np.float32), want) <= F16_BAR
        # and the same bits as the single fused launch of that weight
        single = be.linearAfterRMSNorm(xt, nwt, 1e-6, wt)
        assert rel_l2(o.numpy().astype(np.float32), single.numpy().astype(np.float32)) <= 2e-3
        single.destroy()
        o.destroy()


def test_prologue_empty_problems(be):
    """N = 0 and M = 0 launch nothing and say so (an empty output, no error)."""
    rng = seeded("pro-empty")
    k = 1024
    packed, scales, _ = make_weight("int4-grouped", 16, k, 32, rng)
    w = be.createQuantizedWeight(packed, scales, 16, k, T.resolveWeightFormat("int4-32", "f16"))
    nwt = be.ops.tensorFromArray(norm_weight(k, rng), [k], "f32")
    x0 = be.ops.zeros([0, k], "f16")
    y0 = be.linearAfterRMSNorm(x0, nwt, 1e-6, w)
    assert y0.numpy().shape == (0, 16)
    u0 = be.ops.zeros([0, k], "f16")
    assert be.linearAfterGatedMul(x0, u0, "silu", w).numpy().shape == (0, 16)
    assert be.ops.gatedMul(x0, u0, "silu").numpy().shape == (0, k)


def test_full_size_properties_of_the_fused_forms(be):
    """At the Qwen3-8B decode shapes the oracle would take minutes; what must hold at any
    size: the fused launch equals the two launches apart (same roundings of f(x), f32
    accumulation order aside), RMSNorm ignores a power-of-two rescaling of x (eps = 0), and
    a zero `up` row gives exactly zero."""
    rng = seeded("pro-full")
    n, k = 4096, 12288
    packed = rng.integers(0, 2 ** 32, n * k // 8, dtype=np.uint64).astype(np.uint32)
    scales = f16_round(rng.uniform(0.01, 0.05, n * k // 32)).view(np.uint16)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
    x = make_x(2, k, "f16", rng, std=1.5)
    xt = be.ops.tensorFromArray(x, [2, k], "f16")
    nwt = be.ops.tensorFromArray(norm_weight(k, rng), [k], "f32")
    fused = be.linearAfterRMSNorm(xt, nwt, 0.0, w).numpy().astype(np.float32)
    normed = be.ops.fusedRMSNormForward(xt, nwt, {"numRows": 2, "featureDim": k, "eps": 0.0})
    apart = be.linear(normed, w, fused=True).numpy().astype(np.float32)
    assert rel_l2(fused, apart) <= F16_BAR
    x4 = be.ops.tensorFromArray((x.astype(np.float32) * 4).astype(np.float16), [2, k], "f16")
    again = be.linearAfterRMSNorm(x4, nwt, 0.0, w).numpy().astype(np.float32)
    assert rel_l2(again, fused) <= F16_BAR
    up = make_x(2, k, "f16", rng)
    up[1] = 0
    ut = be.ops.tensorFromArray(up, [2, k], "f16")
    g = be.linearAfterGatedMul(xt, ut, "silu", w).numpy().astype(np.float32)
    assert np.all(g[1] == 0.0) and np.any(g[0] != 0.0)
    prod = be.ops.gatedMul(xt, ut, "silu")
    assert rel_l2(g, be.linear(prod, w, fused=True).numpy().astype(np.float32)) <= F16_BAR
