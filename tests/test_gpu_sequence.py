"""GPU parity of the sequence launch (tlhip_gemv_sequence, tlhip_mlp_decode): several decode
Linears in one launch against the oracle's op-by-op sequence (dequant -> CPU matmul -> bias ->
activation -> mul), and the bounded wait's give-up path driven from the host.

f32 outputs of independent steps: exact products accumulated in f32, so only the order of
the sums differs from the oracle (rel-L2 <= 2e-6).  The MLP block rounds act(gate) * up to
f16 once (the down projection's activation type), like the unfused sequence on f16
tensors: the oracle is fed the same f16-rounded hidden product, and the stated bar 1e-3
holds end to end against the unrounded one."""
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import f16_round, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def weight(be, n, k, rng, element="f32"):
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    return be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", element)), deq


@pytest.mark.parametrize("m", [1, 3, 8, 16])
def test_independent_steps_match_the_oracle_and_separate_launches(be, m):
    """Five Linears of different shapes (ragged row blocks, K of 2048..12288, one with a
    bias and an activation, one with a residual) as one launch."""
    rng = np.random.default_rng(zlib.crc32(repr(("seq", m)).encode()))
    shapes = [(4096, 4096), (1000, 3072), (2048, 12288), (24, 4096), (5000, 3584), (13000, 1024), (20000, 256)]
    steps, wants = [], []
    for i, (n, k) in enumerate(shapes):
        w, deq = weight(be, n, k, rng)
        x = make_x(m, k, "f16", rng)
        xt = be.ops.tensorFromArray(x, [m, k], "f16")
        st = {"input": xt, "weight": w}
        bias = act = res = None
        if i == 1:
            bias = rng.standard_normal(n).astype(np.float32)
            act = "silu"
            st["bias"] = be.ops.tensorFromArray(bias, [n], "f32")
            st["activation"] = act
        want = O.linear(x.astype(np.float32), deq, bias, act or "none", threads=8)
        if i == 2:
            res = rng.standard_normal((m, n)).astype(np.float32)
            st["binary"] = ("add", be.ops.tensorFromArray(res, [m, n], "f32"))
            want = want + res
        steps.append(st)
        wants.append(want)
    before = T.getQuantGemvDispatchCount()
    outs = be.linearSequence(steps)
    assert T.getQuantGemvDispatchCount() == before + len(shapes)
    got = [o.numpy() for o in outs]
    assert be.sequenceStatus() == 0
    for (n, k), g, want in zip(shapes, got, wants):
        assert g.shape == (m, n) and g.dtype == np.float32
        assert rel_l2(g, want) <= 2e-6, ((n, k), rel_l2(g, want))
    again = [o.numpy() for o in be.linearSequence(steps)]
    for g, h in zip(got, again):
        assert np.array_equal(g, h)  # the sums are formed in a fixed order


@pytest.mark.parametrize("one_launch", [True, False], ids=["sequence-launch", "three-launches"])
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("m,hidden,ff", [(1, 4096, 12288), (8, 4096, 12288), (16, 4096, 12288), (5, 3072, 3072), (16, 2048, 8192)])
def test_mlp_block_from_one_call(be, m, hidden, ff, act, one_launch):
    """down(act(gate(x)) * up(x)): the reference's three Linears and two elementwise ops
    (packages/qwen3-browser/src/model.ts:357-361; gemma2: gelu) against the oracle, as the
    sequence launch and as tlhip_mlp_decode runs it by default (gate and up grouped, the
    gated multiply, down)."""
    rng = np.random.default_rng(zlib.crc32(repr(("mlp", m, hidden, ff, act)).encode()))
    gate, dg = weight(be, ff, hidden, rng, "f16")
    up, du = weight(be, ff, hidden, rng, "f16")
    down, dd = weight(be, hidden, ff, rng, "f32")
    x = make_x(m, hidden, "f16", rng, std=0.5)
    xt = be.ops.tensorFromArray(x, [m, hidden], "f16")
    before = T.getQuantGemvDispatchCount()
    y = be.mlpDecode(xt, gate, up, down, act, oneLaunch=one_launch).numpy()
    counted = T.getQuantGemvDispatchCount() - before
    assert counted == 2 if one_launch else counted >= 2   # the sequence's steps / the launches' Linears
    assert be.sequenceStatus() == 0
    xf = x.astype(np.float32)
    oact = "gelu_tanh" if act == "gelu" else act
    g_lin, u_lin = O.linear(xf, dg, threads=8), O.linear(xf, du, threads=8)
    h = O.gated(g_lin, u_lin, oact)
    want_exact = O.linear(h, dd, threads=8)
    assert y.shape == (m, hidden) and y.dtype == np.float32
    assert rel_l2(y, want_exact) <= 1e-3, rel_l2(y, want_exact)
    # against the same sequence on f16 tensors: the sequence launch rounds the hidden product
    # once, the three launches round gate and up to f16 first, as the model's ops would;
    # what is left is the order of the sums and the hardware exp of the activation
    if one_launch:
        h16 = f16_round(h)
    else:
        h16 = f16_round(O.gated(f16_round(g_lin).astype(np.float32), f16_round(u_lin).astype(np.float32), oact))
    want_f16 = O.linear(h16.astype(np.float32), dd, threads=8)
    assert rel_l2(y, want_f16) <= 2e-4, rel_l2(y, want_f16)
    # and the same call twice gives the same bits
    y2 = be.mlpDecode(xt, gate, up, down, act, oneLaunch=one_launch).numpy()
    assert np.array_equal(y, y2)


def test_mlp_block_from_one_call_in_the_reference_format(be):
    """tlhip_mlp_decode takes any weight format (its launches are the library's ordinary
    ones): the reference's int8 in groups of 64, gelu as in Gemma-2."""
    m, hidden, ff = 4, 1024, 4096
    rng = np.random.default_rng(91)
    ws = []
    for n, k, element in ((ff, hidden, "f16"), (ff, hidden, "f16"), (hidden, ff, "f32")):
        packed, scales, deq = make_weight("int8-grouped", n, k, 64, rng)
        ws.append((be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int8-64", element)), deq))
    (gate, dg), (up, du), (down, dd) = ws
    x = make_x(m, hidden, "f16", rng, std=0.5)
    y = be.mlpDecode(be.ops.tensorFromArray(x, [m, hidden], "f16"), gate, up, down, "gelu").numpy()
    xf = x.astype(np.float32)
    h = O.gated(O.linear(xf, dg, threads=8), O.linear(xf, du, threads=8), "gelu_tanh")
    assert rel_l2(y, O.linear(h, dd, threads=8)) <= 1e-3


def test_a_waiting_step_never_reads_what_the_buffer_held_before(be):
    """The hidden buffer is the caller's and lives across launches: the down projection of
    every launch must read what THIS launch's gate/up step wrote (its activation loads are
    agent-scope loads; nothing invalidates the caches in between), never the lines of the
    launch before.  Three launches back to back on one hidden buffer, activations that
    differ in sign and size, each against the oracle."""
    m, hidden, ff = 8, 2048, 6144
    rng = np.random.default_rng(77)
    gate, dg = weight(be, ff, hidden, rng, "f16")
    up, du = weight(be, ff, hidden, rng, "f16")
    down, dd = weight(be, hidden, ff, rng, "f32")
    h = be._alloc([m, ff], "f16")
    xs_host = [make_x(m, hidden, "f16", rng, std=s) * sign for s, sign in ((0.5, 1.0), (2.0, -1.0), (0.1, 1.0))]
    xts = [be.ops.tensorFromArray(x, [m, hidden], "f16") for x in xs_host]
    ys = [be._alloc([m, hidden], "f32") for _ in xs_host]
    for xt, y in zip(xts, ys):   # no synchronisation in between
        be.linearSequence([{"input": xt, "weight": gate, "up": up, "activation": "silu", "out": h},
                           {"input": h, "weight": down, "wait": True, "out": y}])
    assert be.sequenceStatus() == 0
    for x, y in zip(xs_host, ys):
        xf = x.astype(np.float32)
        hid = O.linear(xf, dg, None, "silu", threads=8).astype(np.float32) * O.linear(xf, du, threads=8).astype(np.float32)
        want = O.linear(f16_round(hid).astype(np.float32), dd, threads=8)
        assert rel_l2(y.numpy(), want) <= 2e-4, rel_l2(y.numpy(), want)


def test_a_wait_that_cannot_be_satisfied_gives_up_and_reports(be):
    """The give-up path, forced from the host: every wait's threshold is made unreachable
    and the polls are capped, so each workgroup's wait expires, the kernel leaves normally,
    and the status call reports the error; the next launch works again."""
    rng = np.random.default_rng(11)
    gate, _ = weight(be, 4096, 3072, rng, "f16")
    up, _ = weight(be, 4096, 3072, rng, "f16")
    down, dd = weight(be, 3072, 4096, rng, "f32")
    xt = be.ops.tensorFromArray(make_x(4, 3072, "f16", rng), [4, 3072], "f16")
    good = be.mlpDecode(xt, gate, up, down, "silu", oneLaunch=True).numpy()
    assert be.sequenceStatus() == 0
    L.call("tlhip_debug_sequence", 1, 2000)
    try:
        be.mlpDecode(xt, gate, up, down, "silu", oneLaunch=True)
        with pytest.raises(L.TlhipError, match="a wait for earlier steps"):
            be.sequenceStatus()
    finally:
        L.call("tlhip_debug_sequence", 0, 0)
    again = be.mlpDecode(xt, gate, up, down, "silu", oneLaunch=True).numpy()
    assert be.sequenceStatus() == 0
    assert np.array_equal(good, again)


def test_sequence_refuses_what_it_is_not_built_for(be):
    rng = np.random.default_rng(2)
    w, _ = weight(be, 256, 1152, rng)
    x = be.ops.tensorFromArray(make_x(2, 1152, "f16", rng), [2, 1152], "f16")
    with pytest.raises(L.TlhipError, match="multiple of 256"):
        be.linearSequence([{"input": x, "weight": w}])
    w2, _ = weight(be, 256, 4096, rng)
    x2 = be.ops.tensorFromArray(make_x(2, 4096, "f16", rng), [2, 4096], "f16")
    with pytest.raises(L.TlhipError, match="nothing to wait for"):
        be.linearSequence([{"input": x2, "weight": w2, "wait": True}])
    p8, s8, _ = make_weight("int8-row", 256, 4096, 0, rng)
    w8 = be.createQuantizedWeight(p8, s8, 256, 4096, T.resolveWeightFormat("int8-row", "f32"))
    with pytest.raises(L.TlhipError, match="int4 weights with group size 32"):
        be.linearSequence([{"input": x2, "weight": w8}])
    # only activations may be an earlier step's output: a residual that the first step writes
    w3, _ = weight(be, 4096, 4096, rng, "f16")
    first_out = be._alloc([2, 4096], "f16")
    with pytest.raises(L.TlhipError, match="overlaps the output of step 0"):
        be.linearSequence([{"input": x2, "weight": w3, "out": first_out},
                           {"input": first_out, "weight": w3, "wait": True, "binary": ("add", first_out)}])

