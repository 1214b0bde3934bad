"""GPU: captured graphs of the decode path replay to the eager result.

A graph with a K-sliced matrix-core GEMV (partial tiles and arrival counters in
the stream's workspace) and the LM-head top-k (workspace again) is replayed
several times, with the program's own eager launches and synchronisations
between the replays, and every replay is compared bit for bit with the eager
result.  Also the rules the header states: no memset into a capture, no
workspace creation under capture, replay on the capture stream only, and a
workspace that outlives its stream while a graph still points into it."""
import ctypes as C

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


def _problem(be, n, k, m, seed):
    rng = np.random.default_rng(seed)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    x = make_x(m, k, "f16", rng)
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    return w, xt, O.linear(x.astype(np.float32), deq, threads=8)


def _gemv(be, w, xt, m, out, cfg, stream=None):
    qw = be._qweight(w, False)
    return L.load().tlhip_matmul_quantized_config(C.byref(qw), xt.ptr, L.F16, m, out.ptr, L.F32, 1.0, None,
                                                  C.byref(cfg), stream)


def test_graph_with_k_slices_and_topk_replays_bit_exact(be):
    n, k, m, topk = 2048, 12288, 16, 64
    w, xt, want = _problem(be, n, k, m, 3)
    cfg = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 2, 4, 4)  # 4 K slices across workgroups
    y = be._alloc([m, n], "f32")
    tv, ti = be._alloc([topk], "f32"), be._alloc([topk], "i32")
    other = be._alloc([m, n], "f32")

    def enqueue():
        L.check(_gemv(be, w, xt, m, y, cfg))
        L.call("tlhip_topk", y.ptr, 0, n, topk, tv.ptr, ti.ptr, L.I32, None)  # top-k of the first output row

    enqueue()  # eager: creates the stream's workspace, gives the reference result
    ref_y, ref_v, ref_i = y.numpy(), tv.numpy(), ti.numpy()
    assert rel_l2(ref_y, want) <= 2e-6
    order = np.argsort(-ref_y[0], kind="stable")[:topk]
    assert np.array_equal(ref_i, order.astype(np.int32))

    graph = C.c_void_p()
    L.call("tlhip_graph_begin_capture", None)
    enqueue()
    L.call("tlhip_graph_end_capture", None, C.byref(graph))
    w2, xt2, want2 = _problem(be, 1040, 12288, 8, 4)
    cfg2 = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 2, 4, 2)
    try:
        for replay in range(5):
            # wipe the outputs, then eager work of another K-sliced problem on the same
            # workspace, then a synchronisation, then the replay
            L.call("tlhip_memset", y.ptr, 0xFF, y.nbytes, None)
            L.call("tlhip_memset", tv.ptr, 0xFF, tv.nbytes, None)
            L.call("tlhip_memset", ti.ptr, 0xFF, ti.nbytes, None)
            out2 = be._alloc([8, 1040], "f32")
            L.check(_gemv(be, w2, xt2, 8, out2, cfg2))
            assert rel_l2(out2.numpy(), want2) <= 2e-6
            out2.destroy()
            be.synchronize()
            L.call("tlhip_graph_launch", graph, None)
            assert np.array_equal(y.numpy().view(np.uint32), ref_y.view(np.uint32)), replay
            assert np.array_equal(tv.numpy().view(np.uint32), ref_v.view(np.uint32)), replay
            assert np.array_equal(ti.numpy(), ref_i), replay
    finally:
        L.call("tlhip_graph_destroy", graph)
    L.call("tlhip_graph_destroy", graph)  # idempotent
    for t in (y, tv, ti, other):
        t.destroy()


@pytest.mark.parametrize("fmt,g,cfg", [("int4-grouped", 32, (3, 128, 128, 128, 2, 2, 4)),
                                       ("int8-grouped", 64, (3, 256, 128, 128, 2, 4, 2)),
                                       ("int8-row", 0, (2, 64, 128, 64, 2, 2, 8)),
                                       ("int8-row", 0, None)])
def test_graph_with_k_sliced_tiled_gemm_replays_bit_exact(be, fmt, g, cfg):
    """A tiled GEMM whose K slices leave their partial sums in the stream's workspace and a
    second launch adds them (or, with no configuration named, whatever the routing picks for
    150 rows of f32 activations: a cast into the same workspace, then tiles): captured,
    replayed five times with eager K-sliced work on the same workspace in between, every
    replay bit-equal to the eager result."""
    rng = np.random.default_rng(7)
    m, n, k = 150, 640, 2048
    packed, scales, deq = make_weight(fmt, n, k, g, rng)
    xdt = "f16" if cfg else "f32"
    x = make_x(m, k, xdt, rng, std=0.5)
    name = "int8-row" if fmt == "int8-row" else f"{fmt.split('-')[0]}-{g}"
    w = be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(name, "f32"))
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    bias = be.ops.tensorFromArray(rng.standard_normal(n).astype(np.float32), [n], "f32")
    y = be._alloc([m, n], "f32")
    qw = be._qweight(w, False)
    ep = be.makeEpilogue(bias, "gelu")
    kc = L.KernelConfig.of(*cfg) if cfg else None

    def enqueue():
        if kc is not None:
            L.check(L.load().tlhip_matmul_quantized_config(C.byref(qw), xt.ptr, L.F16, m, y.ptr, L.F32, 1.0,
                                                           C.byref(ep), C.byref(kc), None))
        else:
            L.check(L.load().tlhip_matmul_quantized(C.byref(qw), xt.ptr, L.F32, m, y.ptr, L.F32, 1.0, C.byref(ep), None))

    enqueue()
    ref = y.numpy()
    want = O.linear(x.astype(np.float32), deq, bias.numpy(), "gelu", threads=8)
    assert rel_l2(ref, want) <= 1e-3
    graph = C.c_void_p()
    L.call("tlhip_graph_begin_capture", None)
    enqueue()
    L.call("tlhip_graph_end_capture", None, C.byref(graph))
    w2, xt2, want2 = _problem(be, 1040, 12288, 8, 4)
    cfg2 = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 2, 4, 2)
    try:
        for replay in range(5):
            L.call("tlhip_memset", y.ptr, 0xFF, y.nbytes, None)
            out2 = be._alloc([8, 1040], "f32")
            L.check(_gemv(be, w2, xt2, 8, out2, cfg2))
            assert rel_l2(out2.numpy(), want2) <= 2e-6
            out2.destroy()
            be.synchronize()
            L.call("tlhip_graph_launch", graph, None)
            assert np.array_equal(y.numpy().view(np.uint32), ref.view(np.uint32)), replay
    finally:
        L.call("tlhip_graph_destroy", graph)
    for t in (y, xt, w, bias):
        t.destroy()


def test_capture_rules(be):
    n, k, m = 512, 12288, 16
    w, xt, want = _problem(be, n, k, m, 5)
    cfg = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 2, 4, 4)
    y = be._alloc([m, n], "f32")
    s = C.c_void_p()
    L.call("tlhip_stream_create", C.byref(s))
    graph = C.c_void_p()
    # 1. a stream's first K-sliced call under capture: refused, nothing is allocated
    L.call("tlhip_graph_begin_capture", s)
    rc = _gemv(be, w, xt, m, y, cfg, s)
    assert rc == L.ERR_STATE and "capture" in L.last_error()
    # 2. no memset into a capture
    rc = L.load().tlhip_memset(y.ptr, 0, y.nbytes, s)
    assert rc == L.ERR_STATE and "captured" in L.last_error()
    L.call("tlhip_graph_end_capture", s, C.byref(graph))
    L.call("tlhip_graph_destroy", graph)
    # 3. after one eager call on the stream the same capture works ...
    L.check(_gemv(be, w, xt, m, y, cfg, s))
    L.call("tlhip_stream_synchronize", s)
    ref = y.numpy()
    assert rel_l2(ref, want) <= 2e-6
    L.call("tlhip_graph_begin_capture", s)
    L.check(_gemv(be, w, xt, m, y, cfg, s))
    L.call("tlhip_graph_end_capture", s, C.byref(graph))
    # 4. ... and replays on its capture stream only
    rc = L.load().tlhip_graph_launch(graph, None)
    assert rc == L.ERR_INVALID and "captured on" in L.last_error()
    for _ in range(3):
        L.call("tlhip_memset", y.ptr, 0xFF, y.nbytes, s)
        L.call("tlhip_graph_launch", graph, s)
        L.call("tlhip_stream_synchronize", s)
        assert np.array_equal(y.numpy().view(np.uint32), ref.view(np.uint32))
    # 5. the stream goes first, the graph (which points into the stream's workspace) second
    L.call("tlhip_stream_destroy", s)
    L.call("tlhip_graph_destroy", graph)
    y.destroy()


def test_noalloc_entry_point_under_capture_on_a_fresh_stream(be):
    """tlhip_gemv_noalloc needs no workspace: a fresh stream's first call may be captured."""
    n, k, m = 512, 12288, 16
    w, xt, want = _problem(be, n, k, m, 6)
    assert be.selectedConfig(w, "f16", m, "f32").p3 > 1
    y = be._alloc([m, n], "f32")
    s = C.c_void_p()
    L.call("tlhip_stream_create", C.byref(s))
    qw = be._qweight(w, False)
    graph = C.c_void_p()
    L.call("tlhip_graph_begin_capture", s)
    L.call("tlhip_gemv_noalloc", C.byref(qw), xt.ptr, L.F16, m, y.ptr, L.F32, 1.0, None, s)
    L.call("tlhip_graph_end_capture", s, C.byref(graph))
    for _ in range(3):
        L.call("tlhip_memset", y.ptr, 0xFF, y.nbytes, s)
        L.call("tlhip_graph_launch", graph, s)
        L.call("tlhip_stream_synchronize", s)
        assert rel_l2(y.numpy(), want) <= 2e-6
    L.call("tlhip_graph_destroy", graph)
    L.call("tlhip_stream_destroy", s)
    y.destroy()
