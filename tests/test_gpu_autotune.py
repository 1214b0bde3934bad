"""GPU: the library's tuner and the levels of kernel choice.

selectMatmulChoice's order (src/backend/webgpu/matmul/dispatch.ts:171-192) with
the shape-class level of autotune.ts:269-300 in between: exact tuned winner,
nearest tuned problem of the class, heuristic default; each re-gated on
applicability.  The tuner times batches of launches with the weight rotating
through alias buffers; its winner must be selected afterwards, give the oracle's
answer, and not lose to the default on the same rotating pool."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
TUNING = os.path.join(os.path.dirname(os.path.abspath(T.__file__)), "tuning", "mi355x.json")


@pytest.fixture(scope="module")
def be():
    return T.getBackend()


def _weight(be, n, k, seed, element="f32"):
    rng = np.random.default_rng(seed)
    packed, scales, deq = make_weight("int4-grouped", n, k, 32, rng)
    return be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat("int4-32", element)), deq


def _time(be, qws, xt, m, out, cfg, reps=200):
    """us per launch of `cfg` with the weights rotating, events on the library stream."""
    fn = L.load().tlhip_matmul_quantized_config
    e0, e1 = C.c_void_p(), C.c_void_p()
    L.call("tlhip_event_create", C.byref(e0))
    L.call("tlhip_event_create", C.byref(e1))
    best = 1e30
    for _ in range(4):
        L.call("tlhip_event_record", e0, None)
        for i in range(reps):
            L.check(fn(C.byref(qws[i % len(qws)]), xt.ptr, L.F16, m, out.ptr, L.F32, 1.0, None, C.byref(cfg), None))
        L.call("tlhip_event_record", e1, None)
        L.call("tlhip_event_synchronize", e1)
        us = C.c_double()
        L.call("tlhip_event_elapsed_us", e0, e1, C.byref(us))
        best = min(best, us.value / reps)
    L.call("tlhip_event_destroy", e0)
    L.call("tlhip_event_destroy", e1)
    return best


def test_tuning_file_is_loaded_when_the_backend_is_created(be):
    entries = json.load(open(TUNING))["entries"]
    assert int(L.load().tlhip_counter(b"tuning_entries_loaded")) >= len(entries)
    T.importTuningCache(open(TUNING).read())  # another test may have cleared the cache since
    for n, k in ((4096, 4096), (12288, 4096), (4096, 12288)):
        scales = np.zeros(n * k // 32, np.uint16)
        w = be.createQuantizedWeight(np.zeros(n * k // 8, np.uint32), scales, n, k, T.resolveWeightFormat("int4-32", "f16"))
        for m in (1, 2, 4, 8, 16):
            want = tuple(entries[f"{m}_{n}_{k}_int4-grouped_g32_f16_f16"])
            assert be.selectedConfig(w, "f16", m, "f16").as_tuple() == want
        w.destroy()


def test_shape_class_level_sits_between_the_tuned_winner_and_the_default(be):
    T.clearTuningCache()
    try:
        near, _ = _weight(be, 6144, 2048, 1)
        far, _ = _weight(be, 256, 2048, 2)        # another size class
        tuned, _ = _weight(be, 8192, 2048, 3)
        wide = be.createQuantizedWeight(np.zeros(40960 * 2048 // 8, np.uint32), np.zeros(40960 * 64, np.uint16), 40960, 2048,
                                        T.resolveWeightFormat("int4-32", "f32"))  # same class, N five times larger
        default_near = be.selectedConfig(near, "f16", 8, "f32").as_tuple()
        default_near16 = be.selectedConfig(near, "f16", 16, "f32").as_tuple()
        default_far = be.selectedConfig(far, "f16", 8, "f32").as_tuple()
        default_wide = be.selectedConfig(wide, "f16", 8, "f32").as_tuple()
        seeded = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 4, 1, 2, 1)
        assert seeded.as_tuple() != default_near
        be.seedPerShapeMatmulChoice(tuned, "f16", 8, "f32", seeded)
        assert be.selectedConfig(tuned, "f16", 8, "f32").as_tuple() == seeded.as_tuple()
        # same class (rows, weight size class, K class, format, types), N within a factor of two
        assert be.selectedConfig(near, "f16", 8, "f32").as_tuple() == seeded.as_tuple()
        # another class, or the same class but N more than a factor of two away: the heuristic default stays
        assert be.selectedConfig(far, "f16", 8, "f32").as_tuple() == default_far
        assert be.selectedConfig(wide, "f16", 8, "f32").as_tuple() == default_wide
        # the same rows class but another row count: decode winners do not carry over
        assert be.selectedConfig(near, "f16", 16, "f32").as_tuple() == default_near16
        # other rows class: untouched
        assert be.selectedConfig(near, "f16", 1, "f32").variant == L.VARIANT_GEMV
        # an exact winner beats the class
        own = L.KernelConfig.of(L.VARIANT_GEMV_MFMA, 8, 1, 8, 1)
        be.seedPerShapeMatmulChoice(near, "f16", 8, "f32", own)
        assert be.selectedConfig(near, "f16", 8, "f32").as_tuple() == own.as_tuple()
    finally:
        T.clearTuningCache()
        T.importTuningCache(open(TUNING).read())


def test_tuner_on_a_rotating_pool_picks_an_applicable_winner_that_does_not_lose_to_the_default(be):
    n, k, m = 4096, 2048, 8
    pool = [_weight(be, n, k, 10 + i) for i in range(3)]
    ws = [w for w, _ in pool]
    qws = (L.QWeight * len(ws))(*[be._qweight(w, False) for w in ws])
    rng = np.random.default_rng(7)
    x = make_x(m, k, "f16", rng)
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    out = be._alloc([m, n], "f32")
    T.clearTuningCache()
    try:
        default = be.selectedConfig(ws[0], "f16", m, "f32")
        runs0 = T.getAutotuneRunCount()
        best_us = C.c_double()
        opts = L.AutotuneOptions(0, 3, 3, 0, 10.0, 0)
        L.call("tlhip_autotune_pool", qws, len(ws), xt.ptr, L.F16, m, out.ptr, L.F32, None, C.byref(opts), None,
               C.byref(best_us))
        assert T.getAutotuneRunCount() == runs0 + 1
        winner = be.selectedConfig(ws[0], "f16", m, "f32")
        cands = [c.as_tuple() for c in be.candidates(ws[0], "f16", m, "f32")]
        assert winner.as_tuple() in cands
        assert 1.0 < best_us.value < 100.0
        # the winner computes the right thing ...
        y = be.linear(xt, ws[1], config=winner)
        assert rel_l2(y.numpy(), O.linear(x.astype(np.float32), pool[1][1], threads=8)) <= 2e-6
        y.destroy()
        # ... and how it compares with the default on the same rotating pool is reported, not
        # asserted: a test's outcome must not depend on a clock (boxes differ by several per cent)
        t_def = _time(be, list(qws), xt, m, out, default)
        t_win = _time(be, list(qws), xt, m, out, winner)
        print(f"autotune winner {winner.as_tuple()} {t_win:.2f} us, default {default.as_tuple()} {t_def:.2f} us")
        assert t_win > 0 and t_def > 0
        # the key carries the format and the types: the export holds it
        assert f"{m}_{n}_{k}_int4-grouped_g32_f16_f32" in json.loads(T.exportTuningCache())["entries"]
    finally:
        T.clearTuningCache()
        T.importTuningCache(open(TUNING).read())


def test_lazy_tuning_at_first_dispatch_then_cached(be):
    n, k, m = 1536, 1024, 4
    w, deq = _weight(be, n, k, 21)
    rng = np.random.default_rng(8)
    x = make_x(m, k, "f16", rng)
    xt = be.ops.tensorFromArray(x, [m, k], "f16")
    want = O.linear(x.astype(np.float32), deq)
    T.clearTuningCache()
    T.setAutotuneEnabled(True)
    try:
        runs0 = T.getAutotuneRunCount()
        y = be.linear(xt, w)
        assert T.getAutotuneRunCount() == runs0 + 1
        assert rel_l2(y.numpy(), want) <= 2e-6
        y.destroy()
        key = f"{m}_{n}_{k}_int4-grouped_g32_f16_f32"
        entries = json.loads(T.exportTuningCache())["entries"]
        assert key in entries
        assert be.selectedConfig(w, "f16", m, "f32").as_tuple() == tuple(entries[key])
        y = be.linear(xt, w)  # cached: no second run
        assert T.getAutotuneRunCount() == runs0 + 1
        assert rel_l2(y.numpy(), want) <= 2e-6
        y.destroy()
        # a neighbour of the same class takes the quick search (fewer candidates), still one run
        w2, deq2 = _weight(be, 2048, 1024, 22)
        y = be.linear(xt, w2)
        assert T.getAutotuneRunCount() == runs0 + 2
        assert rel_l2(y.numpy(), O.linear(x.astype(np.float32), deq2)) <= 2e-6
        y.destroy()
    finally:
        T.setAutotuneEnabled(False)
        T.clearTuningCache()
        T.importTuningCache(open(TUNING).read())
