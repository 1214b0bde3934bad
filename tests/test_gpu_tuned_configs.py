"""GPU parity of exactly what the benchmark times: every (problem, kernel
configuration) pair of the committed tuning file, at its own shape, against the
oracle (bit-exact dequant -> CPU-backend matmul).  A stale entry (a configuration
the library no longer accepts for its problem) turns this file red.

Tolerances: rel-L2 <= 1e-3 (the stated bar); f32 outputs of the decode kernels
<= 2e-6 (exact products, f32 accumulate: order noise only).  Prefill entries
(M > 16) are checked on a row sample: an output row depends on its own
activation row only, so the sample is exact for the rows it holds."""
import json
import os
import zlib

import numpy as np
import pytest

import torchlette_amd as T
from oracle import quant_oracle as O
from torchlette_amd import _lib as L
from helpers import fmt_name, make_weight, make_x, rel_l2

pytestmark = pytest.mark.gpu
TUNING = os.path.join(os.path.dirname(os.path.abspath(T.__file__)), "tuning", "mi355x.json")
ENTRIES = json.load(open(TUNING))["entries"]


def parse_key(key):
    m, n, k, fmt, g, xdt, ydt = key.split("_")
    return int(m), int(n), int(k), fmt, int(g[1:]), xdt, ydt


def sort_key(key):
    m, n, k, fmt, g, xdt, ydt = parse_key(key)
    return (fmt, g, n, k, ydt, m)  # entries that share a weight run back to back


KEYS = sorted(ENTRIES, key=sort_key)
_cache = {}


def weight_for(be, fmt, n, k, g, element):
    ident = (fmt, n, k, g, element)
    if _cache.get("ident") != ident:
        old = _cache.pop("w", None)
        if old is not None:
            old.destroy()
        _cache.clear()
        rng = np.random.default_rng(zlib.crc32(repr(ident).encode()))
        packed, scales, deq = make_weight(fmt, n, k, g, rng)
        _cache.update(ident=ident, deq=deq,
                      w=be.createQuantizedWeight(packed, scales, n, k, T.resolveWeightFormat(fmt_name(fmt, g), element)))
    return _cache["w"], _cache["deq"]


@pytest.fixture(scope="module")
def be():
    be = T.getBackend()
    yield be
    _cache.clear()


def test_the_file_has_the_benchmark_shapes():
    have = {parse_key(k)[:3] for k in ENTRIES}
    for n, k in ((4096, 4096), (12288, 4096), (4096, 12288)):
        for m in (1, 2, 4, 8, 16):
            assert (m, n, k) in have
    for m in (1, 8):
        assert (m, 256000, 2304) in have and (m, 9216, 2304) in have and (m, 2304, 9216) in have
    for m in (512, 2048):
        assert (m, 12288, 4096) in have


@pytest.mark.parametrize("key", KEYS)
def test_tuned_entry_matches_oracle_at_its_own_shape(be, key):
    m, n, k, fmt, g, xdt, ydt = parse_key(key)
    cfg = L.KernelConfig.of(*ENTRIES[key])
    w, deq = weight_for(be, fmt, n, k, g, ydt)
    # the library accepts the entry for this problem and, once imported, selects it
    T.importTuningCache(json.dumps({"version": 1, "entries": {key: ENTRIES[key]}}))
    assert be.selectedConfig(w, xdt, m, ydt).as_tuple() == cfg.as_tuple(), "stale or inapplicable tuning entry"
    rng = np.random.default_rng(zlib.crc32(key.encode()))
    x = make_x(m, k, xdt, rng, std=0.5 if m > 16 else 1.0)
    xt = be.ops.tensorFromArray(x, [m, k], xdt)
    y = be.linear(xt, w, config=cfg)
    got = y.numpy()
    y.destroy()
    xt.destroy()
    assert got.shape == (m, n)
    assert got.dtype == (np.float16 if ydt == "f16" else np.float32)
    if m > 16:
        rows = np.sort(rng.choice(m, 24, replace=False))
        want = O.linear(x[rows].astype(np.float32), deq, threads=O.max_threads())
        got = got[rows]
    else:
        want = O.linear(x.astype(np.float32), deq, threads=O.max_threads())
    err = rel_l2(got, want)
    assert err <= 1e-3, err
    if ydt == "f32" and m <= 16:
        assert err <= 2e-6, err
