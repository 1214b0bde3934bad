"""The loader's packed-weight cache (CPU): key format, round trip, stale and damaged
entries, failure to write, and that the Python and JavaScript sides read each other's
files."""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from torchlette_amd.packed_cache import PackedWeightCache, packedKey

HERE = os.path.dirname(os.path.abspath(__file__))
ADDON_DIR = os.path.join(HERE, "..", "torchlette_amd", "addon")


def sample(seed=0, n=8, k=128, g=64):
    rng = np.random.default_rng(seed)
    return (rng.integers(0, 2 ** 32, n * k // 4, dtype=np.uint64).astype(np.uint32),
            rng.integers(0, 2 ** 16, n * k // g, dtype=np.uint32).astype(np.uint16), n, k)


def test_key_is_the_reference_key():
    # idb-cache.ts:171-178: `${url}#${name}#${scheme}g${groupSize}`
    assert packedKey("https://h/m.safetensors", "model.layers.0.mlp.up_proj.weight", "int8-grouped", 64) == \
        "https://h/m.safetensors#model.layers.0.mlp.up_proj.weight#int8-groupedg64"


def test_round_trip_and_miss(tmp_path):
    c = PackedWeightCache(str(tmp_path / "cache"))
    packed, scales, n, k = sample()
    key = packedKey("u", "t", "int8-grouped", 64)
    assert c.getCachedPacked(key) is None
    c.putCachedPacked(key, packed, scales, n, k)
    got = c.getCachedPacked(key)
    assert got["n"] == n and got["k"] == k
    assert np.array_equal(got["packed"], packed) and np.array_equal(got["scales"], scales)
    assert got["scales"].dtype == np.uint16
    # a change of group size is another key: re-quantize, never a stale packing
    assert c.getCachedPacked(packedKey("u", "t", "int8-grouped", 128)) is None
    # overwrite
    p2, s2, _, _ = sample(1)
    c.putCachedPacked(key, p2, s2, n, k)
    assert np.array_equal(c.getCachedPacked(key)["packed"], p2)
    assert [f for f in os.listdir(c.directory) if f.endswith(".part")] == []


def test_row_scales_keep_their_type(tmp_path):
    c = PackedWeightCache(str(tmp_path))
    packed, _, n, k = sample()
    rs = np.linspace(0.001, 0.01, n).astype(np.float32)
    c.putCachedPacked("k", packed, rs, n, k)
    got = c.getCachedPacked("k")
    assert got["scales"].dtype == np.float32 and np.array_equal(got["scales"], rs)


@pytest.mark.parametrize("damage", ["truncate", "extend", "foreign_key", "garbage_header", "empty"])
def test_damaged_entries_are_misses(tmp_path, damage):
    c = PackedWeightCache(str(tmp_path))
    packed, scales, n, k = sample()
    c.putCachedPacked("key", packed, scales, n, k)
    path = c._path("key")
    data = open(path, "rb").read()
    if damage == "truncate":
        data = data[:-3]
    elif damage == "extend":
        data += b"\0"
    elif damage == "foreign_key":
        head, body = data.split(b"\n", 1)
        h = json.loads(head)
        h["key"] = "other"
        data = json.dumps(h).encode() + b"\n" + body
    elif damage == "garbage_header":
        data = b"not json\n" + data
    else:
        data = b""
    open(path, "wb").write(data)
    assert c.getCachedPacked("key") is None


def test_unwritable_directory_is_no_cache(tmp_path):
    blocker = tmp_path / "file"
    blocker.write_text("x")
    c = PackedWeightCache(str(blocker / "sub"))  # a path under a regular file cannot be created
    packed, scales, n, k = sample()
    c.putCachedPacked("key", packed, scales, n, k)  # must not raise
    assert c.getCachedPacked("key") is None


@pytest.mark.skipif(shutil.which("node") is None, reason="no node binary on this machine")
def test_python_and_javascript_share_the_files(tmp_path):
    c = PackedWeightCache(str(tmp_path))
    packed, scales, n, k = sample(3)
    key = packedKey("https://h/m", "w", "int8-grouped", 64)
    c.putCachedPacked(key, packed, scales, n, k)
    code = f'''
      const P = require("./packed_cache.js");
      const c = new P.PackedWeightCache({json.dumps(str(tmp_path))});
      (async () => {{
        const key = P.packedKey("https://h/m", "w", "int8-grouped", 64);
        const got = await c.getCachedPacked(key);
        const miss = await c.getCachedPacked(P.packedKey("https://h/m", "w", "int8-grouped", 128));
        const key2 = P.packedKey("js", "w2", "int8-grouped", 64);
        await c.putCachedPacked(key2, got.packed.map((v) => (v ^ 0xffffffff) >>> 0), got.scales, got.n, got.k);
        console.log(JSON.stringify({{key, n: got.n, k: got.k, p0: got.packed[0], plen: got.packed.length,
                                    s0: got.scales[0], slen: got.scales.length, miss: miss === null}}));
      }})();'''
    proc = subprocess.run([shutil.which("node"), "-e", code], capture_output=True, text=True, cwd=ADDON_DIR, timeout=60)
    assert proc.returncode == 0, proc.stderr
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    assert out == {"key": key, "n": n, "k": k, "p0": int(packed[0]), "plen": packed.size, "s0": int(scales[0]),
                   "slen": scales.size, "miss": True}
    back = c.getCachedPacked(packedKey("js", "w2", "int8-grouped", 64))
    assert np.array_equal(back["packed"], ~packed) and np.array_equal(back["scales"], scales)
