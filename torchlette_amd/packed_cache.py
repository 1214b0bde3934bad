"""On-disk cache of packed (quantized) weights: the loader's packed-operand cache
(packages/gemma2-browser/src/idb-cache.ts:154-220, used by browser-loader.ts:654-699
and examples/qwen3/loader.ts:228-254), with a directory standing in for IndexedDB.

Host-side quantization is O(N*K) and dominates a cold load, so the packed words and
scales are stored under the key ``url#tensor#scheme g G``: a change of scheme or group
size changes the key and re-quantizes instead of reusing a stale packing.  Every failure
(unwritable directory, truncated or foreign file) degrades to "no cache", as in the
reference.

File format (shared with addon/packed_cache.js): one file per key, named by the SHA-256
of the key; a header line of JSON ``{"key", "n", "k", "packed_bytes", "scales_bytes"}``
terminated by ``\\n``, then the packed u32 words and the scales, raw little-endian.
"""
from __future__ import annotations

import hashlib
import json
import os
import tempfile
from typing import Callable, Optional

import numpy as np


def packedKey(url: str, name: str, scheme: str, groupSize: int) -> str:
    """idb-cache.ts:171-178."""
    return f"{url}#{name}#{scheme}g{groupSize}"


class PackedWeightCache:
    def __init__(self, directory: str):
        self.directory = directory

    def _path(self, key: str) -> str:
        return os.path.join(self.directory, hashlib.sha256(key.encode("utf-8")).hexdigest() + ".tlpk")

    def getCachedPacked(self, key: str) -> Optional[dict]:
        """{packed: u32[...], scales: u16[...] (f32 for int8-row), n, k} or None."""
        try:
            with open(self._path(key), "rb") as f:
                head = json.loads(f.readline().decode("utf-8"))
                if head.get("key") != key:
                    return None
                pb, sb = int(head["packed_bytes"]), int(head["scales_bytes"])
                packed = f.read(pb)
                scales = f.read(sb)
                if len(packed) != pb or len(scales) != sb or f.read(1):
                    return None
            sdt = np.float32 if head.get("scales_dtype") == "f32" else np.uint16
            return {"packed": np.frombuffer(packed, np.uint32).copy(), "scales": np.frombuffer(scales, sdt).copy(),
                    "n": int(head["n"]), "k": int(head["k"])}
        except (OSError, ValueError, KeyError, TypeError):
            return None

    def putCachedPacked(self, key: str, packed, scales, n: int, k: int) -> None:
        """Best effort; a failure leaves no partial file behind."""
        tmp = None
        try:
            packed = np.ascontiguousarray(packed, np.uint32)
            scales = np.ascontiguousarray(scales)
            if scales.dtype not in (np.uint16, np.float32):
                scales = scales.astype(np.uint16)
            os.makedirs(self.directory, exist_ok=True)
            head = {"key": key, "n": int(n), "k": int(k), "packed_bytes": packed.nbytes, "scales_bytes": scales.nbytes,
                    "scales_dtype": "f32" if scales.dtype == np.float32 else "u16"}
            fd, tmp = tempfile.mkstemp(dir=self.directory, suffix=".part")
            with os.fdopen(fd, "wb") as f:
                f.write(json.dumps(head).encode("utf-8") + b"\n")
                f.write(packed.tobytes())
                f.write(scales.tobytes())
            os.replace(tmp, self._path(key))
            tmp = None
        except OSError:
            pass
        finally:
            if tmp is not None:
                try:
                    os.unlink(tmp)
                except OSError:
                    pass


def loadQuantizedWeight(backend, cache: Optional[PackedWeightCache], url: str, name: str, n: int, k: int,
                        weightFormat: str, fetchF32: Callable[[], object], elementType: str = "f16",
                        onDevice: bool = False):
    """The loader's branch for a projection weight (browser-loader.ts:654-699): look the
    packed form up; on a miss fetch the f32 weight, quantize it (on the host, or on the
    device when ``onDevice``: same bits), store it; then createQuantizedWeight.
    ``fetchF32`` is only called on a miss, as the loader skips the tensor's bytes in the
    stream on a hit.  int8 grouped formats only (the quantizer's)."""
    from .backend import quantizeLinearWeight, resolveWeightFormat

    fmt = resolveWeightFormat(weightFormat, elementType)
    g = fmt.packing.groupSize
    if fmt.packing.scheme != "int8-grouped":
        raise ValueError("loadQuantizedWeight: the quantizer produces int8-grouped weights")
    if k % 4 != 0 or k % g != 0:
        raise ValueError(f"loadQuantizedWeight: K={k} must be divisible by 4 and by the group size {g}")
    key = packedKey(url, name, fmt.packing.scheme, g)
    cached = cache.getCachedPacked(key) if cache is not None else None
    if cached is not None and (cached["n"] != n or cached["k"] != k):
        cached = None
    if cached is None:
        w = np.ascontiguousarray(fetchF32(), np.float32).reshape(n, k)
        if onDevice:
            wt = backend.ops.tensorFromArray(w, [n, k], "f32")
            q = backend.quantizeLinearWeightOnDevice(wt, g, elementType)
            wt.destroy()
            if cache is not None:
                packed = backend._download_raw(q, n * k // 4, np.uint32)
                scales = backend._download_raw(q.scales, n * k // g, np.uint16)
                cache.putCachedPacked(key, packed, scales, n, k)
            return q
        packed, scales = quantizeLinearWeight(w, n, k, g)
        cached = {"packed": packed, "scales": scales, "n": n, "k": k}
        if cache is not None:
            cache.putCachedPacked(key, packed, scales, n, k)
    return backend.createQuantizedWeight(cached["packed"], cached["scales"], n, k, fmt)
