"use strict";
/* On-disk cache of packed weights for the JavaScript host side: packedKey,
 * getCachedPacked, putCachedPacked of packages/gemma2-browser/src/idb-cache.ts:154-220
 * with a directory standing in for IndexedDB.  Same file format as
 * torchlette_amd/packed_cache.py: a JSON header line {key, n, k, packed_bytes,
 * scales_bytes, scales_dtype}, then the packed u32 words and the scales, raw
 * little-endian; the file is named by the SHA-256 of the key.  Failures degrade to "no
 * cache". */
const fs = require("fs");
const path = require("path");
const crypto = require("crypto");

function packedKey(url, name, scheme, groupSize) {
  return `${url}#${name}#${scheme}g${groupSize}`;
}

class PackedWeightCache {
  constructor(directory) {
    this.directory = directory;
  }
  _path(key) {
    return path.join(this.directory, crypto.createHash("sha256").update(key, "utf8").digest("hex") + ".tlpk");
  }
  async getCachedPacked(key) {
    try {
      const buf = fs.readFileSync(this._path(key));
      const nl = buf.indexOf(10);
      if (nl < 0) return null;
      const head = JSON.parse(buf.slice(0, nl).toString("utf8"));
      if (head.key !== key) return null;
      const pb = head.packed_bytes, sb = head.scales_bytes;
      if (buf.length !== nl + 1 + pb + sb) return null;
      const body = buf.buffer.slice(buf.byteOffset + nl + 1, buf.byteOffset + buf.length);  // aligned copy
      const packed = new Uint32Array(body, 0, pb / 4);
      const scales = head.scales_dtype === "f32" ? new Float32Array(body.slice(pb)) : new Uint16Array(body.slice(pb));
      return { packed, scales, n: head.n, k: head.k };
    } catch (e) {
      return null;
    }
  }
  async putCachedPacked(key, packed, scales, n, k) {
    let tmp = null;
    try {
      fs.mkdirSync(this.directory, { recursive: true });
      const p = Buffer.from(packed.buffer, packed.byteOffset, packed.byteLength);
      const s = Buffer.from(scales.buffer, scales.byteOffset, scales.byteLength);
      const head = { key, n, k, packed_bytes: p.length, scales_bytes: s.length,
                     scales_dtype: scales instanceof Float32Array ? "f32" : "u16" };
      tmp = this._path(key) + "." + process.pid + ".part";
      fs.writeFileSync(tmp, Buffer.concat([Buffer.from(JSON.stringify(head) + "\n", "utf8"), p, s]));
      fs.renameSync(tmp, this._path(key));
      tmp = null;
    } catch (e) {
      /* unwritable directory, quota: proceed without cache */
    } finally {
      if (tmp) {
        try {
          fs.unlinkSync(tmp);
        } catch (e) { /* nothing to remove */ }
      }
    }
  }
}

module.exports = { packedKey, PackedWeightCache };
