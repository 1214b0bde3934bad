"""TEST INFRASTRUCTURE — NOT PRODUCT CODE.

Two independent CPU restatements of torchlette's quantized-weight linear path:

* ``C``  — ctypes bindings to ``libquant_ref.so`` (``quant_ref.c``), the literal
  scalar restatement (same loop order, same roundings) of the reference code.
* the ``np_*`` functions — a vectorised numpy float64 restatement of the same
  closed forms, written separately so that the two can be checked against each
  other and against numpy's own IEEE binary16 routines.

Reference files followed (paths relative to the torchlette tree):
  src/backend/quantize.ts:22-156           f16 codec, quantize, dequantize
  docs/quantization-design.md:52-75        int8 / int4 packing
  src/backend/cpu/numeric.ts:510-595       matmul arithmetic
  src/ops/semantic/{catalog,composite,erf}.ts  activation formulas
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libquant_ref.so")

UNARY = {"none": 0, "relu": 1, "silu": 2, "gelu": 3, "gelu_tanh": 3, "gelu_erf": 4,
         "sigmoid": 5, "tanh": 6}


def build(force: bool = False) -> str:
    """Compile quant_ref.c with gcc (via the Makefile beside it)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "quant_ref.c"))
    ):
        subprocess.run(["make", "-C", _HERE, "-B", "libquant_ref.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.ref_f32_to_f16_bits.restype = ctypes.c_uint16
        L.ref_f32_to_f16_bits.argtypes = [ctypes.c_float]
        L.ref_f16_bits_to_f64.restype = ctypes.c_double
        L.ref_f16_bits_to_f64.argtypes = [ctypes.c_uint16]
        L.ref_f32_to_f16_bits_array.argtypes = [vp, vp, i64]
        L.ref_f16_bits_to_f32_array.argtypes = [vp, vp, i64]
        L.ref_quantize_int8_grouped.restype = ci
        L.ref_quantize_int8_grouped.argtypes = [vp, i64, i64, i64, vp, vp]
        L.ref_dequant_int8_grouped.argtypes = [vp, vp, i64, i64, i64, vp]
        L.ref_dequant_int8_row.argtypes = [vp, vp, i64, i64, vp]
        L.ref_dequant_int4_grouped.argtypes = [vp, vp, i64, i64, i64, vp]
        L.ref_matmul_nt.argtypes = [vp, vp, i64, i64, i64, vp, ci]
        L.ref_matmul_strided.argtypes = [vp, i64, i64, vp, i64, i64, i64, i64, i64, vp]
        L.ref_bias_add.argtypes = [vp, vp, i64, i64]
        L.ref_unary.argtypes = [ci, vp, i64]
        L.ref_unary_scalar.restype = ctypes.c_double
        L.ref_unary_scalar.argtypes = [ci, ctypes.c_double]
        L.ref_max_threads.restype = ci
        L.ref_mul.argtypes = [vp, vp, vp, i64]
        L.ref_mul.restype = None
        L.ref_rmsnorm.argtypes = [vp, vp, vp, i64, i64, ctypes.c_double]
        L.ref_rmsnorm.restype = None
        for f in ("ref_f32_to_f16_bits_array", "ref_f16_bits_to_f32_array",
                  "ref_dequant_int8_grouped", "ref_dequant_int8_row", "ref_dequant_int4_grouped",
                  "ref_matmul_nt", "ref_matmul_strided", "ref_bias_add", "ref_unary"):
            getattr(L, f).restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------
# C restatement wrappers
# --------------------------------------------------------------------------

def f32_to_f16_bits(x) -> np.ndarray:
    x = _c(x, np.float32).ravel()
    out = np.empty(x.size, np.uint16)
    lib().ref_f32_to_f16_bits_array(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(bits) -> np.ndarray:
    bits = _c(bits, np.uint16).ravel()
    out = np.empty(bits.size, np.float32)
    lib().ref_f16_bits_to_f32_array(_p(bits), _p(out), bits.size)
    return out


def quantize_int8_grouped(weight, n: int, k: int, group_size: int = 64):
    """quantizeLinearWeight (quantize.ts:77-131).  Raises like the reference."""
    weight = _c(weight, np.float32).ravel()
    if weight.size != n * k:
        raise ValueError(f"quantize: expected {n * k} elements, got {weight.size}")
    if k % 4 != 0:
        raise ValueError(f"quantize: K={k} must be divisible by 4")
    if k % group_size != 0:
        raise ValueError(f"quantize: K={k} must be divisible by groupSize={group_size}")
    packed = np.zeros(n * (k // 4), np.uint32)
    scales = np.zeros(n * (k // group_size), np.uint16)
    rc = lib().ref_quantize_int8_grouped(_p(weight), n, k, group_size, _p(packed), _p(scales))
    assert rc == 0
    return packed, scales


def dequant_int8_grouped(packed, scales, n: int, k: int, group_size: int) -> np.ndarray:
    packed, scales = _c(packed, np.uint32).ravel(), _c(scales, np.uint16).ravel()
    assert packed.size == n * k // 4 and scales.size == n * k // group_size
    out = np.empty((n, k), np.float32)
    lib().ref_dequant_int8_grouped(_p(packed), _p(scales), n, k, group_size, _p(out))
    return out


def dequant_int8_row(packed, row_scales, n: int, k: int) -> np.ndarray:
    packed, row_scales = _c(packed, np.uint32).ravel(), _c(row_scales, np.float32).ravel()
    assert packed.size == n * k // 4 and row_scales.size == n
    out = np.empty((n, k), np.float32)
    lib().ref_dequant_int8_row(_p(packed), _p(row_scales), n, k, _p(out))
    return out


def dequant_int4_grouped(packed, scales, n: int, k: int, group_size: int = 32) -> np.ndarray:
    packed, scales = _c(packed, np.uint32).ravel(), _c(scales, np.uint16).ravel()
    assert packed.size == n * k // 8 and scales.size == n * k // group_size
    out = np.empty((n, k), np.float32)
    lib().ref_dequant_int4_grouped(_p(packed), _p(scales), n, k, group_size, _p(out))
    return out


def dequant(fmt: str, packed, scales, n: int, k: int, group_size: int = 0) -> np.ndarray:
    if fmt == "int8-grouped":
        return dequant_int8_grouped(packed, scales, n, k, group_size)
    if fmt == "int8-row":
        return dequant_int8_row(packed, scales, n, k)
    if fmt == "int4-grouped":
        return dequant_int4_grouped(packed, scales, n, k, group_size)
    raise ValueError(fmt)


def matmul_nt(a, w, threads: int = 1) -> np.ndarray:
    """CPU-backend matmul of a[M,K] with the transposed view of w[N,K]."""
    a, w = _c(a, np.float32), _c(w, np.float32)
    m, k = a.shape
    n, k2 = w.shape
    if k != k2:
        raise ValueError("matmul dimension mismatch")
    out = np.empty((m, n), np.float32)
    lib().ref_matmul_nt(_p(a), _p(w), m, n, k, _p(out), threads)
    return out


def matmul(a, b) -> np.ndarray:
    """CPU-backend matmul for 1-D/2-D operands with arbitrary strides."""
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    a1, b1 = a.ndim == 1, b.ndim == 1
    am = a[None, :] if a1 else a
    bm = b[:, None] if b1 else b
    if am.shape[-1] != bm.shape[-2]:
        raise ValueError("matmul dimension mismatch")
    m, k = am.shape
    n = bm.shape[1]
    out = np.empty((m, n), np.float32)
    es = 4
    lib().ref_matmul_strided(am.ctypes.data, am.strides[0] // es, am.strides[1] // es,
                             bm.ctypes.data, bm.strides[0] // es, bm.strides[1] // es,
                             m, n, k, _p(out))
    if a1 and b1:
        return out.reshape(())
    if a1:
        return out.reshape(n)
    if b1:
        return out.reshape(m)
    return out


def bias_add(y, bias) -> np.ndarray:
    y = np.array(y, np.float32, copy=True, order="C")
    bias = _c(bias, np.float32)
    m, n = y.shape
    assert bias.shape == (n,)
    lib().ref_bias_add(_p(y), _p(bias), m, n)
    return y


def unary(op: str, y) -> np.ndarray:
    y = np.array(y, np.float32, copy=True, order="C")
    lib().ref_unary(UNARY[op], _p(y), y.size)
    return y


def mul(a, b) -> np.ndarray:
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    assert a.shape == b.shape
    out = np.empty_like(a)
    lib().ref_mul(_p(a), _p(b), _p(out), a.size)
    return out


def rmsnorm(x, weight, eps: float = 1e-6) -> np.ndarray:
    """tensor.rmsnorm on the CPU backend (decomposed-ops.ts:221-233)."""
    x = _c(x, np.float32)
    weight = _c(weight, np.float32)
    d = x.shape[-1]
    assert weight.shape == (d,)
    out = np.empty_like(x)
    lib().ref_rmsnorm(_p(x), _p(weight), _p(out), x.size // d if d else 0, d, float(eps))
    return out


def gated(gate, up, act: str = "silu") -> np.ndarray:
    """The MLP's `mul(act(gate), up)` as two CPU ops, each storing f32
    (packages/qwen3-browser/src/model.ts:357-361; gemma2-browser model.ts:411-415)."""
    return mul(unary(act, gate), up)


def linear(x, w_dequant, bias=None, act: str = "none", threads: int = 1) -> np.ndarray:
    """api.linear (+ optional activation) as the CPU backend runs it: matmul,
    then add, then the unary op — three ops, each storing f32
    (torchlette.ts:887-894; numeric.ts:439-446, 573-579)."""
    y = matmul_nt(x, w_dequant, threads)
    if bias is not None:
        y = bias_add(y, bias)
    if act != "none":
        y = unary(act, y)
    return y


def max_threads() -> int:
    return int(lib().ref_max_threads())


# --------------------------------------------------------------------------
# numpy restatement (independent of the C code)
# --------------------------------------------------------------------------

def np_f16_bits_to_f64(bits) -> np.ndarray:
    bits = np.asarray(bits, np.uint16).astype(np.int64)
    sign = np.where((bits >> 15) & 1, -1.0, 1.0)
    exp = (bits >> 10) & 0x1F
    frac = (bits & 0x3FF).astype(np.float64)
    sub = sign * 2.0 ** -14 * (frac / 1024.0)
    nor = sign * np.ldexp(1.0, (exp - 15).astype(np.int32)) * (1.0 + frac / 1024.0)
    with np.errstate(invalid="ignore"):
        special = np.where(frac == 0, sign * np.inf, np.nan)
    return np.where(exp == 0, sub, np.where(exp == 31, special, nor))


def np_f32_to_f16_bits(x) -> np.ndarray:
    """Closed-form restatement of f32ToF16Bits, not a transcription of its bit
    steps: RNE (numpy) where the result is a normal f16; round-half-up of
    |x|/2^-24 in the subnormal range; +-0x7c00 for overflow/inf/NaN."""
    x = np.asarray(x, np.float32)
    u = x.view(np.uint32)
    sign = ((u >> 16) & 0x8000).astype(np.uint16)
    e = ((u >> 23) & 0xFF).astype(np.int32)
    with np.errstate(over="ignore", invalid="ignore"):
        ax = np.abs(x).astype(np.float64)
        rne = np.abs(x).astype(np.float16).view(np.uint16)
        sub = np.floor(np.where(e < 113, ax, 0.0) * 2.0 ** 24 + 0.5).astype(np.uint16)
    out = np.where(e >= 113, rne, np.where(e < 102, 0, sub)).astype(np.uint16)
    out = np.where(e >= 143, 0x7C00, out).astype(np.uint16)
    return (out | sign).astype(np.uint16)


def np_unpack_int8(packed, n: int, k: int) -> np.ndarray:
    """[N,K/4] u32, byte lane k&3 of word k>>2 (little-endian) -> int8 [N,K]."""
    p = np.ascontiguousarray(packed, np.uint32).reshape(n, k // 4)
    lanes = np.stack([(p >> (8 * b)) & 0xFF for b in range(4)], axis=-1).reshape(n, k)
    return lanes.astype(np.uint8).view(np.int8)


def np_pack_int8(q) -> np.ndarray:
    q = np.asarray(q, np.int8)
    n, k = q.shape
    b = q.view(np.uint8).astype(np.uint32).reshape(n, k // 4, 4)
    return (b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16) | (b[..., 3] << 24)).reshape(-1)


def np_unpack_int4(packed, n: int, k: int) -> np.ndarray:
    p = np.ascontiguousarray(packed, np.uint32).reshape(n, k // 8)
    nib = np.stack([(p >> (4 * j)) & 0xF for j in range(8)], axis=-1).reshape(n, k).astype(np.int8)
    return np.where(nib >= 8, nib - 16, nib).astype(np.int8)


def np_pack_int4(q) -> np.ndarray:
    q = np.asarray(q, np.int8)
    n, k = q.shape
    u = (q.astype(np.int32) & 0xF).astype(np.uint32).reshape(n, k // 8, 8)
    w = np.zeros((n, k // 8), np.uint32)
    for j in range(8):
        w |= u[..., j] << np.uint32(4 * j)
    return w.reshape(-1)


def np_dequant_int8_grouped(packed, scales, n, k, group_size) -> np.ndarray:
    q = np_unpack_int8(packed, n, k).astype(np.float64)
    s = np_f16_bits_to_f64(np.asarray(scales, np.uint16).reshape(n, k // group_size))
    with np.errstate(invalid="ignore", over="ignore"):
        return ((q / 127.0) * np.repeat(s, group_size, axis=1)).astype(np.float32)


def np_dequant_int8_row(packed, row_scales, n, k) -> np.ndarray:
    q = np_unpack_int8(packed, n, k).astype(np.float64)
    s = np.asarray(row_scales, np.float32).astype(np.float64).reshape(n, 1)
    return (q * s).astype(np.float32)


def np_dequant_int4_grouped(packed, scales, n, k, group_size=32) -> np.ndarray:
    q = np_unpack_int4(packed, n, k).astype(np.float64)
    s = np_f16_bits_to_f64(np.asarray(scales, np.uint16).reshape(n, k // group_size))
    with np.errstate(invalid="ignore", over="ignore"):
        return (q * np.repeat(s, group_size, axis=1)).astype(np.float32)


def np_quantize_int8_grouped(weight, n, k, group_size=64):
    w = np.asarray(weight, np.float32).reshape(n, k // group_size, group_size).astype(np.float64)
    a = np.abs(w)
    absmax = np.max(np.where(np.isnan(a), 0.0, a), axis=-1)
    sbits = np_f32_to_f16_bits(absmax.astype(np.float32))
    s = np_f16_bits_to_f64(sbits)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        inv = np.where(s > 0, 127.0 / s, 0.0)
        t = w * inv[..., None]
        fl = np.floor(t)
        r = np.where(t - fl >= 0.5, fl + 1.0, fl)
    q = np.where(np.isnan(r), 0.0, np.clip(r, -127.0, 127.0)).astype(np.int8).reshape(n, k)
    return np_pack_int8(q), sbits.reshape(-1)


def np_matmul_nt(a, w) -> np.ndarray:
    """float64 dot, one rounding to f32.  Differs from the sequential-k loop
    only in the order of f64 additions (about 1e-16 relative)."""
    return (np.asarray(a, np.float32).astype(np.float64)
            @ np.asarray(w, np.float32).astype(np.float64).T).astype(np.float32)


def np_unary(op: str, y) -> np.ndarray:
    x = np.asarray(y, np.float32).astype(np.float64)
    if op == "relu":
        r = np.where(x > 0, x, 0.0)
    elif op == "silu":
        r = x / (1.0 + np.exp(-x))
    elif op in ("gelu", "gelu_tanh"):
        r = 0.5 * x * (1.0 + np.tanh(0.7978845608 * (x + 0.044715 * x * x * x)))
    elif op == "sigmoid":
        r = 1.0 / (1.0 + np.exp(-x))
    elif op == "tanh":
        r = np.tanh(x)
    elif op == "none":
        r = x
    else:
        raise ValueError(op)
    return r.astype(np.float32)


# --------------------------------------------------------------------------
# Seeded synthetic inputs shared by the tests, the smoke check and the bench
# --------------------------------------------------------------------------

_LCG_BLOCK = 1 << 16
_lcg_tables = None


def _lcg_jump_tables():
    """mult[i], add[i] with s_{i+1 steps} = mult[i]*s + add[i] mod 2^32."""
    global _lcg_tables
    if _lcg_tables is None:
        mult = np.empty(_LCG_BLOCK, np.uint64)
        add = np.empty(_LCG_BLOCK, np.uint64)
        m_, a_ = 1, 0
        for i in range(_LCG_BLOCK):
            m_ = (m_ * 1664525) & 0xFFFFFFFF
            a_ = (a_ * 1664525 + 1013904223) & 0xFFFFFFFF
            mult[i], add[i] = m_, a_
        _lcg_tables = (mult, add)
    return _lcg_tables


def make_lcg(seed: int):
    """examples/qwen3/probe-quant-gemv.ts:44-50 — s = s*1664525+1013904223 mod
    2^32; value = s/2^31 - 1 (a double).  Returns draw(count) -> float64[count],
    continuing the one stream across calls as the probe's closure does."""
    state = [seed & 0xFFFFFFFF]
    mask = np.uint64(0xFFFFFFFF)

    def draw(count: int) -> np.ndarray:
        mult, add = _lcg_jump_tables()
        out = np.empty(count, np.float64)
        s = np.uint64(state[0])
        done = 0
        while done < count:
            take = min(_LCG_BLOCK, count - done)
            vals = (mult[:take] * s + add[:take]) & mask
            out[done:done + take] = vals.astype(np.float64) / 2.0 ** 31 - 1.0
            s = vals[take - 1]
            done += take
        state[0] = int(s)
        return out

    return draw
