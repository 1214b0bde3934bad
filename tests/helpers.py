"""Seeded synthetic operands for the parity tests (shared with nothing else).

Every f16 quantity is drawn in f32 and rounded to f16, so the oracle (which
holds all values as f32, like the reference's CPU backend) and the GPU see the
same numbers."""
import numpy as np

from oracle import quant_oracle as O


def rel_l2(got, want) -> float:
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))


def per_row_err(got, want) -> float:
    """The reference probe's bar: max |d| / max(1, |ref|) (probe-quant-gemv.ts:166-187)."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    return float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want)))) if got.size else 0.0


def f16_round(a):
    return np.asarray(a, np.float32).astype(np.float16)


def make_weight(fmt: str, n: int, k: int, g: int, rng):
    """Returns (packed u32, scales array, dequantised f32 [n,k] from the oracle)."""
    if fmt == "int4-grouped":
        q = rng.integers(-8, 8, (n, k)).astype(np.int8)
        packed = O.np_pack_int4(q)
        scales = f16_round(rng.uniform(0.01, 0.05, n * (k // g))).view(np.uint16)
        deq = O.dequant_int4_grouped(packed, scales, n, k, g)
    elif fmt == "int8-row":
        q = rng.integers(-127, 128, (n, k)).astype(np.int8)
        packed = O.np_pack_int8(q)
        scales = rng.uniform(0.005, 0.02, n).astype(np.float32)
        deq = O.dequant_int8_row(packed, scales, n, k)
    elif fmt == "int8-grouped":
        w = (rng.random((n, k)) * 2 - 1).astype(np.float32)
        packed, scales = O.quantize_int8_grouped(w, n, k, g)
        deq = O.dequant_int8_grouped(packed, scales, n, k, g)
    else:
        raise ValueError(fmt)
    return packed, scales, deq


def make_x(m: int, k: int, dtype: str, rng, std: float = 1.0):
    x = (rng.standard_normal((m, k)) * std).astype(np.float32)
    if dtype == "f16":
        x = f16_round(x)
    return x


def fmt_name(fmt: str, g: int) -> str:
    return {"int4-grouped": f"int4-{g}", "int8-grouped": f"int8-{g}", "int8-row": "int8-row"}[fmt]
