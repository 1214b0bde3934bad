"""The `hip` backend for torchlette's quantized-weight linear path, host side.

A Python mirror — same names, argument meaning and error behaviour — of the part
of torchlette's backend interface this path touches, over the C ABI of
``include/tlhip.h``:

=====================================  =========================================
here                                   reference (torchlette source tree)
=====================================  =========================================
``StorageFormat``, ``QuantPacking``,   src/backend/types.ts:30-67
``resolveWeightFormat``
``HipTensor`` (a ``BackendTensor``)    src/backend/types.ts:5-28;
                                       src/backend/webgpu/gpu-types.ts:143-158
``quantizeLinearWeight``,              src/backend/quantize.ts:77-156
``dequantizeToF32``
``HipBackend.createQuantizedWeight``   src/runtime/engine.ts:2041-2149
``ops.tensorFromArray``                src/backend/webgpu/ops/creation.ts:51-87
``ops.transpose / permute``            src/backend/webgpu/ops/views.ts:917-934
``ops.matmul`` (the format seam)       src/backend/webgpu/ops/matmul-ops.ts:42-182
``ops.add / relu / silu / gelu /       src/backend/types.ts:340-679 (BackendOps)
cast / read``
``HipBackend.linear``                  src/frontend/torchlette.ts:878-894
``pretuneMatmulShapes``                src/backend/types.ts:688
dispatch counters                      src/backend/webgpu/matmul/dispatch.ts:79-83,
                                       832-864, 943-947
=====================================  =========================================

numpy is used only to carry bytes between the host and the device.  All
arithmetic of the path runs in the HIP kernels; nothing here computes on the
CPU, and a missing ``libtlhip.so`` or GPU raises.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from . import _lib as L

DTYPES = {"f32": np.float32, "f16": np.float16, "u32": np.uint32, "i32": np.int32}
_DT_CODE = {"f32": L.F32, "f16": L.F16}


# ---------------------------------------------------------------- format axis

@dataclass(frozen=True)
class QuantPacking:
    """types.ts:46-55.  ``scheme`` is "int8-grouped" (the reference's), or one
    of the two values this backend adds on the same axis: "int4-grouped"
    (docs/quantization-design.md:69-75) and "int8-row" (one f32 scale per
    output row)."""
    scheme: str
    groupSize: int
    scalesDtype: str = "f16"


@dataclass(frozen=True)
class StorageFormat:
    """types.ts:38-43.  Plain dtype = no ``packing``."""
    elementType: str
    packing: Optional[QuantPacking] = None


_SCHEMES = {"int8-grouped": L.FMT_INT8_GROUPED, "int8-row": L.FMT_INT8_ROW,
            "int4-grouped": L.FMT_INT4_GROUPED}


def resolveWeightFormat(name: str, elementType: str = "f16") -> StorageFormat:
    """types.ts:58-67 for "int8-64" / "int8-128" (any "int8-<G>" is accepted);
    plus "int4-<G>" and "int8-row"."""
    if name.startswith("int8-") and name[5:].isdigit():
        return StorageFormat(elementType, QuantPacking("int8-grouped", int(name[5:]), "f16"))
    if name.startswith("int4-") and name[5:].isdigit():
        return StorageFormat(elementType, QuantPacking("int4-grouped", int(name[5:]), "f16"))
    if name == "int8-row":
        return StorageFormat(elementType, QuantPacking("int8-row", 0, "f32"))
    raise ValueError(f"unknown weight format {name}")


# -------------------------------------------------------------------- tensors

def _strides_for(shape: Sequence[int]) -> List[int]:
    st, acc = [], 1
    for d in reversed(shape):
        st.append(acc)
        acc *= d
    return list(reversed(st))


class HipTensor:
    """BackendTensor over a device allocation (types.ts:5-28)."""

    def __init__(self, backend: "HipBackend", shape, dtype: str, ptr: int, nbytes: int,
                 ownsBuffer: bool = True, strides=None, format: Optional[StorageFormat] = None,
                 scales: Optional["HipTensor"] = None, base: Optional["HipTensor"] = None):
        self._backend = backend
        self.shape = list(shape)
        self.dtype = dtype
        self.ptr = ptr
        self.nbytes = nbytes
        self.ownsBuffer = ownsBuffer
        self.strides = list(strides) if strides is not None else _strides_for(shape)
        self.format = format
        self.scales = scales
        self._base = base  # keeps the owner alive for views
        self._destroyed = False

    @property
    def size(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    @property
    def isContiguous(self) -> bool:
        return self.strides == _strides_for(self.shape)

    def toArray(self) -> list:
        return self._backend.ops.read(self)

    def numpy(self) -> np.ndarray:
        return self._backend._download(self)

    def destroy(self) -> None:
        """Idempotent (src/backend/webgpu/tensor.ts:71-73)."""
        if self._destroyed:
            return
        self._destroyed = True
        if self.ownsBuffer and self.ptr:
            L.call("tlhip_free", self.ptr)
        self.ptr = 0


# ------------------------------------------------------------ host quantizer

def quantizeLinearWeight(weight, n: int, k: int, groupSize: int = 64):
    """quantize.ts:77-131, run by the native host routine of the library.
    Returns (packed u32[n*k/4], scales u16[n*k/groupSize])."""
    w = np.ascontiguousarray(weight, np.float32).ravel()
    if w.size != n * k:
        raise L.TlhipError(1, f"quantize: expected {n * k} elements, got {w.size}")
    packed = np.zeros(max(n * k // 4, 0), np.uint32)
    scales = np.zeros(n * k // groupSize if groupSize > 0 and k % max(groupSize, 1) == 0 else 0, np.uint16)
    L.call("tlhip_quantize_int8_grouped", w.ctypes.data, n, k, groupSize, packed.ctypes.data,
           scales.ctypes.data)
    return packed, scales


def f32ToF16Bits(value: float) -> int:
    return int(L.load().tlhip_f32_to_f16_bits(float(np.float32(value))))


def f16BitsToF32(bits: int) -> float:
    return float(L.load().tlhip_f16_bits_to_f32(int(bits) & 0xFFFF))


# -------------------------------------------------------------------- backend

class _Ops:
    """BackendOps subset for the Linear path."""

    def __init__(self, backend: "HipBackend"):
        self._b = backend

    # creation / readback -------------------------------------------------
    def tensorFromArray(self, values, shape, dtype: str = "f32") -> HipTensor:
        """creation.ts:51-87.  ``values`` may be numbers, or raw f16 bit
        patterns as a uint16 array when dtype is "f16" (creation.ts:368-414)."""
        if dtype not in DTYPES:
            raise ValueError(f"unsupported dtype {dtype}")
        arr = np.asarray(values)
        if dtype == "f16" and arr.dtype == np.uint16:
            host = np.ascontiguousarray(arr).view(np.float16)
        else:
            host = np.ascontiguousarray(arr, DTYPES[dtype])
        n = 1
        for d in shape:
            n *= d
        if host.size != n:
            raise ValueError("Tensor data length does not match shape")
        return self._b._upload(host.reshape(-1), list(shape), dtype)

    def zeros(self, shape, dtype: str = "f32") -> HipTensor:
        t = self._b._alloc(list(shape), dtype)
        if t.nbytes:
            L.call("tlhip_memset", t.ptr, 0, t.nbytes, self._b.stream)
        return t

    def read(self, a: HipTensor) -> list:
        return self._b._download(a).ravel().tolist()

    # views ---------------------------------------------------------------
    def permute(self, a: HipTensor, dims: Sequence[int]) -> HipTensor:
        """A view; copies ``format`` and ``scales`` (views.ts:925-934)."""
        rank = len(a.shape)
        dims = [d % rank for d in dims]
        return HipTensor(self._b, [a.shape[d] for d in dims], a.dtype, a.ptr, a.nbytes, False,
                         [a.strides[d] for d in dims], a.format, a.scales, a)

    def transpose(self, a: HipTensor, options=None, dim0: int = -2, dim1: int = -1) -> HipTensor:
        if options:
            dim0, dim1 = options.get("dim0", dim0), options.get("dim1", dim1)
        dims = list(range(len(a.shape)))
        dims[dim0], dims[dim1] = dims[dim1], dims[dim0]
        return self.permute(a, dims)

    def reshape(self, a: HipTensor, shape) -> HipTensor:
        if not a.isContiguous:
            raise NotImplementedError("reshape of a non-contiguous hip tensor")
        n = 1
        for d in shape:
            n *= d
        if n != a.size:
            raise ValueError("View shape does not match tensor size")
        return HipTensor(self._b, shape, a.dtype, a.ptr, a.nbytes, False, None, a.format, a.scales, a)

    def contiguous(self, a: HipTensor) -> HipTensor:
        if a.isContiguous:
            return a
        raise NotImplementedError("materialising a strided hip tensor is outside this path")

    # the seam ------------------------------------------------------------
    def matmul(self, a: HipTensor, b: HipTensor, options=None) -> HipTensor:
        """matmul-ops.ts:42-59: a packed B operand goes to matmulQuantizedB."""
        if b.format is not None and b.format.packing is not None:
            return self._b._matmulQuantizedB(a, b, None)
        raise NotImplementedError(
            "hip backend: dense matmul is outside the quantized-weight linear path")

    # unfused neighbours of the matmul --------------------------------------
    def add(self, a: HipTensor, b: HipTensor) -> HipTensor:
        """Only the Linear bias case: b is [N] (or [1,N]) broadcast over a's rows."""
        n = a.shape[-1]
        if b.size != n or a.dtype not in _DT_CODE or b.dtype not in _DT_CODE or not a.isContiguous:
            raise NotImplementedError("hip backend add: only a[...,N] + bias[N]")
        out = self._b._alloc(a.shape, a.dtype)
        L.call("tlhip_bias_add", a.ptr, _DT_CODE[a.dtype], b.ptr, _DT_CODE[b.dtype], out.ptr,
               a.size // n if n else 0, n, self._b.stream)
        return out

    def _unary(self, name: str, a: HipTensor) -> HipTensor:
        if a.dtype not in _DT_CODE or not a.isContiguous:
            raise NotImplementedError(f"hip backend {name}: contiguous f32/f16 only")
        out = self._b._alloc(a.shape, a.dtype)
        L.call("tlhip_unary", L.UNARY[name], a.ptr, _DT_CODE[a.dtype], out.ptr, a.size, self._b.stream)
        return out

    def relu(self, a):
        return self._unary("relu", a)

    def silu(self, a):
        return self._unary("silu", a)

    def sigmoid(self, a):
        return self._unary("sigmoid", a)

    def tanh(self, a):
        return self._unary("tanh", a)

    def gelu(self, a, options=None):
        """CPU backend default is the tanh form (src/backend/cpu/numeric.ts:626-630)."""
        approximate = (options or {}).get("approximate", "tanh")
        return self._unary("gelu_tanh" if approximate == "tanh" else "gelu_erf", a)

    def mul(self, a: HipTensor, b: HipTensor) -> HipTensor:
        """Elementwise product of two tensors of one shape and dtype (the MLP's
        `mul(act(gate), up)`, packages/qwen3-browser/src/model.ts:357-361)."""
        return self.gatedMul(a, b, "none")

    def gatedMul(self, gate: HipTensor, up: HipTensor, activation: str = "silu") -> HipTensor:
        """`mul(activation(gate), up)` in one pass."""
        if (gate.dtype not in _DT_CODE or gate.dtype != up.dtype or list(gate.shape) != list(up.shape)
                or not gate.isContiguous or not up.isContiguous):
            raise NotImplementedError("hip backend mul: two contiguous f32/f16 tensors of one shape")
        act = "gelu_tanh" if activation == "gelu" else activation
        out = self._b._alloc(gate.shape, gate.dtype)
        L.call("tlhip_gated_mul", L.UNARY[act], gate.ptr, up.ptr, _DT_CODE[gate.dtype], out.ptr, gate.size,
               self._b.stream)
        return out

    def fusedRMSNormForward(self, x: HipTensor, weight: HipTensor, config: dict,
                            outDtype: Optional[str] = None) -> HipTensor:
        """BackendOps.fusedRMSNormForward (src/backend/types.ts:635-640): x [N,D],
        weight f32 [D], config {numRows, featureDim, eps}."""
        rows, d, eps = int(config["numRows"]), int(config["featureDim"]), float(config["eps"])
        if x.dtype not in _DT_CODE or weight.dtype != "f32" or not x.isContiguous:
            raise NotImplementedError("hip backend rmsnorm: contiguous f32/f16 x, f32 weight")
        if x.size != rows * d or weight.size != d:
            raise ValueError("fusedRMSNormForward: shape mismatch")
        out_dtype = outDtype or x.dtype
        out = self._b._alloc(x.shape, out_dtype)
        L.call("tlhip_rmsnorm", x.ptr, _DT_CODE[x.dtype], weight.ptr, out.ptr, _DT_CODE[out_dtype], rows, d, eps,
               self._b.stream)
        return out

    def cast(self, a: HipTensor, dtype: str) -> HipTensor:
        if a.dtype == dtype:
            return a
        if a.dtype not in _DT_CODE or dtype not in _DT_CODE or not a.isContiguous:
            raise NotImplementedError("hip backend cast: f32 <-> f16 only")
        out = self._b._alloc(a.shape, dtype)
        L.call("tlhip_cast", a.ptr, _DT_CODE[a.dtype], out.ptr, _DT_CODE[dtype], a.size, self._b.stream)
        return out


class HipBackend:
    """Backend {name, ops, pretuneMatmulShapes} (types.ts:681-696) for "hip"."""

    name = "hip"

    def __init__(self, device_index: int = 0):
        L.call("tlhip_init", device_index)
        self.stream = None  # the library stream
        self.ops = _Ops(self)
        self._state: list = []  # registerState: persistent weights are never recycled

    # plumbing ------------------------------------------------------------
    def _alloc(self, shape, dtype: str) -> HipTensor:
        n = 1
        for d in shape:
            n *= d
        nbytes = n * np.dtype(DTYPES[dtype]).itemsize
        p = C.c_void_p()
        L.call("tlhip_malloc", nbytes, C.byref(p))
        return HipTensor(self, shape, dtype, p.value or 0, nbytes)

    def _upload(self, host: np.ndarray, shape, dtype: str) -> HipTensor:
        t = self._alloc(shape, dtype)
        if t.nbytes:
            L.call("tlhip_memcpy_h2d", t.ptr, host.ctypes.data, t.nbytes, self.stream)
            L.call("tlhip_stream_synchronize", self.stream)  # host buffer may be freed by the caller
        return t

    def _download(self, t: HipTensor) -> np.ndarray:
        if t.format is not None and t.format.packing is not None:
            raise ValueError("a packed weight must be dequantised explicitly before it is read")
        if not t.isContiguous:
            raise NotImplementedError("read of a strided hip tensor")
        host = np.empty(t.size, DTYPES[t.dtype])
        if t.nbytes:
            L.call("tlhip_memcpy_d2h", host.ctypes.data, t.ptr, t.nbytes, self.stream)
        L.call("tlhip_stream_synchronize", self.stream)
        return host.reshape(t.shape)

    def _download_raw(self, t: HipTensor, count: int, dtype) -> np.ndarray:
        """The first `count` elements of t's buffer as `dtype`, whatever t's logical view
        says (the packed words or scale bits of a quantized weight, for the loader's cache)."""
        host = np.empty(count, dtype)
        if host.nbytes > t.nbytes:
            raise ValueError("_download_raw: more bytes than the buffer holds")
        if host.nbytes:
            L.call("tlhip_memcpy_d2h", host.ctypes.data, t.ptr, host.nbytes, self.stream)
        L.call("tlhip_stream_synchronize", self.stream)
        return host

    def synchronize(self) -> None:
        L.call("tlhip_stream_synchronize", self.stream)

    def deviceInfo(self) -> dict:
        info = L.DeviceInfo()
        L.call("tlhip_device_info", C.byref(info))
        return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes) else getattr(info, f))
                for f, _ in info._fields_}

    # weights -------------------------------------------------------------
    def createQuantizedWeight(self, packed, scalesBits, n: int, k: int, format: StorageFormat) -> HipTensor:
        """engine.ts:2041-2149: validate, upload packed u32 and the scales,
        present the logical [N,K] tensor with ``format`` and ``scales`` set.
        For "int8-row" ``scalesBits`` is the f32 per-row scale vector."""
        packing = format.packing
        if packing is None:
            raise ValueError("createQuantizedWeight: format.packing is required")
        if packing.scheme not in _SCHEMES:
            raise ValueError(f"createQuantizedWeight: unsupported scheme {packing.scheme}")
        per_word = 8 if packing.scheme == "int4-grouped" else 4
        if k % per_word != 0:
            raise ValueError(f"createQuantizedWeight: K={k} must be divisible by {per_word}")
        packed = np.ascontiguousarray(packed, np.uint32).ravel()
        wordsPerRow = k // per_word
        if packed.size != n * wordsPerRow:
            raise ValueError(f"createQuantizedWeight: packed length {packed.size} != {n * wordsPerRow}")
        if packing.scheme == "int8-row":
            scales_host = np.ascontiguousarray(scalesBits, np.float32).ravel()
            want, sdtype = n, "f32"
        else:
            if packing.groupSize <= 0 or k % packing.groupSize != 0:
                raise ValueError(
                    f"createQuantizedWeight: K={k} must be divisible by groupSize={packing.groupSize}")
            scales_host = np.ascontiguousarray(scalesBits, np.uint16).ravel()
            want, sdtype = n * (k // packing.groupSize), "f16"
        if scales_host.size != want:
            raise ValueError(f"createQuantizedWeight: scales length {scales_host.size} != {want}")
        packedT = self._upload(packed, [n, wordsPerRow], "u32")
        scalesT = self._upload(scales_host.view(np.float16) if sdtype == "f16" else scales_host,
                               [want], sdtype)
        logical = HipTensor(self, [n, k], format.elementType, packedT.ptr, packedT.nbytes, False,
                            [k, 1], format, scalesT, packedT)
        self._state.extend([packedT, scalesT, logical])
        return logical

    def quantizeLinearWeightOnDevice(self, weight: HipTensor, groupSize: int = 64,
                                     elementType: str = "f32") -> HipTensor:
        """quantizeLinearWeight (quantize.ts:77-131) for a weight that is already
        on the device (quantize-at-load, examples/qwen3/loader.ts:228-254): f32
        [N,K] in, the logical packed [N,K] weight with ``format`` and ``scales``
        out, bit-identical to the host quantizer followed by
        ``createQuantizedWeight``."""
        if weight.dtype != "f32" or len(weight.shape) != 2 or not weight.isContiguous:
            raise ValueError("quantizeLinearWeightOnDevice: weight must be a contiguous f32 [N,K] tensor")
        n, k = weight.shape
        if k % 4 != 0:
            raise ValueError(f"quantizeLinearWeight: K={k} must be divisible by 4")
        if groupSize <= 0 or k % groupSize != 0:
            raise ValueError(f"quantizeLinearWeight: K={k} must be divisible by groupSize={groupSize}")
        packedT = self._alloc([n, k // 4], "u32")
        scalesT = self._alloc([n * (k // groupSize)], "f16")
        L.call("tlhip_quantize_int8_grouped_device", weight.ptr, n, k, groupSize, packedT.ptr, scalesT.ptr,
               self.stream)
        fmt = StorageFormat(elementType, QuantPacking("int8-grouped", groupSize))
        logical = HipTensor(self, [n, k], elementType, packedT.ptr, packedT.nbytes, False, [k, 1], fmt,
                            scalesT, packedT)
        self._state.extend([packedT, scalesT, logical])
        return logical

    def readTopK(self, a: HipTensor, k: int, offset: int = 0, length: Optional[int] = None):
        """types.ts:669-678: the top-k (values descending, ties to the smaller index)
        of a contiguous f32 tensor (or of [offset, offset+length) of it), selected on
        the device; only 2k numbers are read back."""
        if a.dtype != "f32" or not a.isContiguous:
            raise ValueError("readTopK: a contiguous f32 tensor")
        length = a.size - offset if length is None else length
        if offset < 0 or length < 0 or offset + length > a.size:
            raise ValueError("readTopK: range outside the tensor")
        vals, idx = self._alloc([k], "f32"), self._alloc([k], "i32")
        L.call("tlhip_topk", a.ptr, offset, length, k, vals.ptr, idx.ptr, L.I32, self.stream)
        v, i = self._download(vals), self._download(idx)
        vals.destroy()
        idx.destroy()
        return v, i

    def deviceTopK(self, logits: HipTensor, k: int) -> HipTensor:
        """types.ts:632-634: [.., V] -> packed [1, 2, k] on the device, row 0 the
        values (descending), row 1 the token ids as f32."""
        if logits.dtype != "f32" or not logits.isContiguous:
            raise ValueError("deviceTopK: a contiguous f32 logits row")
        out = self._alloc([1, 2, k], "f32")
        L.call("tlhip_topk", logits.ptr, 0, logits.size, k, out.ptr, out.ptr + 4 * k, L.F32, self.stream)
        return out

    def dequantizeToF32(self, w: HipTensor) -> HipTensor:
        """Explicit dequant of a packed weight to f32 [N,K] on the device
        (quantize.ts:138-156; matmul/dispatch.ts:949-1037)."""
        qw = self._qweight(w, transposed=False)
        out = self._alloc([qw.n, qw.k], "f32")
        L.call("tlhip_dequant", C.byref(qw), out.ptr, self.stream)
        return out

    def _qweight(self, w: HipTensor, transposed: bool) -> L.QWeight:
        packing = w.format.packing if w.format else None
        scales = w.scales
        if packing is None or scales is None:
            raise ValueError("matmulQuantizedB: missing packing/scales on B operand")
        if packing.scheme not in _SCHEMES:
            raise ValueError(f"matmulQuantizedB: unsupported scheme {packing.scheme}")
        if transposed:
            k, n = w.shape[-2], w.shape[-1]
            if w.strides[-2:] != [1, k]:
                raise ValueError("matmulQuantizedB: B must be the transposed view of a [N,K] packed weight")
        else:
            n, k = w.shape[-2], w.shape[-1]
        return L.QWeight(_SCHEMES[packing.scheme], packing.groupSize, n, k, w.ptr, scales.ptr)

    # the seam ------------------------------------------------------------
    def _matmulQuantizedB(self, a: HipTensor, b: HipTensor, epilogue: Optional[L.Epilogue],
                          config: Optional[L.KernelConfig] = None) -> HipTensor:
        """matmul-ops.ts:113-182.  B arrives as the transposed [K,N] view of the
        logical [N,K] weight; A is [..., M, K].  Leading dimensions of A are
        folded into M (the weight is shared across them)."""
        qw = self._qweight(b, transposed=True)
        if a.dtype not in _DT_CODE:
            raise ValueError(f"matmulQuantizedB: unsupported activation dtype {a.dtype}")
        if not a.shape or a.shape[-1] != qw.k:
            raise ValueError("matmul dimension mismatch")
        if not a.isContiguous:
            raise NotImplementedError("matmulQuantizedB: strided activations")
        lead = a.shape[:-1] if len(a.shape) > 1 else [1]
        m = 1
        for d in lead:
            m *= d
        # f16 out only when activations and the weight's element type are both f16
        # (dense rule, src/backend/webgpu/matmul/gemv.ts:27-29)
        out_dtype = "f16" if (a.dtype == "f16" and b.format.elementType == "f16") else "f32"
        out_shape = (a.shape[:-1] if len(a.shape) > 1 else []) + [qw.n]
        if len(a.shape) == 1:
            out_shape = [qw.n]
        for size in getattr(epilogue, "_binary_sizes", []):
            if size != m * qw.n:
                raise ValueError(f"a binary epilogue input must be an [M,N] = [{m},{qw.n}] tensor")
        out = self._alloc(out_shape, out_dtype)
        ep = C.byref(epilogue) if epilogue is not None else None
        if config is None:
            L.call("tlhip_matmul_quantized", C.byref(qw), a.ptr, _DT_CODE[a.dtype], m, out.ptr,
                   _DT_CODE[out_dtype], 1.0, ep, self.stream)
        else:
            L.call("tlhip_matmul_quantized_config", C.byref(qw), a.ptr, _DT_CODE[a.dtype], m, out.ptr,
                   _DT_CODE[out_dtype], 1.0, ep, C.byref(config), self.stream)
        return out

    @staticmethod
    def makeEpilogue(bias: Optional[HipTensor] = None, activation: Optional[str] = None,
                     binary: Optional[Sequence] = None) -> L.Epilogue:
        """EpilogueConfig {ops: [bias?, unary?, binary?]} (matmul/types.ts:13-24); `binary` is
        (op, tensor) with op in add / sub / mul and an [M,N] tensor (a residual, a gate)."""
        return HipBackend.makeEpilogueChain(([("bias", bias)] if bias is not None else []) +
                                            ([("unary", activation)] if activation and activation != "none" else []) +
                                            ([("binary",) + tuple(binary)] if binary is not None else []))

    @staticmethod
    def makeEpilogueChain(ops: Sequence[Sequence]) -> L.Epilogue:
        """EpilogueConfig.ops in the caller's order: ("bias", tensor[N]), ("unary", name),
        ("binary", op, tensor[M,N]), ("cast", "f16") (matmul-skeleton.ts:916-966)."""
        if len(ops) > L.MAX_EPILOGUE_OPS:
            raise ValueError(f"at most {L.MAX_EPILOGUE_OPS} epilogue ops")
        ep = L.Epilogue()
        binary_sizes = []   # checked against M * N at the call: the kernels index these inputs by output element
        for i, op in enumerate(ops):
            if op[0] == "bias":
                ep.ops[i] = L.EpilogueOp(L.EPI_BIAS, 0, op[1].ptr, _DT_CODE[op[1].dtype], 1 if len(op[1].shape) <= 1 else op[1].size // op[1].shape[-1])
            elif op[0] == "unary":
                ep.ops[i] = L.EpilogueOp(L.EPI_UNARY, L.UNARY[op[1]], None, 0, 0)
            elif op[0] == "binary":
                if op[1] not in L.BINARY:
                    raise ValueError(f"Unsupported binary epilogue: {op[1]}")
                if not op[2].isContiguous:
                    raise ValueError("a binary epilogue input must be contiguous")
                ep.ops[i] = L.EpilogueOp(L.EPI_BINARY, L.BINARY[op[1]], op[2].ptr, _DT_CODE[op[2].dtype],
                                         op[2].size // op[2].shape[-1] if op[2].shape and op[2].shape[-1] else 0)
                binary_sizes.append(op[2].size)
            elif op[0] == "cast":
                ep.ops[i] = L.EpilogueOp(L.EPI_CAST_F16 if op[1] == "f16" else L.EPI_NONE, 0, None, 0, 0)
            else:
                raise ValueError(f"unknown epilogue op {op[0]}")
        ep.n_ops = len(ops)
        ep._binary_sizes = binary_sizes
        return ep

    def linear(self, input: HipTensor, weight: HipTensor, bias: Optional[HipTensor] = None,
               activation: Optional[str] = None, fused: bool = False,
               config: Optional[L.KernelConfig] = None) -> HipTensor:
        """api.linear (torchlette.ts:878-894): transpose view, matmul, add.
        ``fused=False`` issues the ops one by one as a plain Backend receives
        them; ``fused=True`` hands bias/activation to the kernel epilogue (what
        the fused side door would do for a matmul -> bias -> activation chain)."""
        wT = self.ops.transpose(weight)
        if fused:
            ep = self.makeEpilogue(bias, activation)
            return self._matmulQuantizedB(input, wT, ep, config)
        y = self._matmulQuantizedB(input, wT, None, config) if config is not None else self.ops.matmul(input, wT)
        if bias is not None:
            y2 = self.ops.add(y, bias)
            y.destroy()
            y = y2
        if activation and activation != "none":
            y2 = self.ops._unary("gelu_tanh" if activation == "gelu" else activation, y)
            y.destroy()
            y = y2
        return y

    def linearGrouped(self, input: HipTensor, weights: Sequence[HipTensor],
                      biases: Optional[Sequence[Optional[HipTensor]]] = None,
                      activation: Optional[str] = None, _prologue: Optional[L.Prologue] = None) -> List[HipTensor]:
        """Up to four decode Linears on the same activations (q/k/v, or gate/up) in
        one launch: the results of ``[linear(input, w, b, activation, fused=True)
        for w, b in zip(weights, biases)]``.  f16 activations, at most 16 rows (with a
        prologue: one row)."""
        if not 1 <= len(weights) <= 4:
            raise ValueError("linearGrouped: a group holds 1..4 weights")
        biases = list(biases) if biases is not None else [None] * len(weights)
        qws = [self._qweight(w, transposed=False) for w in weights]
        m = input.size // qws[0].k
        if input.dtype != "f16" or not 1 <= m <= 16 or (m != 1 and _prologue is not None):
            raise ValueError("linearGrouped: f16 activations, 1..16 rows (one row with a prologue)")
        out_dtype = "f16" if all(w.format.elementType == "f16" for w in weights) else "f32"
        outs = [self._alloc(list(input.shape[:-1]) + [qw.n], out_dtype) for qw in qws]
        eps = [self.makeEpilogue(b, activation) for b in biases]
        probs = (L.GemvProblem * len(weights))()
        for i, (qw, o, ep) in enumerate(zip(qws, outs, eps)):
            probs[i].w = qw
            probs[i].x = input.ptr
            probs[i].y = o.ptr
            probs[i].epilogue = C.pointer(ep) if ep is not None else None
        if _prologue is not None:
            L.call("tlhip_gemv_grouped_prologue", probs, len(weights), C.byref(_prologue), _DT_CODE[input.dtype],
                   _DT_CODE[out_dtype], 1.0, self.stream)
        else:
            L.call("tlhip_gemv_grouped_rows", probs, len(weights), _DT_CODE[input.dtype], m, _DT_CODE[out_dtype], 1.0,
                   self.stream)
        return outs

    # several Linears in one launch ------------------------------------------
    def linearSequence(self, steps: Sequence[dict]) -> List[HipTensor]:
        """A sequence of decode Linears as ONE launch (tlhip_gemv_sequence).  Each step is a
        dict: ``input`` (HipTensor [m, K] f16), ``weight``, optional ``up`` (a second weight:
        the step computes ``act(input w^T) * (input up^T)``), ``bias``, ``activation``,
        ``binary`` ((op, tensor[m, N])), ``wait`` (the step reads what an earlier step of the
        call writes), ``out`` (an existing tensor to write, e.g. one a later step reads).
        Returns the outputs in order."""
        if not 1 <= len(steps) <= 16:
            raise ValueError("linearSequence: 1..16 steps")
        arr = (L.SequenceStep * len(steps))()
        outs, keep = [], []
        m = None
        for i, st in enumerate(steps):
            x, w = st["input"], st["weight"]
            qw = self._qweight(w, transposed=False)
            if x.dtype != "f16" or not x.isContiguous or x.shape[-1] != qw.k:
                raise ValueError("linearSequence: activations must be contiguous [m, K] f16")
            mi = x.size // qw.k
            if m is None:
                m = mi
            if mi != m or not 1 <= m <= 16:
                raise ValueError("linearSequence: every step takes the same 1..16 rows")
            out_dtype = "f16" if w.format.elementType == "f16" else "f32"
            out = st.get("out")
            if out is None:
                out = self._alloc(list(x.shape[:-1]) + [qw.n], out_dtype)
            elif out.size != m * qw.n or not out.isContiguous:
                raise ValueError("linearSequence: out must be a contiguous [m, N] tensor")
            ep = self.makeEpilogue(st.get("bias"), st.get("activation"), st.get("binary"))
            if any(sz != m * qw.n for sz in ep._binary_sizes):
                raise ValueError("a binary epilogue input must hold M*N elements")
            keep.append(ep)
            arr[i].w = qw
            if st.get("up") is not None:
                arr[i].w_up = self._qweight(st["up"], transposed=False)
                arr[i].gated = 1
            arr[i].x = x.ptr
            arr[i].y = out.ptr
            arr[i].epilogue = C.pointer(ep)
            arr[i].y_dtype = _DT_CODE[out.dtype]
            arr[i].wait = 1 if st.get("wait") else 0
            outs.append(out)
        L.call("tlhip_gemv_sequence", arr, len(steps), L.F16, m, 1.0, self.stream)
        return outs

    def mlpDecode(self, input: HipTensor, gate: HipTensor, up: HipTensor, down: HipTensor,
                  activation: str = "silu", oneLaunch: bool = False) -> HipTensor:
        """down(act(gate(x)) * up(x)) (packages/qwen3-browser/src/model.ts:357-361) from one
        call: tlhip_mlp_decode, which runs the faster form (today the three launches the model
        issues); oneLaunch=True asks for the sequence launch (a gated step and the down
        projection waiting for it, int4 weights in groups of 32 only)."""
        qg, qu, qd = (self._qweight(w, transposed=False) for w in (gate, up, down))
        if input.dtype != "f16" or not input.isContiguous or input.shape[-1] != qg.k:
            raise ValueError("mlpDecode: activations must be contiguous [m, K] f16")
        m = input.size // qg.k
        h = self._alloc([m, qg.n], "f16")
        act = "gelu_tanh" if activation == "gelu" else activation
        try:
            if oneLaunch:
                return self.linearSequence([{"input": input, "weight": gate, "up": up, "activation": act, "out": h},
                                            {"input": h, "weight": down, "wait": True}])[1]
            out_dtype = "f16" if down.format.elementType == "f16" else "f32"
            y = self._alloc(list(input.shape[:-1]) + [qd.n], out_dtype)
            L.call("tlhip_mlp_decode", C.byref(qg), C.byref(qu), C.byref(qd), L.UNARY[act], input.ptr, L.F16, m, h.ptr,
                   y.ptr, _DT_CODE[out_dtype], None, self.stream)
            return y
        finally:
            h.destroy()  # tlhip_free waits for the device: the launch that reads h is over by then

    def sequenceStatus(self) -> int:
        """Waits for the stream; raises if a sequence launch gave up a wait."""
        err = C.c_int()
        L.call("tlhip_sequence_status", self.stream, C.byref(err))
        return err.value

    # the producers of a decode Linear's input, fused into its GEMV ------------
    def _prologue(self, kind: int, operand: HipTensor, activation: str = "none", eps: float = 0.0) -> L.Prologue:
        act = "gelu_tanh" if activation == "gelu" else activation
        return L.Prologue(kind, L.UNARY[act], eps, 0, operand.ptr)

    # Every workgroup of the GEMV forms f(x) for itself, so the fused form costs M * K
    # extra work per workgroup: measured on MI355X it beats the separate launch (about
    # 3 us inside a HIP graph) for one or two activation rows and loses from three on.
    fusedPrologueMaxRows = 2

    def _linearWithPrologue(self, input: HipTensor, pro: L.Prologue, weight: HipTensor,
                            bias: Optional[HipTensor], activation: Optional[str]) -> Optional[HipTensor]:
        """One fused launch, or None when no built kernel covers the request (or the
        separate launches are faster)."""
        qw = self._qweight(weight, transposed=False)
        if input.dtype not in _DT_CODE or not input.isContiguous or input.shape[-1] != qw.k:
            raise ValueError("linear: activations must be contiguous [..., K] of f32/f16")
        m = input.size // qw.k if qw.k else 0
        if m > self.fusedPrologueMaxRows:
            return None
        out_dtype = "f16" if (input.dtype == "f16" and weight.format.elementType == "f16") else "f32"
        out = self._alloc(list(input.shape[:-1]) + [qw.n], out_dtype)
        ep = self.makeEpilogue(bias, activation)
        rc = L.load().tlhip_gemv_prologue(C.byref(qw), C.byref(pro), input.ptr, _DT_CODE[input.dtype], m, out.ptr,
                                         _DT_CODE[out_dtype], 1.0, C.byref(ep), self.stream)
        if rc == L.ERR_UNSUPPORTED:
            out.destroy()
            return None
        L.check(rc)
        return out

    def linearAfterRMSNorm(self, input: HipTensor, normWeight: HipTensor, eps: float, weight: HipTensor,
                           bias: Optional[HipTensor] = None, activation: Optional[str] = None) -> HipTensor:
        """`linear(rmsnorm(input, normWeight, eps), weight, bias)` (+ activation): the
        norm is applied while the GEMV stages its activations when a fused kernel
        covers the shape (M <= 4), else as its own launch."""
        if normWeight.dtype != "f32" or normWeight.size != input.shape[-1]:
            raise ValueError("linearAfterRMSNorm: norm weight must be f32 [K]")
        out = self._linearWithPrologue(input, self._prologue(L.PRO_RMSNORM, normWeight, eps=eps), weight, bias,
                                       activation)
        if out is not None:
            return out
        d = input.shape[-1]
        normed = self.ops.fusedRMSNormForward(input, normWeight, {"numRows": input.size // d, "featureDim": d,
                                                                  "eps": eps})
        out = self.linear(normed, weight, bias, activation, fused=True)
        normed.destroy()
        return out

    def linearAfterGatedMul(self, gate: HipTensor, up: HipTensor, gateActivation: str, weight: HipTensor,
                            bias: Optional[HipTensor] = None, activation: Optional[str] = None) -> HipTensor:
        """`linear(mul(gateActivation(gate), up), weight, bias)`: the MLP's down
        projection with its input formed while the GEMV stages it (M <= 4)."""
        if gate.dtype != up.dtype or list(gate.shape) != list(up.shape) or not up.isContiguous:
            raise ValueError("linearAfterGatedMul: gate and up must share shape and dtype")
        out = self._linearWithPrologue(gate, self._prologue(L.PRO_GATED_MUL, up, gateActivation), weight, bias,
                                       activation)
        if out is not None:
            return out
        x = self.ops.gatedMul(gate, up, gateActivation)
        out = self.linear(x, weight, bias, activation, fused=True)
        x.destroy()
        return out

    def linearGroupedAfterRMSNorm(self, input: HipTensor, normWeight: HipTensor, eps: float,
                                  weights: Sequence[HipTensor],
                                  biases: Optional[Sequence[Optional[HipTensor]]] = None,
                                  activation: Optional[str] = None) -> List[HipTensor]:
        """linearGrouped on `rmsnorm(input, normWeight, eps)`: q/k/v (or gate/up) of a
        decode step and the norm in front of them in one launch."""
        return self.linearGrouped(input, weights, biases, activation,
                                  _prologue=self._prologue(L.PRO_RMSNORM, normWeight, eps=eps))

    # tuning + counters -----------------------------------------------------
    def pretuneMatmulShapes(self, shapes: Sequence[Sequence[int]]) -> None:
        flat = (C.c_int64 * (3 * len(shapes)))(*[int(v) for s in shapes for v in s])
        L.call("tlhip_pretune_matmul_shapes", flat, len(shapes))

    def autotune(self, input: HipTensor, weight: HipTensor) -> float:
        """Benchmark all candidates for this (activation, weight) problem and
        cache the winner; returns its median time in microseconds."""
        qw = self._qweight(weight, transposed=False)
        m = input.size // qw.k
        out_dtype = "f16" if (input.dtype == "f16" and weight.format.elementType == "f16") else "f32"
        out = self._alloc([m, qw.n], out_dtype)
        best = C.c_double()
        L.call("tlhip_autotune", C.byref(qw), input.ptr, _DT_CODE[input.dtype], m, out.ptr,
               _DT_CODE[out_dtype], C.byref(best))
        out.destroy()
        return best.value

    def candidates(self, weight: HipTensor, x_dtype: str, m: int, y_dtype: str) -> List[L.KernelConfig]:
        qw = self._qweight(weight, transposed=False)
        cnt = C.c_int()
        L.call("tlhip_candidate_count", C.byref(qw), _DT_CODE[x_dtype], m, _DT_CODE[y_dtype], C.byref(cnt))
        out = []
        for i in range(cnt.value):
            kc = L.KernelConfig()
            L.call("tlhip_candidate_get", C.byref(qw), _DT_CODE[x_dtype], m, _DT_CODE[y_dtype], i, C.byref(kc))
            out.append(kc)
        return out

    def seedPerShapeMatmulChoice(self, weight: HipTensor, x_dtype: str, m: int, y_dtype: str,
                                 config: L.KernelConfig) -> None:
        """dispatch.ts:99-107: record a winner without benchmarking."""
        qw = self._qweight(weight, transposed=False)
        L.call("tlhip_tune_cache_seed", C.byref(qw), _DT_CODE[x_dtype], m, _DT_CODE[y_dtype], C.byref(config))

    def selectedConfig(self, weight: HipTensor, x_dtype: str, m: int, y_dtype: str) -> L.KernelConfig:
        qw = self._qweight(weight, transposed=False)
        kc = L.KernelConfig()
        L.call("tlhip_selected_config", C.byref(qw), _DT_CODE[x_dtype], m, _DT_CODE[y_dtype], C.byref(kc))
        return kc


def setAutotuneEnabled(enabled: bool) -> None:
    L.call("tlhip_set_autotune_enabled", 1 if enabled else 0)


def isAutotuneEnabled() -> bool:
    return bool(L.load().tlhip_is_autotune_enabled())


def exportTuningCache() -> str:
    need = C.c_size_t()
    L.call("tlhip_tune_cache_export", None, 0, C.byref(need))
    buf = C.create_string_buffer(need.value)
    L.call("tlhip_tune_cache_export", buf, need.value, C.byref(need))
    return buf.value.decode()


def importTuningCache(text: str) -> None:
    L.call("tlhip_tune_cache_import", text.encode())


def clearTuningCache() -> None:
    L.call("tlhip_tune_cache_clear")


def getQuantGemvDispatchCount() -> int:
    return int(L.load().tlhip_counter(b"quant_gemv_dispatches"))


def getQuantGemmDispatchCount() -> int:
    return int(L.load().tlhip_counter(b"quant_gemm_dispatches"))


def getDequantI8DispatchCount() -> int:
    return int(L.load().tlhip_counter(b"dequant_dispatches"))


def getAutotuneRunCount() -> int:
    return int(L.load().tlhip_counter(b"autotune_runs"))


def resetMatmulState() -> None:
    """dispatch.ts:194-206: caches, autotune mode and counters."""
    L.call("tlhip_tune_cache_clear")
    L.call("tlhip_set_autotune_enabled", 0)
    L.call("tlhip_counters_reset")


_backend: Optional[HipBackend] = None


def getBackend(device_index: int = 0) -> HipBackend:
    """registerBackend/getBackend (src/backend/registry.ts:15-17) for "hip"."""
    global _backend
    if _backend is None:
        _backend = HipBackend(device_index)
    return _backend
