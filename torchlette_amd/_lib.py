"""ctypes binding of the C ABI in ``include/tlhip.h`` (``libtlhip.so``).

This is the Python-side equivalent of the N-API addon a torchlette checkout
would use: one function per exported symbol, errors turned into exceptions with
the library's message (the reference's only error channel is ``throw new
Error(msg)``, src/backend/webgpu/ops/matmul-ops.ts:121-126).

There is no fallback: if the shared library is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TLHIP_LIBRARY names another build of the same library (e.g. one under test).
LIB_PATH = os.environ.get("TLHIP_LIBRARY") or os.path.join(_HERE, "libtlhip.so")

FMT_INT8_GROUPED, FMT_INT8_ROW, FMT_INT4_GROUPED = 0, 1, 2
F32, F16, I32 = 0, 1, 2
UNARY = {"none": 0, "relu": 1, "silu": 2, "gelu": 3, "gelu_tanh": 3, "gelu_erf": 4,
         "sigmoid": 5, "tanh": 6}
EPI_NONE, EPI_BIAS, EPI_UNARY, EPI_BINARY, EPI_CAST_F16 = 0, 1, 2, 3, 4
BINARY = {"add": 0, "sub": 1, "mul": 2}
MAX_EPILOGUE_OPS = 4
VARIANT_GEMV, VARIANT_GEMV_MFMA, VARIANT_TILED, VARIANT_TILED_DIRECT, VARIANT_GEMV_XREG, VARIANT_GEMV_WAVE = 0, 1, 2, 3, 4, 5


class TlhipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(message)
        self.code = code


class EpilogueOp(C.Structure):
    _fields_ = [("kind", C.c_int32), ("unary", C.c_int32), ("input", C.c_void_p),
                ("input_dtype", C.c_int32), ("rows", C.c_int32)]


class Epilogue(C.Structure):
    _fields_ = [("n_ops", C.c_int32), ("reserved", C.c_int32), ("ops", EpilogueOp * MAX_EPILOGUE_OPS)]


class QWeight(C.Structure):
    _fields_ = [("format", C.c_int32), ("group_size", C.c_int32), ("n", C.c_int64), ("k", C.c_int64),
                ("packed", C.c_void_p), ("scales", C.c_void_p)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("arch", C.c_char * 32), ("compute_units", C.c_int32),
                ("wavefront_size", C.c_int32), ("lds_bytes_per_block", C.c_int32),
                ("clock_khz", C.c_int32), ("memory_clock_khz", C.c_int32),
                ("memory_bus_bits", C.c_int32), ("total_memory_bytes", C.c_int64),
                ("l2_bytes", C.c_int64)]


class KernelConfig(C.Structure):
    _fields_ = [("variant", C.c_int32)] + [(f"p{i}", C.c_int32) for i in range(7)]

    def as_tuple(self):
        return (self.variant, self.p0, self.p1, self.p2, self.p3, self.p4, self.p5, self.p6)

    @classmethod
    def of(cls, *vals):
        vals = list(vals) + [0] * (8 - len(vals))
        return cls(*vals)


class Prologue(C.Structure):
    _fields_ = [("kind", C.c_int32), ("unary", C.c_int32), ("eps", C.c_float), ("reserved", C.c_int32),
                ("operand", C.c_void_p)]


PRO_NONE, PRO_RMSNORM, PRO_GATED_MUL = 0, 1, 2
ERR_INVALID, ERR_DEVICE, ERR_STATE, ERR_UNSUPPORTED = 1, 2, 3, 4


class AutotuneOptions(C.Structure):
    _fields_ = [("reps", C.c_int32), ("batches", C.c_int32), ("retime_top", C.c_int32), ("quick", C.c_int32),
                ("warm_ms", C.c_double), ("pool_bytes", C.c_uint64)]


class GemvProblem(C.Structure):
    _fields_ = [("w", QWeight), ("x", C.c_void_p), ("y", C.c_void_p), ("epilogue", C.POINTER(Epilogue))]


class SequenceStep(C.Structure):
    _fields_ = [("w", QWeight), ("w_up", QWeight), ("x", C.c_void_p), ("y", C.c_void_p),
                ("epilogue", C.POINTER(Epilogue)), ("y_dtype", C.c_int32), ("gated", C.c_int32),
                ("wait", C.c_int32), ("reserved", C.c_int32)]


# name -> (restype, argtypes); every symbol include/tlhip.h declares.
_vp, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
_QW, _EP, _KC = C.POINTER(QWeight), C.POINTER(Epilogue), C.POINTER(KernelConfig)
SIGNATURES = {
    "tlhip_init": (_i, [_i]),
    "tlhip_shutdown": (_i, []),
    "tlhip_last_error": (C.c_char_p, []),
    "tlhip_device_info": (_i, [C.POINTER(DeviceInfo)]),
    "tlhip_malloc": (_i, [_sz, C.POINTER(_vp)]),
    "tlhip_free": (_i, [_vp]),
    "tlhip_memset": (_i, [_vp, _i, _sz, _vp]),
    "tlhip_memcpy_h2d": (_i, [_vp, _vp, _sz, _vp]),
    "tlhip_memcpy_d2h": (_i, [_vp, _vp, _sz, _vp]),
    "tlhip_memcpy_d2d": (_i, [_vp, _vp, _sz, _vp]),
    "tlhip_host_alloc": (_i, [_sz, C.POINTER(_vp)]),
    "tlhip_host_free": (_i, [_vp]),
    "tlhip_stream_create": (_i, [C.POINTER(_vp)]),
    "tlhip_stream_destroy": (_i, [_vp]),
    "tlhip_stream_synchronize": (_i, [_vp]),
    "tlhip_event_create": (_i, [C.POINTER(_vp)]),
    "tlhip_event_destroy": (_i, [_vp]),
    "tlhip_event_record": (_i, [_vp, _vp]),
    "tlhip_event_synchronize": (_i, [_vp]),
    "tlhip_event_elapsed_us": (_i, [_vp, _vp, C.POINTER(C.c_double)]),
    "tlhip_graph_begin_capture": (_i, [_vp]),
    "tlhip_graph_end_capture": (_i, [_vp, C.POINTER(_vp)]),
    "tlhip_graph_launch": (_i, [_vp, _vp]),
    "tlhip_graph_destroy": (_i, [_vp]),
    "tlhip_f32_to_f16_bits": (C.c_uint16, [_f]),
    "tlhip_f16_bits_to_f32": (_f, [C.c_uint16]),
    "tlhip_quantize_int8_grouped_device": (_i, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "tlhip_quantize_int8_grouped": (_i, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "tlhip_epilogue_check": (_i, [_QW, _i64, _EP]),
    "tlhip_dequant": (_i, [_QW, _vp, _vp]),
    "tlhip_gemv": (_i, [_QW, _vp, _i, _i64, _vp, _i, _f, _EP, _vp]),
    "tlhip_gemv_noalloc": (_i, [_QW, _vp, _i, _i64, _vp, _i, _f, _EP, _vp]),
    "tlhip_gemv_grouped": (_i, [C.POINTER(GemvProblem), _i, _i, _i, _f, _vp]),
    "tlhip_gemv_grouped_rows": (_i, [C.POINTER(GemvProblem), _i, _i, _i64, _i, _f, _vp]),
    "tlhip_gemv_sequence": (_i, [C.POINTER(SequenceStep), _i, _i, _i64, _f, _vp]),
    "tlhip_mlp_decode": (_i, [_QW, _QW, _QW, _i, _vp, _i, _i64, _vp, _vp, _i, _EP, _vp]),
    "tlhip_sequence_status": (_i, [_vp, C.POINTER(_i)]),
    "tlhip_debug_sequence": (_i, [_i, C.c_uint32]),
    "tlhip_gemv_prologue": (_i, [_QW, C.POINTER(Prologue), _vp, _i, _i64, _vp, _i, _f, _EP, _vp]),
    "tlhip_gemv_grouped_prologue": (_i, [C.POINTER(GemvProblem), _i, C.POINTER(Prologue), _i, _i, _f, _vp]),
    "tlhip_rmsnorm": (_i, [_vp, _i, _vp, _vp, _i, _i64, _i64, _f, _vp]),
    "tlhip_gated_mul": (_i, [_i, _vp, _vp, _i, _vp, _i64, _vp]),
    "tlhip_gemm_prefill": (_i, [_QW, _vp, _i, _i64, _vp, _i, _f, _EP, _vp]),
    "tlhip_matmul_quantized": (_i, [_QW, _vp, _i, _i64, _vp, _i, _f, _EP, _vp]),
    "tlhip_matmul_quantized_config": (_i, [_QW, _vp, _i, _i64, _vp, _i, _f, _EP, _KC, _vp]),
    "tlhip_bias_add": (_i, [_vp, _i, _vp, _i, _vp, _i64, _i64, _vp]),
    "tlhip_unary": (_i, [_i, _vp, _i, _vp, _i64, _vp]),
    "tlhip_cast": (_i, [_vp, _i, _vp, _i, _i64, _vp]),
    "tlhip_topk": (_i, [_vp, _i64, _i64, _i, _vp, _vp, _i, _vp]),
    "tlhip_candidate_count": (_i, [_QW, _i, _i64, _i, C.POINTER(_i)]),
    "tlhip_candidate_get": (_i, [_QW, _i, _i64, _i, _i, _KC]),
    "tlhip_selected_config": (_i, [_QW, _i, _i64, _i, _KC]),
    "tlhip_selected_route": (_i, [_QW, _i, _i64, _i, C.POINTER(_i64), _KC, _KC]),
    "tlhip_set_autotune_enabled": (_i, [_i]),
    "tlhip_is_autotune_enabled": (_i, []),
    "tlhip_autotune": (_i, [_QW, _vp, _i, _i64, _vp, _i, C.POINTER(C.c_double)]),
    "tlhip_autotune_pool": (_i, [_QW, _i, _vp, _i, _i64, _vp, _i, _EP, C.POINTER(AutotuneOptions), _vp,
                                C.POINTER(C.c_double)]),
    "tlhip_tune_cache_seed": (_i, [_QW, _i, _i64, _i, _KC]),
    "tlhip_pretune_matmul_shapes": (_i, [C.POINTER(_i64), _i]),
    "tlhip_tune_cache_export": (_i, [C.c_char_p, _sz, C.POINTER(_sz)]),
    "tlhip_tune_cache_import": (_i, [C.c_char_p]),
    "tlhip_tune_cache_clear": (_i, []),
    "tlhip_counter": (C.c_uint64, [C.c_char_p]),
    "tlhip_counters_reset": (_i, []),
}

_lib = None


def load() -> C.CDLL:
    """Load libtlhip.so and declare every signature.  Raises if it is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C torchlette_amd/csrc` "
                "(or __graft_entry__.build()); the hip backend has no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().tlhip_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise TlhipError(rc, last_error())


def call(name: str, *args):
    """Call an int-returning entry point and raise on a non-zero code."""
    check(getattr(load(), name)(*args))
