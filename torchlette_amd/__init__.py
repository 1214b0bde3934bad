"""torchlette `hip` backend: the quantized-weight linear path on MI355X (gfx950).

``torchlette_amd.backend`` is the host-side mirror of torchlette's backend
interface for this path; ``torchlette_amd._lib`` binds the C ABI of
``include/tlhip.h``; ``torchlette_amd/csrc`` holds the HIP kernels.
"""
from . import _lib  # noqa: F401
from .backend import (  # noqa: F401
    HipBackend, HipTensor, QuantPacking, StorageFormat, clearTuningCache, exportTuningCache,
    f16BitsToF32, f32ToF16Bits, getAutotuneRunCount, getBackend, getDequantI8DispatchCount,
    getQuantGemmDispatchCount, getQuantGemvDispatchCount, importTuningCache, isAutotuneEnabled,
    quantizeLinearWeight, resetMatmulState, resolveWeightFormat, setAutotuneEnabled,
)
from .packed_cache import PackedWeightCache, loadQuantizedWeight, packedKey  # noqa: F401
