"""fp_quant — MI355X (gfx950) engine behind FP-Quant's inference surface.

Exports the names the reference package exports (inference_lib/src/fp_quant/__init__.py:5-12);
the arithmetic runs in hand-written HIP kernels reached through the C ABI of libfpq_hip.so.
"""
from .module import FPQuantLinear
from .utils import (
    FPQuantConfig,
    FPQuantDtype,
    finalize_master_weights,
    replace_quantize_with_fp_quant_linear,
    replace_with_fp_quant_linear,
)

__version__ = "0.3.2"   # the release of the reference package whose surface this mirrors (inference_lib/setup.py:5)
__all__ = [
    "FPQuantLinear",
    "FPQuantConfig",
    "FPQuantDtype",
    "replace_with_fp_quant_linear",
    "replace_quantize_with_fp_quant_linear",
    "finalize_master_weights",
]
