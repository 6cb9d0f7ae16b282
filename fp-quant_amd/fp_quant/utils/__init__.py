"""Configuration, model surgery, producer fusion and export helpers of the fp_quant package."""
from . import config, export, fuse, replace
from .config import FPQuantConfig, FPQuantDtype, validate_config
from .fuse import fuse_producers, unfuse_producers
from .replace import (
    finalize_master_weights,
    release_row_major_weights,
    replace_quantize_with_fp_quant_linear,
    replace_with_fp_quant_linear,
    restore_row_major_weights,
)

__all__ = [
    "FPQuantConfig",
    "FPQuantDtype",
    "validate_config",
    "replace_with_fp_quant_linear",
    "replace_quantize_with_fp_quant_linear",
    "finalize_master_weights",
    "release_row_major_weights",
    "restore_row_major_weights",
    "fuse_producers",
    "unfuse_producers",
    "config",
    "export",
    "fuse",
    "replace",
]
