from .config import FPQuantConfig, FPQuantDtype, validate_config
from .replace import (
    finalize_master_weights,
    replace_quantize_with_fp_quant_linear,
    replace_with_fp_quant_linear,
)
from .fuse import fuse_producers, unfuse_producers
