"""Configuration surface of the quantized linear layer.

Field names, defaults and the accepted/rejected combinations are those of the reference
(inference_lib/src/fp_quant/utils/config.py:6-61) so existing configs load unchanged.
"""
from dataclasses import dataclass, field
from enum import Enum
from typing import List, Literal


class FPQuantDtype(Enum):
    MXFP4 = "mxfp4"
    NVFP4 = "nvfp4"
    MXFP8 = "mxfp8"
    BF16 = "bf16"


QuantMethod = Literal["quest", "abs_max"]
TransformInit = Literal["hadamard", "identity", "gsr"]

_ROTATION_SIZES = {
    FPQuantDtype.NVFP4: (16, 32, 64, 128),
    FPQuantDtype.MXFP4: (32, 64, 128),
}


@dataclass
class FPQuantConfig:
    forward_dtype: FPQuantDtype = FPQuantDtype.MXFP4
    forward_method: QuantMethod = "quest"
    backward_dtype: FPQuantDtype = FPQuantDtype.MXFP4
    store_master_weights: bool = False
    hadamard_group_size: int = 32
    pseudoquantization: bool = False
    transform_init: TransformInit = "hadamard"
    modules_to_not_convert: List[str] = field(default_factory=lambda: ["lm_head"])


def validate_config(config: FPQuantConfig) -> None:
    """Raise ValueError for the combinations the reference rejects (config.py:28-61)."""
    fwd, bwd = config.forward_dtype, config.backward_dtype
    if fwd == FPQuantDtype.NVFP4 and config.forward_method != "abs_max":
        raise ValueError("NVFP4 can only be used with abs_max method")
    sizes = _ROTATION_SIZES.get(fwd)
    if sizes is not None and config.hadamard_group_size not in sizes:
        raise ValueError(
            f"{fwd.name} can only be used with hadamard_group_size in {list(sizes)}"
        )
    # same precedence as the reference's unparenthesised `a or b and c`
    if fwd == FPQuantDtype.MXFP8 or (bwd == FPQuantDtype.MXFP8 and fwd != FPQuantDtype.MXFP4):
        raise ValueError("MXFP8 can only be used on backward in combination with MXFP4 forward")
    if bwd == FPQuantDtype.MXFP4 and fwd != FPQuantDtype.MXFP4:
        raise ValueError("MXFP4 backward can only be used with MXFP4 forward")
