"""Configuration surface of the quantized linear layer.

`FPQuantDtype`, `FPQuantConfig` (field names, order and defaults) and the combinations that
`validate_config` accepts or rejects are those of the reference
(inference_lib/src/fp_quant/utils/config.py:6-61), so existing configs load unchanged.  On top of
that: the group size a format scales over, and the conversion to and from the `quantization_config`
entry that checkpoints carry (src/quantization/qconfig.py:3-21).
"""
from dataclasses import dataclass, field, fields
from enum import Enum
from typing import Any, Dict, List, Literal, Mapping


class FPQuantDtype(Enum):
    MXFP4 = "mxfp4"   # E2M1 codes, one E8M0 scale per 32 values
    NVFP4 = "nvfp4"   # E2M1 codes, one E4M3 scale per 16 values and a per-tensor fp32 multiplier
    MXFP8 = "mxfp8"   # backward only (training), not computed by this engine
    BF16 = "bf16"     # backward of the inference configuration

    @property
    def scale_group(self) -> int:
        """Values that share one scale (0 for formats without group scales)."""
        return {"mxfp4": 32, "nvfp4": 16, "mxfp8": 32}.get(self.value, 0)


QuantMethod = Literal["quest", "abs_max"]
TransformInit = Literal["hadamard", "identity", "gsr"]

# rotation block sizes a forward format accepts
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

    @classmethod
    def from_dict(cls, entry: Mapping[str, Any]) -> "FPQuantConfig":
        """From a checkpoint's `quantization_config` entry: dtype names become enum members, keys
        this class does not know (`quant_method`, ...) are ignored."""
        known = {f.name for f in fields(cls)}
        kwargs = {k: v for k, v in entry.items() if k in known}
        for key in ("forward_dtype", "backward_dtype"):
            if key in kwargs and not isinstance(kwargs[key], FPQuantDtype):
                kwargs[key] = FPQuantDtype(str(kwargs[key]).lower())
        if "modules_to_not_convert" in kwargs:
            kwargs["modules_to_not_convert"] = list(kwargs["modules_to_not_convert"] or [])
        return cls(**kwargs)

    def to_dict(self) -> Dict[str, Any]:
        """The `quantization_config` entry of a saved model config (dtype names as strings)."""
        out: Dict[str, Any] = {"quant_method": "fp_quant"}
        for f in fields(self):
            value = getattr(self, f.name)
            out[f.name] = value.value if isinstance(value, FPQuantDtype) else value
        out["modules_to_not_convert"] = list(self.modules_to_not_convert)
        return out


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
