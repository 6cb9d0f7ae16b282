"""Model surgery: swap nn.Linear modules for FPQuantLinear.

Same three entry points, arguments and skip rule (dotted name ends with an entry of
`modules_to_not_convert`) as inference_lib/src/fp_quant/utils/replace.py:7-144.
"""
from typing import Iterator, List, Optional, Tuple

from torch import nn

from .config import FPQuantConfig


def _linears(model: nn.Module, prefix: Optional[List[str]]) -> Iterator[Tuple[nn.Module, str, str]]:
    """(parent, child name, dotted name relative to the call root) for every nn.Linear,
    parents before children, in registration order."""
    base = ".".join(prefix) + "." if prefix else ""
    for parent_name, parent in list(model.named_modules()):
        for child_name, child in list(parent.named_children()):
            if isinstance(child, nn.Linear):
                dotted = f"{parent_name}.{child_name}" if parent_name else child_name
                yield parent, child_name, base + dotted


def _skipped(dotted: str, config: FPQuantConfig) -> bool:
    return any(dotted.endswith(key) for key in config.modules_to_not_convert)


def replace_with_fp_quant_linear(
    model,
    fp_quant_linear_config: FPQuantConfig,
    current_key_name=None,
    has_been_replaced=False,
):
    """Replace every eligible nn.Linear by an *empty* (meta-device) FPQuantLinear, for
    loaders that fill the buffers afterwards.  Returns (model, has_been_replaced)."""
    from accelerate import init_empty_weights

    from ..module import FPQuantLinear

    for parent, name, dotted in _linears(model, current_key_name):
        if _skipped(dotted, fp_quant_linear_config):
            continue
        old = parent._modules[name]
        with init_empty_weights():
            new = FPQuantLinear(
                old.in_features,
                old.out_features,
                config=fp_quant_linear_config,
                bias=old.bias is not None,
            )
        new.source_cls = type(old)
        new.requires_grad_(False)
        parent._modules[name] = new
        has_been_replaced = True
    return model, has_been_replaced


def replace_quantize_with_fp_quant_linear(
    model,
    fp_quant_linear_config: FPQuantConfig,
    current_key_name=None,
    has_been_replaced=False,
):
    """Replace every eligible nn.Linear by an FPQuantLinear holding its weight/bias and
    quantize it on the spot (`pre_forward`).  Returns the model."""
    from ..module import FPQuantLinear

    for parent, name, dotted in _linears(model, current_key_name):
        if _skipped(dotted, fp_quant_linear_config):
            continue
        old = parent._modules[name]
        new = FPQuantLinear(
            old.in_features,
            old.out_features,
            config=fp_quant_linear_config,
            bias=old.bias is not None,
            device=old.weight.device,
            dtype=old.weight.dtype,
        )
        new.weight.data = old.weight.data
        if old.bias is not None:
            new.bias.data = old.bias.data
        new.pre_forward()
        parent._modules[name] = new
    return model


def finalize_master_weights(model, current_key_name=None):
    """Drop master weights: clear `store_master_weights` and re-run `pre_forward` on every
    FPQuantLinear of the model."""
    from ..module import FPQuantLinear

    for module in model.modules():
        if isinstance(module, FPQuantLinear):
            if module.config.store_master_weights:
                module.config.store_master_weights = False  # the config object is shared
            module.pre_forward()


def release_row_major_weights(model) -> int:
    """Hold every eligible layer's 4-bit weight once, in the packed layout the GEMM kernels read
    (FPQuantLinear.release_row_major): frees the row-major `qweight` / `scales` copies, half of the
    weight memory of a quantized model.  state_dict() and load_state_dict() keep speaking the
    reference's row-major tensors.  Call it after the linears have been replaced and quantized (before or
    after fuse_producers).  Returns the number of layers that are in that state afterwards."""
    from ..module import FPQuantLinear

    count = 0
    for module in model.modules():
        if isinstance(module, FPQuantLinear) and module.release_row_major():
            count += 1
    for module in model.modules():   # groups of projections built on the old tensors follow their members
        build = getattr(module, "_fpq_weight_group_build", None)
        if build is not None:
            build()
    return count


def restore_row_major_weights(model) -> None:
    """Undo release_row_major_weights."""
    from ..module import FPQuantLinear

    for module in model.modules():
        if isinstance(module, FPQuantLinear):
            module.restore_row_major()
    for module in model.modules():
        build = getattr(module, "_fpq_weight_group_build", None)
        if build is not None:
            build()
