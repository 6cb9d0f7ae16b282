"""Fuse the elementwise producers of a decoder block into the quantizers that consume them.

In a Llama-style block the RMSNorm output is only read by the q/k/v (or gate/up) projections and
`act_fn(gate) * up` only by `down_proj` (src/utils/llama_utils.py:60-71, 132-160 of the reference
keep one activation quantizer per such group).  With those projections being FPQuantLinear layers,
`fuse_producers` patches the block so that

* each RMSNorm computes its bf16 output and the rotated, quantized form of it in one kernel; the
  projections that are then called with that output find the quantized form and go straight to
  their GEMM;
* the MLP quantizes bf16(silu(gate)) * up directly from `gate` and `up`, without writing the product.

Results are those of the unfused modules with one bf16 rounding per PyTorch operator (normalise,
scale by the weight; silu, multiply); parameters, buffers and state-dict keys are untouched.  Calls
that cannot take the fused kernels (tracing, CPU tensors, other dtypes, training, rotations without
a fused kernel) run the original forward.
"""
import types
from typing import Optional

import torch
from torch import nn

from .config import FPQuantDtype


def _eager():
    from ..module import eager

    return eager


def _is_real_quant_linear(layer) -> bool:
    from ..module import FPQuantLinear

    if not isinstance(layer, FPQuantLinear) or layer.qweight is None or layer.scales is None:
        return False
    cfg = layer.config
    return (cfg.forward_method == "abs_max" and cfg.forward_dtype in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4)
            and cfg.backward_dtype == FPQuantDtype.BF16 and not cfg.store_master_weights
            and not cfg.pseudoquantization)


def _fusable_call(x: torch.Tensor) -> bool:
    return (x.is_cuda and x.dtype == torch.bfloat16 and not torch.compiler.is_compiling()
            and not (torch.is_grad_enabled() and x.requires_grad))


def _is_llama_rmsnorm(norm) -> bool:
    """Modules computing weight * (x / rms(x)).to(dtype) as transformers' LlamaRMSNorm does (the
    (1 + weight) variants are not)."""
    name = type(norm).__name__
    return (isinstance(norm, nn.Module) and name.endswith("RMSNorm") and "Gemma" not in name
            and isinstance(getattr(norm, "weight", None), torch.Tensor) and norm.weight.dim() == 1
            and isinstance(getattr(norm, "variance_epsilon", None), float))


def fuse_rmsnorm(norm: nn.Module, consumer) -> bool:
    """Make `norm` leave its output quantized for `consumer` (an FPQuantLinear fed by it, standing
    for all layers fed by it: they share rotation and activation scale).  False if not applicable."""
    if not _is_llama_rmsnorm(norm) or not _is_real_quant_linear(consumer):
        return False
    if getattr(norm, "_fpq_unfused_forward", None) is not None:
        return True
    unfused = norm.forward
    peer = [consumer]   # in a list: not registered as a submodule of the norm

    def forward(self, hidden_states):
        layer = peer[0]
        if _fusable_call(hidden_states) and self.weight.dtype == torch.bfloat16:
            y = _eager().rmsnorm_quantize(hidden_states, self.weight, self.variance_epsilon,
                                            layer.forward_hadamard_matrix, layer.act_global_scale,
                                            layer.config.forward_dtype == FPQuantDtype.NVFP4)
            if y is not None:
                return y
        return unfused(hidden_states)

    norm._fpq_unfused_forward = unfused
    norm.forward = types.MethodType(forward, norm)
    return True


def fuse_gated_mlp(mlp: nn.Module) -> bool:
    """Patch a `down_proj(act_fn(gate_proj(x)) * up_proj(x))` MLP with SiLU activation whose three
    projections are FPQuantLinear layers.  False if the module is not of that form."""
    parts = [getattr(mlp, n, None) for n in ("gate_proj", "up_proj", "down_proj")]
    act = getattr(mlp, "act_fn", None)
    is_silu = isinstance(act, nn.SiLU) or type(act).__name__ in ("SiLUActivation", "SiLU")
    if not is_silu or not all(_is_real_quant_linear(p) for p in parts):
        return False
    if getattr(mlp, "_fpq_unfused_forward", None) is not None:
        return True
    unfused = mlp.forward

    def forward(self, x):
        if not _fusable_call(x):
            return unfused(x)
        gate = self.gate_proj(x)
        up = self.up_proj(x)
        down = self.down_proj
        inter = gate.shape[-1]
        qa = _eager().silu_mul_quantize(gate.reshape(-1, inter), up.reshape(-1, inter),
                                          down.forward_hadamard_matrix, down.act_global_scale,
                                          down.config.forward_dtype == FPQuantDtype.NVFP4)
        if qa is None:
            return down(self.act_fn(gate) * up)
        return down.forward_quantized(qa, gate.shape[:-1])

    mlp._fpq_unfused_forward = unfused
    mlp.forward = types.MethodType(forward, mlp)
    return True


def fuse_producers(model: nn.Module) -> int:
    """Apply fuse_rmsnorm / fuse_gated_mlp to every decoder block of `model` that has the Llama
    layout (`input_layernorm`, `self_attn.q_proj`, `post_attention_layernorm`, `mlp.gate_proj`).
    Call it after the linears have been replaced and quantized.  Returns the number of patches."""
    count = 0
    for block in model.modules():
        attn, mlp = getattr(block, "self_attn", None), getattr(block, "mlp", None)
        if attn is None or mlp is None:
            continue
        count += int(fuse_rmsnorm(getattr(block, "input_layernorm", None), getattr(attn, "q_proj", None)))
        count += int(fuse_rmsnorm(getattr(block, "post_attention_layernorm", None), getattr(mlp, "gate_proj", None)))
        count += int(fuse_gated_mlp(mlp))
    return count


def unfuse_producers(model: nn.Module) -> None:
    """Undo fuse_producers."""
    for module in model.modules():
        unfused: Optional[object] = getattr(module, "_fpq_unfused_forward", None)
        if unfused is not None:
            module.forward = unfused
            module._fpq_unfused_forward = None
