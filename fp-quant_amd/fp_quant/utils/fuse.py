"""Fuse the elementwise producers of a decoder block into the quantizers that consume them.

In a Llama-style block the RMSNorm output is only read by the q/k/v (or gate/up) projections and
`act_fn(gate) * up` only by `down_proj` (src/utils/llama_utils.py:60-71, 132-160 of the reference
keep one activation quantizer per such group).  With those projections being FPQuantLinear layers,
`fuse_producers` patches the block so that

* each RMSNorm computes its bf16 output and the rotated, quantized form of it in one kernel; the
  projections that are then called with that output find the quantized form and go straight to
  their GEMM;
* the MLP quantizes bf16(silu(gate)) * up directly from `gate` and `up`, without writing the product;
* the two `residual + hidden_states` additions of the block happen in the epilogues of the `o_proj`
  and `down_proj` GEMMs (blocks whose forward is, statement for statement, the one of transformers'
  LlamaDecoderLayer; others keep their additions).

Results are those of the unfused modules with one bf16 rounding per PyTorch operator (normalise,
scale by the weight; silu, multiply); parameters, buffers and state-dict keys are untouched.  Calls
that cannot take the fused kernels (tracing, CPU tensors, other dtypes, training, rotations without
a fused kernel) run the original forward.
"""
import ast
import inspect
import textwrap
import types
from typing import Dict, Optional

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

    def forward(self, x, residual=None):
        """`residual`: added to the result (a fused decoder block passes its skip connection)."""
        if not _fusable_call(x) or (residual is not None and not _fusable_call(residual)):
            y = unfused(x)
            return y if residual is None else residual + y
        gate = self.gate_proj(x)
        up = self.up_proj(x)
        down = self.down_proj
        inter = gate.shape[-1]
        qa = _eager().silu_mul_quantize(gate.reshape(-1, inter), up.reshape(-1, inter),
                                          down.forward_hadamard_matrix, down.act_global_scale,
                                          down.config.forward_dtype == FPQuantDtype.NVFP4)
        if qa is None:
            y = down(self.act_fn(gate) * up)
            return y if residual is None else residual + y
        return down.forward_quantized(qa, gate.shape[:-1], residual)

    mlp._fpq_unfused_forward = unfused
    mlp.forward = types.MethodType(forward, mlp)
    return True


# The decoder block forward whose additions fuse_residual_adds moves into the GEMMs, one entry per
# statement as ast.unparse prints it; entry 2 (the attention call) is checked structurally.
_BLOCK_STATEMENTS = (
    "residual = hidden_states",
    "hidden_states = self.input_layernorm(hidden_states)",
    None,
    "hidden_states = residual + hidden_states",
    "residual = hidden_states",
    "hidden_states = self.post_attention_layernorm(hidden_states)",
    "hidden_states = self.mlp(hidden_states)",
    "hidden_states = residual + hidden_states",
    "return hidden_states",
)


def _attention_call_defaults(block: nn.Module) -> Optional[Dict[str, object]]:
    """If the class's forward is exactly the statements above, with the attention called as
    `hidden_states, _ = self.self_attn(hidden_states=hidden_states, <p>=<p> for every other
    parameter p of forward, **kwargs)`: the defaults of those parameters.  None otherwise."""
    fn = type(block).forward
    try:
        tree = ast.parse(textwrap.dedent(inspect.getsource(fn)))
        params = inspect.signature(fn).parameters
    except (OSError, TypeError, SyntaxError, ValueError):
        return None
    body = tree.body[0].body if tree.body and isinstance(tree.body[0], ast.FunctionDef) else []
    if body and isinstance(body[0], ast.Expr) and isinstance(getattr(body[0], "value", None), ast.Constant):
        body = body[1:]   # docstring
    if len(body) != len(_BLOCK_STATEMENTS):
        return None
    for stmt, want in zip(body, _BLOCK_STATEMENTS):
        if want is not None and ast.unparse(stmt) != want:
            return None
    call = body[2]
    if not (isinstance(call, ast.Assign) and len(call.targets) == 1
            and ast.unparse(call.targets[0]) in ("(hidden_states, _)", "hidden_states, _")
            and isinstance(call.value, ast.Call) and ast.unparse(call.value.func) == "self.self_attn"
            and not call.value.args):
        return None
    names = list(params)
    if len(names) < 2 or names[0] != "self" or names[1] != "hidden_states":
        return None
    defaults: Dict[str, object] = {}
    var_keyword = None
    for name in names[2:]:
        p = params[name]
        if p.kind == inspect.Parameter.VAR_KEYWORD:
            var_keyword = name
        elif p.kind in (inspect.Parameter.POSITIONAL_OR_KEYWORD, inspect.Parameter.KEYWORD_ONLY) \
                and p.default is not inspect.Parameter.empty:
            defaults[name] = p.default
        else:
            return None
    passed = {}
    for kw in call.value.keywords:
        if kw.arg is None:
            if not (isinstance(kw.value, ast.Name) and kw.value.id == var_keyword):
                return None
            var_keyword = None
        elif not (isinstance(kw.value, ast.Name) and kw.value.id == kw.arg):
            return None
        else:
            passed[kw.arg] = True
    if var_keyword is not None or set(passed) != set(defaults) | {"hidden_states"}:
        return None
    return defaults


def fuse_residual_adds(block: nn.Module) -> bool:
    """Move the two `residual + hidden_states` additions of a decoder block into the GEMMs of
    `self_attn.o_proj` and `mlp.down_proj`.  Needs the MLP patched by fuse_gated_mlp, `o_proj` an
    FPQuantLinear, and the block's forward to be the Llama one statement for statement (checked on
    its source); False otherwise.  Each addition that a GEMM cannot take (small batches, NVFP4,
    autograd) is done by PyTorch as before, so results do not depend on which path ran."""
    mlp, attn = getattr(block, "mlp", None), getattr(block, "self_attn", None)
    o_proj = getattr(attn, "o_proj", None)
    if getattr(mlp, "_fpq_unfused_forward", None) is None or not _is_real_quant_linear(o_proj):
        return False
    if getattr(block, "_fpq_unfused_forward", None) is not None:
        return True
    if "forward" in vars(block):   # already patched by someone else
        return False
    defaults = _attention_call_defaults(block)
    if defaults is None:
        return False
    unfused = block.forward

    def forward(self, hidden_states, *args, **kwargs):
        if args or not isinstance(hidden_states, torch.Tensor) or not _fusable_call(hidden_states):
            return unfused(hidden_states, *args, **kwargs)
        out_proj = self.self_attn.o_proj
        normed = self.input_layernorm(hidden_states)
        out_proj._fpq_residual = hidden_states
        try:
            attn_out, _ = self.self_attn(hidden_states=normed, **{**defaults, **kwargs})
        finally:
            pending = out_proj._fpq_residual
            out_proj._fpq_residual = None
        if pending is not None:   # o_proj did not take it
            attn_out = hidden_states + attn_out
        return self.mlp(self.post_attention_layernorm(attn_out), residual=attn_out)

    block._fpq_unfused_forward = unfused
    block.forward = types.MethodType(forward, block)
    return True


def fuse_producers(model: nn.Module) -> int:
    """Apply fuse_rmsnorm / fuse_gated_mlp / fuse_residual_adds to every decoder block of `model` that
    has the Llama layout (`input_layernorm`, `self_attn.q_proj`, `post_attention_layernorm`, `mlp.gate_proj`).
    Call it after the linears have been replaced and quantized.  Returns the number of patches."""
    count = 0
    for block in model.modules():
        attn, mlp = getattr(block, "self_attn", None), getattr(block, "mlp", None)
        if attn is None or mlp is None:
            continue
        count += int(fuse_rmsnorm(getattr(block, "input_layernorm", None), getattr(attn, "q_proj", None)))
        count += int(fuse_rmsnorm(getattr(block, "post_attention_layernorm", None), getattr(mlp, "gate_proj", None)))
        count += int(fuse_gated_mlp(mlp))
        count += int(fuse_residual_adds(block))
    return count


def unfuse_producers(model: nn.Module) -> None:
    """Undo fuse_producers."""
    for module in model.modules():
        unfused: Optional[object] = getattr(module, "_fpq_unfused_forward", None)
        if unfused is not None:
            if getattr(unfused, "__func__", None) is type(module).forward:
                vars(module).pop("forward", None)   # back to the class's method
            else:
                module.forward = unfused
            module._fpq_unfused_forward = None
