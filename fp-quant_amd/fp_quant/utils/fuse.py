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

Under `torch.compile` the norms and additions are left to the compiler (it fuses them itself); what it
cannot know is that q/k/v, and gate/up, quantize the same tensor: there the patched MLP and attention
modules call group operators (one quantization, one GEMM per layer; SiLU*up fused into down_proj's
quantizer), which a captured decode step replays as fewer kernels.

Results follow the operator sequence of the unfused modules with one bf16 rounding per PyTorch operator
(normalise, scale by the weight; silu, multiply), evaluated with correctly rounded fp32 arithmetic in a
fixed order.  They are bit-identical to that definition, not to PyTorch's own kernels: torch's rsqrt and
exp are not correctly rounded, so a few elements per million differ by one bf16 step from the unfused
model (the whole-model test bounds the difference of the logits, it does not require equality).
Parameters, buffers and state-dict keys are untouched.  Calls
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


_eager_module = None


def _eager():
    """fp_quant.module.eager, imported on first use (it needs the built library) and remembered: the import
    statement alone costs most of a microsecond per call."""
    global _eager_module
    if _eager_module is None:
        from ..module import eager

        _eager_module = eager
    return _eager_module


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


def _traceable_call(x: torch.Tensor) -> bool:
    """A call being traced by a compiler that the group operators can serve."""
    return (torch.compiler.is_compiling() and x.is_cuda and x.dtype == torch.bfloat16
            and not (torch.is_grad_enabled() and x.requires_grad))


def _quantize_alike(layers) -> bool:
    """Whether these layers quantize an input identically (format, method, rotation, activation
    scale), so that one quantization can serve them all, and take their bias inside the GEMM."""
    first = layers[0]
    for layer in layers:
        a, b = first.config, layer.config
        if (a.forward_dtype, a.forward_method, a.hadamard_group_size) != (b.forward_dtype, b.forward_method,
                                                                          b.hadamard_group_size):
            return False
        if layer.in_features != first.in_features or layer.qweight.device != first.qweight.device:
            return False
        if not torch.equal(layer.forward_hadamard_matrix, first.forward_hadamard_matrix):
            return False
        if not torch.equal(layer.act_global_scale.float(), first.act_global_scale.float()):
            return False
        if layer.bias is not None and (layer.bias.dtype != torch.bfloat16 or not layer.bias.is_contiguous()):
            return False
    return True


def _weight_group(layers, create: bool = False, previous=None):
    """The layers' packed weights laid end to end (eager.WeightGroup), if they can be multiplied as one:
    abs-max layers (MXFP4 or NVFP4) that quantize alike with equal alpha.  Built when the model is patched
    (`create`), looked up afterwards (None: the layers were rewritten since, or never qualified)."""
    first = layers[0]
    if (first.config.forward_dtype not in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4)
            or first.config.forward_method != "abs_max"):
        return None
    if create:
        if not first.qweight.is_cuda or not _quantize_alike(layers):
            return None
        for layer in layers[1:]:
            if not torch.equal(layer.weight_global_scale.float(), first.weight_global_scale.float()):
                return None
    return _eager().weight_group([(l.qweight, l.scales, l.bias, l.in_features) for l in layers], create,
                                 first.config.forward_dtype == FPQuantDtype.NVFP4, previous)


def _attach_weight_group(module: nn.Module, names) -> None:
    """Build the WeightGroup of module.<names> now and keep it in `module._fpq_weight_group`; rebuilt after
    every load_state_dict into the module (a hook), so that traced code, which cannot check tensor
    addresses and counters, never multiplies by weights that have been replaced."""
    def build(*_):
        layers = [getattr(module, n) for n in names]
        # (built into the buffers of the group it replaces where the shapes allow: a recorded graph keeps
        # pointing at the current weights)
        module._fpq_weight_group = (_weight_group(layers, create=True, previous=getattr(module, "_fpq_weight_group", None))
                                    if all(_is_real_quant_linear(l) for l in layers) else None)

    build()
    module._fpq_weight_group_build = build   # for whoever rewrites the layers' weights by other means
    module._fpq_weight_group_hook = module.register_load_state_dict_post_hook(build)


def _group_linear(layers, x: torch.Tensor, group=None):
    """The outputs of `layers` on `x` from ONE operator: one quantization and, where the layers' packed
    weights lie end to end (`group`, a WeightGroup), one GEMM whose column ranges are the outputs; else
    one GEMM each."""
    first = layers[0]
    if group is not None:
        outs = _eager().linear_cat_w4a4_op(x.reshape(-1, x.shape[-1]), first.forward_hadamard_matrix, group.wp,
                                           group.wsp, group.splits, first.weight_global_scale,
                                           first.act_global_scale, group.bias, group.nvfp4)
        return [o.view(*x.shape[:-1], o.shape[-1]) for o in outs]
    outs = _eager().linear_group_w4a4_op(
        x.reshape(-1, x.shape[-1]), first.forward_hadamard_matrix, [l.qweight for l in layers],
        [l.scales for l in layers], [l.weight_global_scale for l in layers], [l.act_global_scale for l in layers],
        [l.bias for l in layers], first.config.forward_dtype == FPQuantDtype.NVFP4)
    return [o.view(*x.shape[:-1], o.shape[-1]) for o in outs]


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
    down_proj = parts[2]
    # what the traced form needs on top: gate/up quantize alike, a SiLU*up quantizer for down's rotation
    traceable = False
    if down_proj.forward_hadamard_matrix.is_cuda:
        eager = _eager()
        kind, _ = eager.classify_rotation(eager.as_bf16(down_proj.forward_hadamard_matrix))
        g = down_proj.forward_hadamard_matrix.shape[0]
        traceable = (_quantize_alike(parts[:2]) and kind in (eager._engine.ROT_HADAMARD, eager._engine.ROT_IDENTITY)
                     and down_proj.in_features % max(g, 32) == 0
                     and (down_proj.bias is None or (down_proj.bias.dtype == torch.bfloat16
                                                     and down_proj.bias.is_contiguous())))

    def forward(self, x, residual=None):
        """`residual`: added to the result (a fused decoder block passes its skip connection)."""
        if traceable and _traceable_call(x):
            # two operators: gate and up from one quantization of x; SiLU*up quantized as it is
            # formed and multiplied by down's weight
            gate, up = _group_linear((self.gate_proj, self.up_proj), x, self._fpq_weight_group)
            down = self.down_proj
            y = _eager().silu_mul_linear_w4a4_op(gate, up, down.forward_hadamard_matrix, down.qweight, down.scales,
                                                 down.weight_global_scale, down.act_global_scale, down.bias,
                                                 down.config.forward_dtype == FPQuantDtype.NVFP4)
            y = y.view(*x.shape[:-1], y.shape[-1])
            return y if residual is None else residual + y
        if not _fusable_call(x) or (residual is not None and not _fusable_call(residual)):
            y = unfused(x)
            return y if residual is None else residual + y
        pair = _eager_group_linear(self, (self.gate_proj, self.up_proj), x) if traceable else None
        if pair is not None:
            gate, up = pair            # both from one GEMM
        else:
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

    mlp._fpq_weight_group = None
    if traceable:
        _attach_weight_group(mlp, ("gate_proj", "up_proj"))   # gate/up as one GEMM where the format allows
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


class _ProjectionCalls(ast.NodeTransformer):
    """Replaces `self.<q|k|v>_proj(hidden_states)` by the names `__fpq_q`, `__fpq_k`, `__fpq_v`."""

    def __init__(self):
        self.seen = []

    def visit_Call(self, node):
        self.generic_visit(node)
        f = node.func
        if (isinstance(f, ast.Attribute) and isinstance(f.value, ast.Name) and f.value.id == "self"
                and f.attr in ("q_proj", "k_proj", "v_proj") and len(node.args) == 1 and not node.keywords
                and isinstance(node.args[0], ast.Name) and node.args[0].id == "hidden_states"):
            self.seen.append(f.attr)
            return ast.copy_location(ast.Name(id="__fpq_" + f.attr[0], ctx=ast.Load()), node)
        return node


def _eager_group_linear(owner: nn.Module, layers, x: torch.Tensor):
    """Eager counterpart of _group_linear for layers with a WeightGroup: one GEMM (the quantized form of
    `x` is taken from, or left in, the sharing slot); None if there is no group.  The group kept on
    `owner` is checked against the layers' tensors as they are now and rebuilt if they were written to."""
    group = getattr(owner, "_fpq_weight_group", None)
    if group is None:
        return None
    first = layers[0]
    if group.key != tuple(_eager()._member_key(l.qweight, l.scales, l.bias) for l in layers):
        group = owner._fpq_weight_group = _weight_group(layers, create=True, previous=group)
        if group is None:
            return None
    eager = _eager()
    x_flat = x.reshape(-1, x.shape[-1])
    if not x_flat.is_contiguous():
        return None
    outs = eager.linear_cat(x_flat, first.forward_hadamard_matrix, group,
                            eager.linear_alpha(first.weight_global_scale, first.act_global_scale), shared_source=x,
                            act_global_scale=first.act_global_scale)
    lead = x.shape[:-1]
    return [o.view(*lead, o.shape[-1]) for o in outs]


def _qkv(attn, hidden_states):
    """q, k and v projections of `hidden_states`: from one operator when a compiler is tracing
    (which cannot see that the three layers quantize the same tensor); from one GEMM on the layers'
    concatenated packed weights in eager calls that have them; else three ordinary calls (which
    share the quantization by themselves)."""
    layers = (attn.q_proj, attn.k_proj, attn.v_proj)
    if attn._fpq_qkv_alike and _traceable_call(hidden_states):
        return _group_linear(layers, hidden_states, attn._fpq_weight_group)
    if attn._fpq_qkv_alike and _fusable_call(hidden_states):
        outs = _eager_group_linear(attn, layers, hidden_states)
        if outs is not None:
            return outs
    return attn.q_proj(hidden_states), attn.k_proj(hidden_states), attn.v_proj(hidden_states)


def fuse_qkv(attn: nn.Module) -> bool:
    """Give a traced attention module one operator for its q/k/v projections.  The module's own
    `forward` is kept: its source is re-compiled with the three calls `self.q_proj(hidden_states)`,
    `self.k_proj(hidden_states)`, `self.v_proj(hidden_states)` -- which must sit in three consecutive
    statements -- reading the results of one grouped call placed in front of them.  False (nothing
    changed) if the forward does not have that shape or the layers do not quantize alike."""
    layers = [getattr(attn, n, None) for n in ("q_proj", "k_proj", "v_proj")]
    if not all(_is_real_quant_linear(l) for l in layers):
        return False
    if getattr(attn, "_fpq_unfused_forward", None) is not None:
        return True
    fn = type(attn).forward
    if "forward" in vars(attn) or getattr(fn, "__closure__", None) or hasattr(fn, "__wrapped__"):
        return False
    try:
        tree = ast.parse(textwrap.dedent(inspect.getsource(fn)))
    except (OSError, TypeError, SyntaxError):
        return False
    fdef = tree.body[0] if tree.body and isinstance(tree.body[0], ast.FunctionDef) else None
    if fdef is None or fdef.decorator_list or "super" in ast.unparse(fdef):
        return False
    hits = []
    for i, stmt in enumerate(fdef.body):
        rewriter = _ProjectionCalls()
        fdef.body[i] = rewriter.visit(stmt)
        if rewriter.seen:
            hits.append((i, rewriter.seen))
    if ([h[1] for h in hits] != [["q_proj"], ["k_proj"], ["v_proj"]]
            or [h[0] for h in hits] != list(range(hits[0][0], hits[0][0] + 3))):
        return False
    # (the helper is reached through `self`: a name added to a copy of the module's globals would be
    # invisible to a tracer that resolves globals through the module itself)
    grouped = ast.parse("__fpq_q, __fpq_k, __fpq_v = self._fpq_qkv(hidden_states)").body[0]
    fdef.body.insert(hits[0][0], grouped)
    fdef.name = "forward"
    ast.fix_missing_locations(tree)
    namespace = dict(fn.__globals__)
    try:
        exec(compile(tree, f"<{type(attn).__qualname__}.forward with grouped q/k/v>", "exec"), namespace)
    except Exception:
        return False
    attn._fpq_qkv_alike = _quantize_alike(layers)
    attn._fpq_weight_group = None
    if attn._fpq_qkv_alike:
        _attach_weight_group(attn, ("q_proj", "k_proj", "v_proj"))   # q/k/v as one GEMM where the format allows
    attn._fpq_qkv = types.MethodType(_qkv, attn)
    attn._fpq_unfused_forward = attn.forward
    attn.forward = types.MethodType(namespace["forward"], attn)
    return True


def fuse_producers(model: nn.Module) -> int:
    """Apply fuse_rmsnorm / fuse_gated_mlp / fuse_residual_adds / fuse_qkv to every decoder block of `model` that
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
        count += int(fuse_qkv(attn))
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
            hook = getattr(module, "_fpq_weight_group_hook", None)
            if hook is not None:
                hook.remove()
                module._fpq_weight_group_hook = None
                module._fpq_weight_group_build = None
            if hasattr(module, "_fpq_weight_group"):
                module._fpq_weight_group = None
