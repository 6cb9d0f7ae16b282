"""The eager (non-traced) body of FPQuantLinear.forward and what hangs off it.

* `linear_w4a4`: activation rotate+quantize and W4A4 GEMM of one linear with as little host work
  as possible (same kernels and results as the `fp_quant::*` operators of hip_ops, which tracing
  uses; the reference's counterpart is FPQuant4x16NoMasterFn.forward,
  inference_lib/src/fp_quant/module/linear_fns.py:482-534).
* `QuantizedActivations` and the sharing slot: layers that consume the same tensor quantize it once
  (the reference keeps one activation quantizer per such group, src/utils/llama_utils.py:30,103).
* `rmsnorm_quantize`, `silu_mul_quantize`: the quantizers fused with the producer of their input.
"""
import ctypes
import os
import weakref
from typing import List, Optional, Tuple

import torch

from .. import _engine
from .hip_ops import (
    ZERO_NIBBLE_POLICY,
    _current_stream,
    _version,
    as_bf16,
    classify_rotation,
    is_packed_only,
    nv_packed_eligible,
    on_device,
    pack_mxf4,
    pack_nvf4,
    packed_linear_eligible,
    packed_weight,
    packed_weight_ready,
    packed_weights_enabled,
    quantize_mx_packed,
    splitk_workspace,
    SPLIT_K_MAX_ROWS,
    SPLIT_K_ROWS,
    unpack_fp4,
    weight_rows,
)


def cached_on(t: torch.Tensor, slot: str, key, make, remember: bool = True, refresh: bool = False):
    """`make()` remembered on tensor `t` under attribute `slot` while `key` stays the same.
    `remember=False` uses what is remembered but stores nothing new: for callers that may be running
    inside a compiler's graph memory pool, where a tensor that outlives the call is an error.
    `refresh`: make it anew whatever the key says.  A remembered tensor that is outdated is overwritten
    in place where that is possible, so that a recorded graph, which holds its address, reads the new value."""
    hit = getattr(t, slot, None)
    if hit is not None and hit[0] == key and not refresh:
        return hit[1]
    val = make()
    if remember:
        old = hit[1] if hit is not None else None
        if (isinstance(old, torch.Tensor) and isinstance(val, torch.Tensor) and old.shape == val.shape
                and old.dtype == val.dtype and old.device == val.device and old is not val
                and not torch.cuda.is_current_stream_capturing()):
            try:
                old.copy_(val)
                val = old
            except RuntimeError:   # (an inference tensor outside inference mode: replaced instead)
                pass
        try:
            setattr(t, slot, (key, val))
        except (AttributeError, RuntimeError):
            pass
    return val


def linear_alpha(weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor,
                 remember: bool = True, refresh: bool = False) -> torch.Tensor:
    """fp32 one-element `1 / (wgs * ags)` evaluated in the buffers' dtype as the reference does
    (linear_fns.py:505; bf16 buffers round 1/9 to 0.111328125), cached until a buffer changes."""
    key = (_version(weight_global_scale), _version(act_global_scale), act_global_scale.data_ptr(),
           weight_global_scale.data_ptr())
    return cached_on(weight_global_scale, "_fpq_alpha", key,
                     lambda: (1.0 / (weight_global_scale * act_global_scale)).float().reshape(1).contiguous(),
                     remember, refresh)


def as_f32_scalar(t: torch.Tensor, remember: bool = True, refresh: bool = False) -> torch.Tensor:
    if t.dtype == torch.float32 and t.is_contiguous():
        return t
    return cached_on(t, "_fpq_f32", (_version(t), t.data_ptr()), lambda: t.detach().float().contiguous(), remember,
                     refresh)


# Several layers that consume one tensor (q/k/v projections, gate/up projections) would rotate and
# quantize it once each.  The quantized activations of the latest call are kept per device and reused
# while the next call passes the very same tensor object, unmodified (its version counter), with an
# equal rotation and global scale, on the same stream and in the same graph capture (or both outside
# any: work recorded during a capture has not run when the capture ends).  The source is held weakly,
# so a freed tensor whose address is reused can never match, and the entry goes away with it.
# Producers fused with the quantizer (rmsnorm_quantize, silu_mul_quantize) leave their result in the
# same slot for the layers that follow.  The version counter only sees writes made through PyTorch:
# compiled callers (whose generated kernels overwrite reused buffers behind it) never share, and a
# stack that updates activations in place with raw-pointer kernels must set FPQ_SHARE_ACT_QUANT=0.
SHARE_ACT_QUANT = os.environ.get("FPQ_SHARE_ACT_QUANT", "1") != "0"


class QuantizedActivations:
    """Rotated and quantized activations of one [m, k] tensor, in whichever operand layouts have
    been asked for so far (row-major codes/scales, packed MXFP4, packed NVFP4)."""
    __slots__ = ("m", "k", "nvfp4", "ref", "version", "key", "keep", "mx_packed", "row_major", "nv_packed")

    def __init__(self, m: int, k: int, nvfp4: bool):
        self.m, self.k, self.nvfp4 = m, k, nvfp4
        self.ref = self.key = self.keep = None
        self.version = 0
        self.mx_packed = self.row_major = self.nv_packed = None

    def serves(self, want_packed: bool) -> bool:
        """Whether a GEMM on packed (or on row-major) operands can run from what is held: either form
        is made from the other on demand (a re-tiling pass over the 4-bit codes, exact both ways)."""
        return self.row_major is not None or self.mx_packed is not None or self.nv_packed is not None

    def rows(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Row-major codes [m, k/2] and scales (unpacked from the packed form if that is all there is)."""
        if self.row_major is None:
            pc, ps = self.nv_packed if self.nvfp4 else self.mx_packed
            self.row_major = unpack_fp4(pc, ps, self.m, self.k, self.nvfp4)
        return self.row_major

    def packed(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Codes and scales in the packed GEMM layout (re-tiled from the row-major ones if need be)."""
        if self.nvfp4:
            if self.nv_packed is None:
                self.nv_packed = pack_nvf4(self.row_major[0], self.row_major[1], self.m, self.k)
            return self.nv_packed
        if self.mx_packed is None:
            self.mx_packed = pack_mxf4(self.row_major[0], self.row_major[1], self.m, self.k)
        return self.mx_packed


_shared_activations = {}   # device index -> QuantizedActivations of the latest call


def _sharing_key(x_shape, h, kind: int, norm: float, act_global_scale, stream: int, quest: bool = False):
    """What two calls must agree on, besides the source tensor, to share quantized activations, or
    None when nothing may be shared.  Layers own separate but equal rotation and global-scale
    buffers, so those are compared by value: (kind, norm, size) of a recognised rotation, the host
    copy of the scale (read once per buffer); an unrecognised rotation matrix only matches itself."""
    if not SHARE_ACT_QUANT or torch.is_inference_mode_enabled():
        return None   # in inference mode in-place writes to the source could not be noticed
    capture = 0
    if torch.cuda.is_current_stream_capturing():   # (`stream` is the current stream; the cheap test first)
        capture_id = ctypes.c_ulonglong()   # per call: host threads may run layers concurrently
        _engine.check(_engine.lib().fpq_stream_capture_id(stream, ctypes.byref(capture_id)), "fpq_stream_capture_id")
        capture = capture_id.value
    rot = (kind, norm, h.shape[0]) if kind != _engine.ROT_GENERAL else (kind, id(h), _version(h))
    gs = None
    if act_global_scale is not None:
        gs = cached_on(act_global_scale, "_fpq_host", (_version(act_global_scale), act_global_scale.data_ptr()),
                       lambda: float(act_global_scale))
    return (rot, gs, stream, capture, tuple(x_shape), quest)


def _publish(qa: QuantizedActivations, src: torch.Tensor, key, keep) -> None:
    dev = src.device.index

    def source_died(ref, dev=dev):
        # nobody can ask for this tensor's quantized form any more: give the memory back now (a graph
        # capture's memory pool must hold nothing but the captured step's outputs when it ends)
        slot = _shared_activations.get(dev)
        if slot is not None and slot.ref is ref:
            del _shared_activations[dev]

    qa.ref, qa.version, qa.key, qa.keep = weakref.ref(src, source_died), _version(src), key, keep
    _shared_activations[dev] = qa


def _lookup(src: torch.Tensor, key, want_packed: bool) -> Optional[QuantizedActivations]:
    qa = _shared_activations.get(src.device.index)
    if (qa is not None and qa.ref() is src and qa.version == _version(src) and qa.key == key
            and qa.serves(want_packed)):
        return qa
    return None


def quantize_activations(x_flat: torch.Tensor, h: torch.Tensor, kind: int, norm: float,
                         act_global_scale: Optional[torch.Tensor], nvfp4: bool, stream: int,
                         want_packed: bool, remember: bool = True, quest: bool = False) -> QuantizedActivations:
    """Rotate and quantize bf16 [m, k]: straight into the packed layout when the packed GEMM will run
    (row-major first, re-tiled on demand, for the rotations the packed quantizers do not take), row-major
    otherwise."""
    lib = _engine.lib()
    m, k = x_flat.shape
    dev = x_flat.device
    g = h.shape[0]
    qa = QuantizedActivations(m, k, nvfp4)
    if quest and want_packed:
        pc = torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes(m, k), dtype=torch.uint8, device=dev)
        st = lib.fpq_quantize_mx_quest_packed(x_flat.data_ptr(), m, k, kind, g, norm, pc.data_ptr(), ps.data_ptr(),
                                              ZERO_NIBBLE_POLICY, stream)
        if st != _engine.E_UNSUPPORTED:
            _engine.check(st, "fpq_quantize_mx_quest_packed")
            qa.mx_packed = (pc, ps)
            return qa
    if quest:
        # rotations the packed kernel does not take: row-major, the packed form is made from it on demand
        codes = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
        scales = torch.empty(m, k // 32, dtype=torch.uint8, device=dev)
        st = lib.fpq_quantize_mx_quest(x_flat.data_ptr(), m, k, kind, g, norm, h.data_ptr(), codes.data_ptr(),
                                       scales.data_ptr(), m, k // 32, None, ZERO_NIBBLE_POLICY, stream)
        _engine.check(st, "fpq_quantize_mx_quest")
        qa.row_major = (codes, scales)
        return qa
    if want_packed and not nvfp4:
        pc = torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes(m, k), dtype=torch.uint8, device=dev)
        st = lib.fpq_quantize_mx_packed(x_flat.data_ptr(), m, k, kind, g, norm, pc.data_ptr(), ps.data_ptr(),
                                        ZERO_NIBBLE_POLICY, stream)
        if st == _engine.E_UNSUPPORTED:
            pc, ps = quantize_mx_packed(x_flat, h)
        else:
            _engine.check(st, "fpq_quantize_mx_packed")
        qa.mx_packed = (pc, ps)
        return qa
    if nvfp4 and want_packed:
        pc = torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes_nv(m, k), dtype=torch.uint8, device=dev)
        gs = as_f32_scalar(act_global_scale, remember)
        st = lib.fpq_quantize_nv_packed(x_flat.data_ptr(), m, k, kind, g, norm, gs.data_ptr(), pc.data_ptr(),
                                        ps.data_ptr(), ZERO_NIBBLE_POLICY, stream)
        if st != _engine.E_UNSUPPORTED:
            _engine.check(st, "fpq_quantize_nv_packed")
            qa.nv_packed = (pc, ps)
            return qa
    group = 16 if nvfp4 else 32
    codes = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(m, k // group, dtype=torch.uint8, device=dev)
    if nvfp4:
        gs = as_f32_scalar(act_global_scale, remember)
        st = lib.fpq_quantize_nv(x_flat.data_ptr(), m, k, kind, g, norm, h.data_ptr(), gs.data_ptr(),
                                 codes.data_ptr(), scales.data_ptr(), m, k // group, ZERO_NIBBLE_POLICY, stream)
        _engine.check(st, "fpq_quantize_nv")
    else:
        st = lib.fpq_quantize_mx(x_flat.data_ptr(), m, k, kind, g, norm, h.data_ptr(), codes.data_ptr(),
                                 scales.data_ptr(), m, k // group, ZERO_NIBBLE_POLICY, stream)
        _engine.check(st, "fpq_quantize_mx")
    qa.row_major = (codes, scales)
    return qa


def wants_packed(m: int, n: int, k: int, nvfp4: bool) -> bool:
    """Whether the GEMM of an [m, k] x [n, k] linear runs on packed operands."""
    return nv_packed_eligible(m, n, k, fused_linear=True) if nvfp4 else packed_linear_eligible(m, k, "abs_max")


def weight_wants_packed(wq: torch.Tensor, m: int, k: int, nvfp4: bool) -> bool:
    """wants_packed for the weight `wq`: always for one that is held in the packed layout only."""
    return True if is_packed_only(wq) else wants_packed(m, wq.shape[0], k, nvfp4)


def linear_on(qa: QuantizedActivations, wq: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
              bias: Optional[torch.Tensor], stream: int, use_packed: Optional[bool] = None,
              residual: Optional[torch.Tensor] = None,
              packed: Optional[Tuple[torch.Tensor, torch.Tensor, int]] = None,
              remember: bool = False) -> torch.Tensor:
    """bf16 [m, n] = alpha * dq(activations) @ dq(w).T (+ bias) on quantized activations, with the
    kernel and operand layout the shape calls for (`use_packed`: the caller's decision, if it has
    made it already).  `residual` (bf16 [m, n]) is added as a separate bf16 addition would add it:
    inside the packed kernels' epilogue, by a PyTorch addition after the other kernels.  `remember`: the
    call may create and keep what the layer lacks (its split-K workspace)."""
    lib = _engine.lib()
    m, k = qa.m, qa.k
    if packed is not None:   # packed MXFP4 weights of `n` rows handed in directly (a WeightGroup): wq, ws unused
        wp, wsp, n = packed
        if wp.numel() * 2 != n * k:
            raise ValueError("packed weights need activations with the same inner dimension")
        use_packed = True
    elif is_packed_only(wq):   # a layer that holds its weight in the packed layout only
        n = weight_rows(wq, k)
        wp = wsp = None
        use_packed = True
    else:
        n = wq.shape[0]
        if wq.shape[1] * 2 != k:
            raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
        wp = wsp = None
    dev = wp.device if packed is not None else wq.device
    y = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    b_ptr = bias.data_ptr() if bias is not None else None
    if residual is not None and (residual.dtype != torch.bfloat16 or residual.numel() != m * n
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be a contiguous bfloat16 tensor of the output's size on the same device")
    if residual is not None and residual.device != dev:
        raise ValueError("residual must be on the weights' device")
    if use_packed is None:
        use_packed = wants_packed(m, n, k, qa.nvfp4)
    if qa.nvfp4:
        if use_packed:
            xp, xsp = qa.packed()
            if packed is None:
                wp, wsp = packed_weight(wq, ws, True)
            # (NVFP4 runs 129-256 rows as two passes of the kernel that can split K: each may use the workspace;
            # beyond, the tile kernels split K where that fills the CUs)
            workspace = (splitk_workspace(wq, n, k, remember, stream, True)
                         if (m <= SPLIT_K_MAX_ROWS and packed is None) else None)
            if workspace is not None:
                st = lib.fpq_gemm_nvf4_packed_splitk(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                     alpha.data_ptr(), b_ptr,
                                                     residual.data_ptr() if residual is not None else None,
                                                     y.data_ptr(), m, n, k, workspace.data_ptr(), workspace.numel(),
                                                     stream)
                _engine.check(st, "fpq_gemm_nvf4_packed_splitk")
                return y
            if residual is not None:
                st = lib.fpq_gemm_nvf4_packed_residual(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                       alpha.data_ptr(), b_ptr, residual.data_ptr(), y.data_ptr(),
                                                       m, n, k, stream)
                _engine.check(st, "fpq_gemm_nvf4_packed_residual")
                return y
            st = lib.fpq_gemm_nvf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                          alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
            _engine.check(st, "fpq_gemm_nvf4_packed")
        else:
            codes, scales = qa.rows()
            st = lib.fpq_gemm_nvf4(codes.data_ptr(), scales.data_ptr(), scales.shape[-1], wq.data_ptr(),
                                   ws.data_ptr(), ws.shape[-1], alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
            _engine.check(st, "fpq_gemm_nvf4")
        if residual is not None:
            y += residual
        return y
    if use_packed:
        pc, ps = qa.packed()
        if packed is None:
            wp, wsp = packed_weight(wq, ws)
        workspace = splitk_workspace(wq, n, k, remember, stream) if (m <= SPLIT_K_ROWS and packed is None) else None
        if workspace is not None:
            # few weight rows and a long K at decode sizes: K split across workgroups (deterministic sum)
            st = lib.fpq_gemm_mxf4_packed_splitk(pc.data_ptr(), ps.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                 alpha.data_ptr(), b_ptr,
                                                 residual.data_ptr() if residual is not None else None, y.data_ptr(),
                                                 m, n, k, workspace.data_ptr(), workspace.numel(), stream)
        elif residual is not None:
            st = lib.fpq_gemm_mxf4_packed_residual(pc.data_ptr(), ps.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                   alpha.data_ptr(), b_ptr, residual.data_ptr(), y.data_ptr(),
                                                   m, n, k, stream)
        else:
            st = lib.fpq_gemm_mxf4_packed(pc.data_ptr(), ps.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                          alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
        _engine.check(st, "fpq_gemm_mxf4_packed")
        return y
    codes, scales = qa.rows()
    st = lib.fpq_gemm_mxf4(codes.data_ptr(), scales.data_ptr(), scales.shape[-1], wq.data_ptr(), ws.data_ptr(),
                           ws.shape[-1], alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
    _engine.check(st, "fpq_gemm_mxf4")
    if residual is not None:
        y += residual
    return y


def linear_w4a4(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor,
                alpha: torch.Tensor, act_global_scale: torch.Tensor, bias: Optional[torch.Tensor],
                nvfp4: bool, shared_source: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None, remember: bool = True,
                quest: bool = False) -> torch.Tensor:
    """Activation rotate+quantize and W4A4 GEMM of one linear with as little host work as possible:
    the eager (non-traced) body of FPQuantLinear.forward.  Same kernels and results as the
    fused_quantize_* and matmul_* operators; `x_flat` bf16 [M, K] contiguous on the GPU, `alpha`
    fp32 [1], `bias` bf16 [N] or None.  `shared_source` is the tensor object `x_flat` was derived
    from: consecutive calls with the same, unmodified object reuse its quantized form."""
    if not x_flat.is_cuda:
        raise ValueError("fp_quant HIP operators need tensors on a GPU; there is no CPU path")
    dev = x_flat.device
    if torch.cuda.current_device() != dev.index:
        with on_device(dev):
            return linear_w4a4(x_flat, hadamard_matrix, wq, ws, alpha, act_global_scale, bias, nvfp4, shared_source,
                               residual, remember, quest)
    stream = _current_stream(dev.index)
    h = as_bf16(hadamard_matrix)
    kind, norm = classify_rotation(h)
    m, k = x_flat.shape
    want_packed = weight_wants_packed(wq, m, k, nvfp4)
    if want_packed and not remember and not packed_weight_ready(wq, ws, nvfp4):
        want_packed = False   # no packed copy of the weight yet and none may be kept: row-major kernels
    qa = key = None
    if shared_source is not None:
        key = _sharing_key(x_flat.shape, h, kind, norm, act_global_scale if nvfp4 else None, stream, quest)
        if key is not None:
            qa = _lookup(shared_source, key, want_packed)
    if qa is not None:
        if nvfp4:
            as_f32_scalar(act_global_scale)   # remembered now: a later traced call must not have to create it
    else:
        qa = quantize_activations(x_flat, h, kind, norm, act_global_scale, nvfp4, stream, want_packed, remember,
                                  quest)
        if key is not None:
            _publish(qa, shared_source, key, h)
    return linear_on(qa, wq, ws, alpha, bias, stream, want_packed, residual, remember=remember)


@torch.library.custom_op("fp_quant::linear_w4a4_op", mutates_args=())
def linear_w4a4_op(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor,
                   weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor,
                   bias: Optional[torch.Tensor], nvfp4: bool, quest: bool = False) -> torch.Tensor:
    """The whole abs-max forward of one layer as ONE operator, for traced callers (torch.compile):
    inside it runs exactly what an eager call runs (linear_w4a4: cached alpha, packed or row-major
    kernels by shape; no sharing of quantized activations between layers), so a compiled model gives the eager model's
    bits and a captured step holds two kernels per layer instead of the reference's operator chain
    (quantize, four tiny kernels for alpha, GEMM; linear_fns.py:496-514).  The global scales are read
    when the operator runs; a HIP graph recorded around it replays the alpha it was recorded with."""
    x = x_flat if x_flat.is_contiguous() else x_flat.contiguous()
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor")
    if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector")
    # Nothing created here may outlive the call (the compiler may be running it inside its graph
    # memory pool): what `prime` or eager calls have remembered is used, nothing new is remembered.
    # No shared_source: compiler-generated kernels rewrite reused buffers without touching the
    # version counter that sharing relies on.
    alpha = linear_alpha(weight_global_scale, act_global_scale, remember=False)
    return linear_w4a4(x, hadamard_matrix, wq.contiguous(), ws.contiguous(), alpha, act_global_scale, bias, nvfp4,
                       remember=False, quest=quest)


# Layers fed by one tensor (q/k/v, gate/up) as ONE GEMM.  In the packed layout a weight is a sequence of
# 32-row tiles, so the packed weights of several layers with the same K, laid end to end, are the packed
# weight of their concatenation along N: one launch computes [m, n_1 + n_2 + ...] and the layers' outputs
# are column slices of it.  The layers' own packed copies become views into the concatenated buffers, so
# no 4-bit weight is held a further time.  MXFP4 and NVFP4 (one format per group).
class WeightGroup:
    __slots__ = ("key", "wp", "wsp", "bias", "n", "splits", "k", "nvfp4")


def _member_key(wq: torch.Tensor, ws: torch.Tensor, bias: Optional[torch.Tensor]):
    # (a tensor of another shape has another address or another counter: the shape itself need not be compared)
    return (wq.data_ptr(), _version(wq), ws.data_ptr(), _version(ws),
            None if bias is None else (bias.data_ptr(), _version(bias)))


def weight_group(members, create: bool = False, nvfp4: bool = False,
                 previous: Optional["WeightGroup"] = None) -> Optional[WeightGroup]:
    """The WeightGroup of `members` = [(qweight, scales, bias or None, in_features), ...] (one format, same K,
    every N a multiple of 32, biases all absent or all contiguous bf16; weights row-major, or all in the packed
    layout only), remembered on the first member's qweight until a member is written to; built now if
    `create`, else None when there is none.  A group built in place of an outdated one of the same shape
    (`previous`, or the one remembered) is written into that one's buffers, so that the addresses a recorded
    graph holds stay those of the current weights."""
    first = members[0][0]
    key = tuple(_member_key(*m[:3]) for m in members)
    hit = getattr(first, "_fpq_group", None)
    if hit is not None and hit.key == key and hit.nvfp4 == nvfp4:
        return hit
    if previous is None:
        previous = hit
    if not create or not packed_weights_enabled():
        return None
    k = members[0][3]
    sgroup = 16 if nvfp4 else 32
    dev = first.device
    packed_only = is_packed_only(first)
    have_bias = [m[2] is not None for m in members]
    if k < 256 or k % 256 != 0:
        return None
    for wq, ws, bias, k_in in members:
        if (wq.dtype != torch.uint8 or ws.dtype != torch.uint8 or not wq.is_cuda or wq.device != dev or k_in != k
                or not wq.is_contiguous() or not ws.is_contiguous() or is_packed_only(wq) != packed_only):
            return None
        if packed_only:
            if ws.dim() != 1 or wq.numel() * 2 % (32 * k) != 0 or ws.numel() * (sgroup // 2) != wq.numel():
                return None
        elif (wq.dim() != 2 or wq.shape[1] * 2 != k or wq.shape[0] % 32 != 0
                or ws.shape != (wq.shape[0], k // sgroup)):
            return None
        if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous() or bias.device != dev):
            return None
    if any(have_bias) and not all(have_bias):
        return None
    lib = _engine.lib()
    splits = [weight_rows(m[0], k) for m in members]
    n = sum(splits)
    group = WeightGroup()
    group.n, group.splits, group.k, group.nvfp4 = n, splits, k, nvfp4
    scales_bytes = lib.fpq_packed_scales_bytes_nv if nvfp4 else lib.fpq_packed_scales_bytes
    pack = lib.fpq_pack_nvf4 if nvfp4 else lib.fpq_pack_mxf4
    reuse = previous
    if (reuse is not None and (reuse.nvfp4 != nvfp4 or reuse.k != k or reuse.splits != splits or reuse.wp.device != dev
                               or torch.cuda.is_current_stream_capturing())):
        reuse = None
    with on_device(dev):
        stream = _current_stream(dev.index)
        bounds, row = [], 0
        for rows in splits:
            bounds.append((lib.fpq_packed_codes_bytes(row, k), lib.fpq_packed_codes_bytes(row + rows, k),
                           scales_bytes(row, k), scales_bytes(row + rows, k)))
            row += rows
        if packed_only:
            in_place = reuse is not None and all(
                m[0].data_ptr() == reuse.wp.data_ptr() + b[0] and m[1].data_ptr() == reuse.wsp.data_ptr() + b[2]
                for m, b in zip(members, bounds))
            if in_place:     # the members already live in the outdated group's buffers (re-packed there)
                group.wp, group.wsp = reuse.wp, reuse.wsp
            else:
                # the members' buffers laid end to end; the members then live in the new buffers (views) and
                # their own are freed, so the weights are still held once
                group.wp = torch.cat([m[0] for m in members])
                group.wsp = torch.cat([m[1] for m in members])
        elif reuse is not None:
            group.wp, group.wsp = reuse.wp, reuse.wsp
        else:
            group.wp = torch.empty(lib.fpq_packed_codes_bytes(n, k), dtype=torch.uint8, device=dev)
            group.wsp = torch.empty(scales_bytes(n, k), dtype=torch.uint8, device=dev)
        for (wq, ws, _, _), rows, (c0, c1, s0, s1) in zip(members, splits, bounds):
            pc, ps = group.wp[c0:c1], group.wsp[s0:s1]
            if packed_only:
                if wq.data_ptr() != pc.data_ptr() or ws.data_ptr() != ps.data_ptr():
                    wq.data, ws.data = pc, ps
            else:
                st = pack(wq.data_ptr(), ws.data_ptr(), ws.shape[1], rows, k, pc.data_ptr(), ps.data_ptr(), stream)
                _engine.check(st, "fpq_pack")
                # the member's own packed copy: these views (same key as hip_ops.packed_weight uses)
                wq._fpq_packed = ((wq.data_ptr(), _version(wq), ws.data_ptr(), _version(ws), tuple(wq.shape), nvfp4), pc, ps)
    group.key = tuple(_member_key(*m[:3]) for m in members)   # (packed-only members have just moved)
    group.bias = torch.cat([m[2] for m in members]).contiguous() if all(have_bias) else None
    try:
        first._fpq_group = group
    except (AttributeError, RuntimeError):
        pass
    return group


def linear_on_group(qa: QuantizedActivations, wp: torch.Tensor, wsp: torch.Tensor, splits: List[int],
                    alpha: torch.Tensor, bias: Optional[torch.Tensor], stream: int) -> List[torch.Tensor]:
    """ONE GEMM of quantized activations with the packed MXFP4 weights of several layers laid end to end
    (`splits`: the layers' output features); returns the layers' outputs, bf16 [m, n_i] each.  Every
    layer gets a dense matrix of its own from the kernel when all n_i are multiples of 256; else the
    outputs are column ranges of one [m, sum n_i] matrix (rows keep the full stride)."""
    m, k, n = qa.m, qa.k, sum(splits)
    if wp.numel() * 2 != n * k:
        raise ValueError("packed weights need activations with the same inner dimension")
    if len(splits) > 4 or any(s % 256 for s in splits):
        y = linear_on(qa, None, None, alpha, bias, stream, True, packed=(wp, wsp, n))
        return list(y.split(splits, dim=1))
    lib = _engine.lib()
    pc, ps = qa.packed()
    outs = [torch.empty(m, s, dtype=torch.bfloat16, device=wp.device) for s in splits]
    count = len(splits)
    ys = (ctypes.c_void_p * count)(*[o.data_ptr() for o in outs])
    ns = (ctypes.c_int64 * count)(*splits)
    entry = lib.fpq_gemm_nvf4_packed_multi if qa.nvfp4 else lib.fpq_gemm_mxf4_packed_multi
    st = entry(pc.data_ptr(), ps.data_ptr(), wp.data_ptr(), wsp.data_ptr(), alpha.data_ptr(),
               bias.data_ptr() if bias is not None else None, ys, ns, count, m, k, stream)
    _engine.check(st, "fpq_gemm_packed_multi")
    return outs


def linear_cat(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, group: WeightGroup, alpha: torch.Tensor,
               shared_source: Optional[torch.Tensor] = None, remember: bool = True,
               act_global_scale: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
    """The layers of a WeightGroup on `x_flat` (bf16 [m, K], contiguous) from one quantization and ONE
    GEMM: bf16 [m, n_i] per layer (bias included).  `act_global_scale`: the layers' common activation
    scale (NVFP4 groups)."""
    dev = x_flat.device
    if torch.cuda.current_device() != dev.index:
        with on_device(dev):
            return linear_cat(x_flat, hadamard_matrix, group, alpha, shared_source, remember, act_global_scale)
    stream = _current_stream(dev.index)
    h = as_bf16(hadamard_matrix)
    kind, norm = classify_rotation(h)
    ags = act_global_scale if group.nvfp4 else None
    if group.nvfp4 and ags is None:
        raise ValueError("an NVFP4 group needs the activation global scale")
    qa = key = None
    if shared_source is not None:
        key = _sharing_key(x_flat.shape, h, kind, norm, ags, stream)
        if key is not None:
            qa = _lookup(shared_source, key, True)
    if qa is None:
        qa = quantize_activations(x_flat, h, kind, norm, ags, group.nvfp4, stream, True, remember)
        if key is not None:
            _publish(qa, shared_source, key, h)
    return linear_on_group(qa, group.wp, group.wsp, group.splits, alpha, group.bias, stream)


@torch.library.custom_op("fp_quant::linear_cat_w4a4_op", mutates_args=())
def linear_cat_w4a4_op(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, wp: torch.Tensor, wsp: torch.Tensor,
                       splits: List[int], weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor,
                       bias: Optional[torch.Tensor], nvfp4: bool = False) -> List[torch.Tensor]:
    """linear_cat for traced callers: the packed weights of a WeightGroup (made when the model was
    patched, outside any trace) times the activations quantized once; bf16 [m, n_i] per layer."""
    x = x_flat if x_flat.is_contiguous() else x_flat.contiguous()
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor on a GPU")
    n = sum(splits)
    if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous() or bias.numel() != n):
        raise ValueError("bias must be a contiguous bfloat16 vector of sum(splits) elements")
    dev = x.device
    with on_device(dev):
        stream = _current_stream(dev.index)
        h = as_bf16(hadamard_matrix)
        kind, norm = classify_rotation(h)
        alpha = linear_alpha(weight_global_scale, act_global_scale, remember=False)
        qa = quantize_activations(x, h, kind, norm, act_global_scale if nvfp4 else None, nvfp4, stream, True,
                                  remember=False)
        outs = linear_on_group(qa, wp, wsp, list(splits), alpha, bias, stream)
        # operators return tensors that own their memory: column ranges of one matrix are copied out
        return [o.clone() if o._is_view() else o for o in outs]


@linear_cat_w4a4_op.register_fake
def _(x_flat, hadamard_matrix, wp, wsp, splits, weight_global_scale, act_global_scale, bias, nvfp4=False):
    return [x_flat.new_empty((x_flat.shape[0], s), dtype=torch.bfloat16) for s in splits]


# Traced callers, groups of layers.  A compiler cannot see that q/k/v (or gate/up) quantize the same
# tensor, and the sharing slot is closed to it; these operators state the grouping instead.
@torch.library.custom_op("fp_quant::linear_group_w4a4_op", mutates_args=())
def linear_group_w4a4_op(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, wqs: List[torch.Tensor],
                         wss: List[torch.Tensor], weight_global_scales: List[torch.Tensor],
                         act_global_scales: List[torch.Tensor], biases: List[Optional[torch.Tensor]],
                         nvfp4: bool) -> List[torch.Tensor]:
    """Several layers on one input: the activations are rotated and quantized once (with the first
    layer's rotation and activation scale, which the caller has checked to equal the others'), then
    one GEMM per layer -- what consecutive eager calls do through the sharing slot."""
    x = x_flat if x_flat.is_contiguous() else x_flat.contiguous()
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_cuda:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor on a GPU")
    n_layers = len(wqs)
    if not (len(wss) == len(weight_global_scales) == len(act_global_scales) == len(biases) == n_layers) or not n_layers:
        raise ValueError("one entry per layer is needed in every list")
    dev = x.device
    with on_device(dev):
        stream = _current_stream(dev.index)
        h = as_bf16(hadamard_matrix)
        kind, norm = classify_rotation(h)
        m, k = x.shape
        # a GEMM runs on packed operands where the shape calls for it and the packed weight exists
        # already (nothing may be created and kept here); the activations are quantized straight into
        # the packed layout only if every GEMM of the group wants them so (MXFP4), else row-major,
        # from which the packed form is made on demand
        packed = [weight_wants_packed(wq, m, k, nvfp4) and packed_weight_ready(wq, ws, nvfp4)
                  for wq, ws in zip(wqs, wss)]
        qa = quantize_activations(x, h, kind, norm, act_global_scales[0], nvfp4, stream,
                                  all(packed) and not nvfp4, remember=False)
        out = []
        for i in range(n_layers):
            bias = biases[i]
            if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
                raise ValueError("bias must be a contiguous bfloat16 vector")
            alpha = linear_alpha(weight_global_scales[i], act_global_scales[i], remember=False)
            out.append(linear_on(qa, wqs[i].contiguous(), wss[i].contiguous(), alpha, bias, stream, packed[i]))
    return out


@linear_group_w4a4_op.register_fake
def _(x_flat, hadamard_matrix, wqs, wss, weight_global_scales, act_global_scales, biases, nvfp4):
    return [x_flat.new_empty((x_flat.shape[0], weight_rows(wq, x_flat.shape[1])), dtype=torch.bfloat16) for wq in wqs]


@torch.library.custom_op("fp_quant::silu_mul_linear_w4a4_op", mutates_args=())
def silu_mul_linear_w4a4_op(gate: torch.Tensor, up: torch.Tensor, hadamard_matrix: torch.Tensor, wq: torch.Tensor,
                            ws: torch.Tensor, weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor,
                            bias: Optional[torch.Tensor], nvfp4: bool) -> torch.Tensor:
    """down(bf16(silu(gate)) * up) of a gated MLP: the product is quantized as it is formed
    (silu_mul_quantize) and multiplied by the layer's weight; bf16 [m, n]."""
    g2, u2 = gate.reshape(-1, gate.shape[-1]), up.reshape(-1, up.shape[-1])
    wq, ws = wq.contiguous(), ws.contiguous()
    # packed operands only where the packed weight exists already: nothing may be created and kept here
    ready = packed_weight_ready(wq, ws, nvfp4)
    qa = silu_mul_quantize(g2, u2, hadamard_matrix, act_global_scale, nvfp4, remember=False, allow_packed=ready)
    if qa is None:
        raise ValueError("no fused SiLU*up quantizer for these tensors (rotation, strides or alignment)")
    if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector")
    dev = gate.device
    with on_device(dev):
        alpha = linear_alpha(weight_global_scale, act_global_scale, remember=False)
        use_packed = ready and weight_wants_packed(wq, qa.m, qa.k, nvfp4)
        return linear_on(qa, wq, ws, alpha, bias, _current_stream(dev.index), use_packed)


@silu_mul_linear_w4a4_op.register_fake
def _(gate, up, hadamard_matrix, wq, ws, weight_global_scale, act_global_scale, bias, nvfp4):
    rows = gate.numel() // gate.shape[-1]
    return gate.new_empty((rows, weight_rows(wq, gate.shape[-1])), dtype=torch.bfloat16)


def prime(hadamard_matrix: torch.Tensor, weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor,
          refresh: bool = False) -> None:
    """Compute and remember a layer's per-call constants (rotation kind, alpha, fp32 global scale) now,
    in ordinary memory: afterwards neither a traced call nor a graph capture has to create them.
    `refresh`: the buffers may have been rewritten behind their modification counters; alpha and the fp32
    scale are computed anew (into the tensors that held them)."""
    if not weight_global_scale.is_cuda or hadamard_matrix.device != weight_global_scale.device:
        return
    classify_rotation(as_bf16(hadamard_matrix))
    linear_alpha(weight_global_scale, act_global_scale, refresh=refresh)
    as_f32_scalar(act_global_scale, refresh=refresh)
    prepare_device(weight_global_scale.device)


_prepared_devices = set()


def prepare_device(device: torch.device) -> None:
    """The library's per-device set-up (silu lookup table, scratch address), once per device and outside
    any graph capture, so that no later call has to build it on a stream that is being recorded."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index in _prepared_devices:
        return
    with torch.cuda.device(index):
        stream = _current_stream(index)
        st = _engine.lib().fpq_prepare_device(stream)
    if st == _engine.E_UNSUPPORTED:   # called under a capture: a later call outside one does it
        return
    _engine.check(st, "fpq_prepare_device")
    _prepared_devices.add(index)


@linear_w4a4_op.register_fake
def _(x_flat, hadamard_matrix, wq, ws, weight_global_scale, act_global_scale, bias, nvfp4, quest=False):
    return x_flat.new_empty((x_flat.shape[0], weight_rows(wq, x_flat.shape[1])), dtype=torch.bfloat16)


### Quantizers fused with the producer of their input


def _fused_quantize(entry: str, head: tuple, rows: int, cols: int, h: torch.Tensor, kind: int, norm: float,
                    act_global_scale: Optional[torch.Tensor], nvfp4: bool, out: Optional[torch.Tensor],
                    stream: int, dev, remember: bool = True,
                    allow_packed: bool = True) -> Optional[QuantizedActivations]:
    """Common tail of the fused producers: allocate row-major codes/scales and call
    fpq_<entry>_quantize_{mx,nv}; None if the library has no fused kernel for this rotation."""
    lib = _engine.lib()
    group = 16 if nvfp4 else 32
    optr = out.data_ptr() if out is not None else None
    want_packed = allow_packed and not nvfp4 and packed_linear_eligible(rows, cols, "abs_max")
    if want_packed:
        # straight into the operand layout of the packed GEMM (streaming kernel)
        pc = torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes(rows, cols), dtype=torch.uint8, device=dev)
        st = getattr(lib, f"fpq_{entry}_quantize_mx_packed")(*head, rows, cols, kind, h.shape[0], norm, optr,
                                                             pc.data_ptr(), ps.data_ptr(), ZERO_NIBBLE_POLICY, stream)
        if st == _engine.E_UNSUPPORTED:
            return None
        _engine.check(st, f"fpq_{entry}_quantize_mx_packed")
        qa = QuantizedActivations(rows, cols, nvfp4)
        qa.mx_packed = (pc, ps)
        return qa
    if allow_packed and nvfp4 and cols % 256 == 0 and nv_packed_eligible(rows, 32, cols, fused_linear=True):
        # the row counts whose consumers run the packed NVFP4 GEMM: straight into its layout
        gs = as_f32_scalar(act_global_scale, remember)
        pc = torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes_nv(rows, cols), dtype=torch.uint8, device=dev)
        st = getattr(lib, f"fpq_{entry}_quantize_nv_packed")(*head, rows, cols, kind, h.shape[0], norm, gs.data_ptr(),
                                                             optr, pc.data_ptr(), ps.data_ptr(), ZERO_NIBBLE_POLICY,
                                                             stream)
        if st != _engine.E_UNSUPPORTED:
            _engine.check(st, f"fpq_{entry}_quantize_nv_packed")
            qa = QuantizedActivations(rows, cols, nvfp4)
            qa.nv_packed = (pc, ps)
            return qa
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // group, dtype=torch.uint8, device=dev)
    tail = (optr, codes.data_ptr(), scales.data_ptr(), rows, cols // group, ZERO_NIBBLE_POLICY, stream)
    if nvfp4:
        gs = as_f32_scalar(act_global_scale, remember)
        st = getattr(lib, f"fpq_{entry}_quantize_nv")(*head, rows, cols, kind, h.shape[0], norm, gs.data_ptr(), *tail)
    else:
        st = getattr(lib, f"fpq_{entry}_quantize_mx")(*head, rows, cols, kind, h.shape[0], norm, *tail)
    if st == _engine.E_UNSUPPORTED:
        return None
    _engine.check(st, f"fpq_{entry}_quantize")
    qa = QuantizedActivations(rows, cols, nvfp4)
    qa.row_major = (codes, scales)
    return qa


_ROWS_KERNEL_MAX_ROWS = 64   # fpq_rmsnorm_rows_max_rows()


def rmsnorm_quantize(x: torch.Tensor, weight: torch.Tensor, eps: float, hadamard_matrix: torch.Tensor,
                     act_global_scale: Optional[torch.Tensor], nvfp4: bool) -> Optional[torch.Tensor]:
    """RMSNorm of bf16 `x` over its last dimension, y = bf16(weight * bf16(x / rms)), in one pass
    that also leaves y rotated and quantized for the layers that consume it next (they find it
    through the sharing slot when called with the returned tensor).  None if this rotation has no
    fused kernel; the caller then normalises as usual."""
    if not x.is_cuda or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        return None
    x_flat = (x if x.is_contiguous() else x.contiguous()).view(-1, x.shape[-1])
    rows, cols = x_flat.shape
    if rows == 0 or weight.numel() != cols:
        return None
    dev = x.device
    with on_device(dev):
        stream = _current_stream(dev.index)
        h = as_bf16(hadamard_matrix)
        kind, norm = classify_rotation(h)
        if kind not in (_engine.ROT_HADAMARD, _engine.ROT_IDENTITY) or cols % max(h.shape[0], 32) != 0:
            return None
        lib = _engine.lib()
        y = torch.empty_like(x_flat)
        w = weight.contiguous()
        qa = None
        if (rows <= _ROWS_KERNEL_MAX_ROWS and cols % 256 == 0 and cols <= 16384
                and (nv_packed_eligible(rows, 32, cols, fused_linear=True) if nvfp4
                     else packed_linear_eligible(rows, cols, "abs_max"))):
            # a decode step's few rows: statistic, normalisation and quantization in one launch
            pc = torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=dev)
            qa = QuantizedActivations(rows, cols, nvfp4)
            if nvfp4:
                ps = torch.empty(lib.fpq_packed_scales_bytes_nv(rows, cols), dtype=torch.uint8, device=dev)
                gs = as_f32_scalar(act_global_scale)
                st = lib.fpq_rmsnorm_rows_quantize_nv_packed(x_flat.data_ptr(), cols, w.data_ptr(), rows, cols, eps,
                                                             kind, h.shape[0], norm, gs.data_ptr(), None, y.data_ptr(),
                                                             pc.data_ptr(), ps.data_ptr(), ZERO_NIBBLE_POLICY, stream)
                qa.nv_packed = (pc, ps)
            else:
                ps = torch.empty(lib.fpq_packed_scales_bytes(rows, cols), dtype=torch.uint8, device=dev)
                st = lib.fpq_rmsnorm_rows_quantize_mx_packed(x_flat.data_ptr(), cols, w.data_ptr(), rows, cols, eps,
                                                             kind, h.shape[0], norm, None, y.data_ptr(), pc.data_ptr(),
                                                             ps.data_ptr(), ZERO_NIBBLE_POLICY, stream)
                qa.mx_packed = (pc, ps)
            _engine.check(st, "fpq_rmsnorm_rows_quantize_packed")
        if qa is None:
            inv = torch.empty(rows, dtype=torch.float32, device=dev)
            _engine.check(lib.fpq_row_inv_rms(x_flat.data_ptr(), cols, rows, cols, eps, inv.data_ptr(), stream),
                          "fpq_row_inv_rms")
            qa = _fused_quantize("rmsnorm", (x_flat.data_ptr(), cols, inv.data_ptr(), w.data_ptr()), rows, cols, h, kind,
                                 norm, act_global_scale, nvfp4, y, stream, dev)
        if qa is None:
            return None
        y = y.view(x.shape)
        key = _sharing_key(x_flat.shape, h, kind, norm, act_global_scale if nvfp4 else None, stream)
        if key is not None:
            _publish(qa, y, key, h)
    return y


def silu_mul_quantize(gate: torch.Tensor, up: torch.Tensor, hadamard_matrix: torch.Tensor,
                      act_global_scale: Optional[torch.Tensor], nvfp4: bool,
                      remember: bool = True, allow_packed: bool = True) -> Optional[QuantizedActivations]:
    """Quantized bf16(silu(gate)) * up without materialising the product; gate and up are bf16 with a
    contiguous last dimension (two tensors, or two column halves of one).  None if not fusable."""
    if (not gate.is_cuda or gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16 or gate.shape != up.shape
            or gate.dim() != 2 or gate.stride(1) != 1 or up.stride(1) != 1):
        return None
    rows, cols = gate.shape
    if rows == 0:
        return None
    dev = gate.device
    with on_device(dev):
        stream = _current_stream(dev.index)
        h = as_bf16(hadamard_matrix)
        kind, norm = classify_rotation(h)
        if kind not in (_engine.ROT_HADAMARD, _engine.ROT_IDENTITY) or cols % max(h.shape[0], 32) != 0:
            return None
        ld_g = gate.stride(0) if rows > 1 else cols
        ld_u = up.stride(0) if rows > 1 else cols
        if ld_g % 8 or ld_u % 8 or ld_g < cols or ld_u < cols or gate.data_ptr() % 16 or up.data_ptr() % 16:
            return None
        return _fused_quantize("silu_mul", (gate.data_ptr(), ld_g, up.data_ptr(), ld_u), rows, cols, h, kind, norm,
                               act_global_scale, nvfp4, None, stream, dev, remember, allow_packed)
