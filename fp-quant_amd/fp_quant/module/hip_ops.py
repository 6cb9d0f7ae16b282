"""`fp_quant::*` operators of the inference path, backed by libfpq_hip.so.

Same operator names, signatures, output shapes/dtypes and fake (meta) implementations as the
reference's QuTLASS wrappers (inference_lib/src/fp_quant/module/qutlass_ops.py:36-168), so that
`torch.compile(..., fullgraph=True)` keeps working across them.  Differences that stay inside
the boundary: scales are consumed row-major by the GEMMs (no per-call re-tiling), and the
rotation matrix is recognised once (Hadamard / identity / GSR) and applied as butterflies.
"""
from typing import Optional, Tuple

import os

import torch

from .. import _engine
from ..utils import FPQuantDtype  # noqa: F401  (re-exported for parity with the reference module)

HAS_HIP_ENGINE = _engine.available()

# zero-nibble policy used by the operators (see include/fpq.h)
ZERO_NIBBLE_POLICY = _engine.ZERO_REFERENCE

on_device = _engine.on_device


def _version(t: torch.Tensor):
    """Cache key part for everything remembered per tensor: the in-place modification counter, or for
    tensors created under torch.inference_mode() (which have none) a marker -- what is remembered for
    those is only dropped by drop_tensor_caches, which FPQuantLinear runs after load_state_dict."""
    try:
        return t._version
    except RuntimeError:
        return "no-counter"


_TENSOR_CACHES = ("_fpq_rotation", "_fpq_bf16", "_fpq_packed", "_fpq_group", "_fpq_alpha", "_fpq_f32", "_fpq_host",
                  "_fpq_splitk")


def drop_tensor_caches(*tensors, keep=()) -> None:
    """Forget everything remembered on these tensors (packed weights, alpha, converted copies) but the
    attributes named in `keep`: for callers that rewrote their storage in a way the modification counter does
    not see."""
    for t in tensors:
        if isinstance(t, torch.Tensor):
            for name in _TENSOR_CACHES:
                if name not in keep and hasattr(t, name):
                    try:
                        delattr(t, name)
                    except AttributeError:
                        pass


classify_rotation = _engine.classify_rotation


def as_bf16(h: torch.Tensor) -> torch.Tensor:
    """`h` in bfloat16, contiguous; the converted copy is kept on the source tensor so that a
    non-bf16 rotation buffer is converted (and later classified) once, not on every call."""
    if h.dtype == torch.bfloat16 and h.is_contiguous():
        return h
    hit = getattr(h, "_fpq_bf16", None)
    if hit is not None and hit[0] == _version(h):
        return hit[1]
    conv = h.detach().to(torch.bfloat16).contiguous()
    try:
        h._fpq_bf16 = (_version(h), conv)
    except AttributeError:
        pass
    return conv


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


# the current stream's handle without building a torch.cuda.Stream object (several microseconds per call)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device_index: int) -> int:
    if _raw_stream is not None:
        return _raw_stream(device_index)
    return torch.cuda.current_stream().cuda_stream


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("fp_quant HIP operators need tensors on a GPU; there is no CPU path")


def _padded(rows: int, groups: int) -> Tuple[int, int]:
    return (rows + 127) // 128 * 128, (groups + 3) // 4 * 4


### Forward quantization


def quantize_mx_packed(x: torch.Tensor, hadamard_matrix: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """abs_max MXFP4 quantization of bf16 [rows, cols] straight into the packed GEMM layout
    (cols % 256 == 0).  Rotations the packed quantizer has no kernel for go through the row-major
    quantizer and the re-tiling kernel."""
    lib = _engine.lib()
    rows, cols = x.shape
    kind, norm = classify_rotation(hadamard_matrix)
    g = hadamard_matrix.shape[0]
    pc = torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=x.device)
    ps = torch.empty(lib.fpq_packed_scales_bytes(rows, cols), dtype=torch.uint8, device=x.device)
    st = lib.fpq_quantize_mx_packed(x.data_ptr(), rows, cols, kind, g, norm, pc.data_ptr(), ps.data_ptr(),
                                    ZERO_NIBBLE_POLICY, _stream(x))
    if st == _engine.E_UNSUPPORTED:
        codes, scales, _ = fused_quantize_mx_op(x, hadamard_matrix, "abs_max", False)
        return pack_mxf4(codes, scales.view(torch.uint8), rows, cols)
    _engine.check(st, "fpq_quantize_mx_packed")
    return pc, ps


def packed_linear_eligible(rows: int, k: int, forward_method: str) -> bool:
    return forward_method == "abs_max" and rows >= PACKED_LINEAR_MIN_M and k % 256 == 0 and packed_weights_enabled()


@torch.library.custom_op("fp_quant::linear_alpha_op", mutates_args=())
def linear_alpha_op(weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor) -> torch.Tensor:
    """fp32 [1]: `1 / (weight_global_scale * act_global_scale)` with the product and the reciprocal
    each rounded to the buffers' dtype, as eager PyTorch evaluates the reference's expression
    (linear_fns.py:505).  An operator so that a compiler cannot fuse the chain and drop the
    intermediate roundings (bf16 buffers: 1/9 becomes 0.111328125, fused in fp32 it would not)."""
    return (1.0 / (weight_global_scale * act_global_scale)).float().reshape(1)


@linear_alpha_op.register_fake
def _(weight_global_scale, act_global_scale):
    return weight_global_scale.new_empty((1,), dtype=torch.float32)


@torch.library.custom_op("fp_quant::linear_mxf4_packed_op", mutates_args=())
def linear_mxf4_packed_op(
    x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, w: torch.Tensor, ws: torch.Tensor,
    alpha: torch.Tensor, bias: Optional[torch.Tensor],
) -> torch.Tensor:
    """Activation rotate+quantize and W4A4 GEMM of one MXFP4 linear on packed operands: the same
    codes, scales and output bits as fused_quantize_mx_op followed by matmul_mxf4_bf16_tn_op."""
    _require_cuda(x_flat, hadamard_matrix, w, ws, alpha)
    if x_flat.dtype != torch.bfloat16 or x_flat.dim() != 2:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor")
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise ValueError("alpha must be a one-element float32 tensor")
    x = x_flat.contiguous()
    m, k = x.shape
    wq = w.contiguous()
    n = wq.shape[0]
    if wq.dtype != torch.uint8 or wq.shape[1] * 2 != k:
        raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
    ws_b = ws.contiguous().view(torch.uint8)
    b_ptr = None
    if bias is not None:
        if bias.dtype != torch.bfloat16 or bias.numel() != n:
            raise ValueError("bias must be a bfloat16 vector of length N")
        bias = bias.contiguous()
        b_ptr = bias.data_ptr()
    y = torch.empty(m, n, dtype=torch.bfloat16, device=x.device)
    a = alpha.contiguous()
    with on_device(x.device):
        xp, xsp = quantize_mx_packed(x, hadamard_matrix)
        wp, wsp = packed_weight(wq, ws_b)
        st = _engine.lib().fpq_gemm_mxf4_packed(
            xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(), b_ptr,
            y.data_ptr(), m, n, k, _stream(x))
    _engine.check(st, "fpq_gemm_mxf4_packed")
    return y


@linear_mxf4_packed_op.register_fake
def _(x_flat, hadamard_matrix, w, ws, alpha, bias):
    return torch.empty(x_flat.size(0), w.size(0), dtype=torch.bfloat16, device=x_flat.device)



@torch.library.custom_op("fp_quant::fused_quantize_mx_op", mutates_args=())
def fused_quantize_mx_op(
    x_flat: torch.Tensor,
    hadamard_matrix: torch.Tensor,
    forward_method: str,
    return_mask: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    if forward_method not in ("abs_max", "quest"):
        raise ValueError(f"Unsupported forward method: {forward_method}")
    if return_mask and forward_method != "quest":
        raise NotImplementedError("clip masks are only produced by the quest method")
    _require_cuda(x_flat, hadamard_matrix)
    if x_flat.dtype != torch.bfloat16 or x_flat.dim() != 2:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor")
    x = x_flat.contiguous()
    rows, cols = x.shape
    kind, norm = classify_rotation(hadamard_matrix)
    g = hadamard_matrix.shape[0]
    prow, pcol = _padded(rows, cols // 32)
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(prow, pcol, dtype=torch.uint8, device=x.device)
    h = hadamard_matrix.contiguous()
    if forward_method == "quest":
        mask = torch.empty(rows, cols // 8, dtype=torch.uint8, device=x.device) if return_mask else None
        with on_device(x.device):
            st = _engine.lib().fpq_quantize_mx_quest(
                x.data_ptr(), rows, cols, kind, g, norm, h.data_ptr(), codes.data_ptr(), scales.data_ptr(),
                prow, pcol, mask.data_ptr() if mask is not None else None, ZERO_NIBBLE_POLICY, _stream(x))
        _engine.check(st, "fused_quantize_mx_op")
        return codes, scales.view(torch.float8_e8m0fnu), mask
    with on_device(x.device):
        st = _engine.lib().fpq_quantize_mx(
            x.data_ptr(), rows, cols, kind, g, norm, h.data_ptr(), codes.data_ptr(),
            scales.data_ptr(), prow, pcol, ZERO_NIBBLE_POLICY, _stream(x))
    _engine.check(st, "fused_quantize_mx_op")
    return codes, scales.view(torch.float8_e8m0fnu), None


@fused_quantize_mx_op.register_fake
def _(x_flat, hadamard_matrix, forward_method, return_mask):
    rows, cols = x_flat.size(0), x_flat.size(1)
    prow, pcol = _padded(rows, cols // 32)
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=x_flat.device)
    scales = torch.empty(prow, pcol, dtype=torch.float8_e8m0fnu, device=x_flat.device)
    mask = torch.empty(rows, cols // 8, dtype=torch.uint8, device=x_flat.device) if return_mask else None
    return codes, scales, mask


@torch.library.custom_op("fp_quant::fused_quantize_nv_op", mutates_args=())
def fused_quantize_nv_op(
    x_flat: torch.Tensor,
    hadamard_matrix: torch.Tensor,
    global_scale: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    _require_cuda(x_flat, hadamard_matrix, global_scale)
    if x_flat.dtype != torch.bfloat16:
        raise ValueError("x_flat must be a bfloat16 tensor")
    if global_scale.dtype != torch.float32 or global_scale.numel() != 1:
        raise ValueError("global_scale must be a one-element float32 tensor")
    x = x_flat.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    kind, norm = classify_rotation(hadamard_matrix)
    g = hadamard_matrix.shape[0]
    prow, pcol = _padded(rows, cols // 16)
    codes = torch.empty(*x.shape[:-1], cols // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(prow, pcol, dtype=torch.uint8, device=x.device)
    h = hadamard_matrix.contiguous()
    gs = global_scale.contiguous()
    with on_device(x.device):
        st = _engine.lib().fpq_quantize_nv(
            x.data_ptr(), rows, cols, kind, g, norm, h.data_ptr(), gs.data_ptr(), codes.data_ptr(),
            scales.data_ptr(), prow, pcol, ZERO_NIBBLE_POLICY, _stream(x))
    _engine.check(st, "fused_quantize_nv_op")
    return codes, scales.view(torch.float8_e4m3fn)


@fused_quantize_nv_op.register_fake
def _(x_flat, hadamard_matrix, global_scale):
    cols = x_flat.size(-1)
    rows = x_flat.numel() // cols
    prow, pcol = _padded(rows, cols // 16)
    codes = torch.empty(*x_flat.shape[:-1], cols // 2, dtype=torch.uint8, device=x_flat.device)
    scales = torch.empty(prow, pcol, dtype=torch.float8_e4m3fn, device=x_flat.device)
    return codes, scales


def rotated_absmax(x: torch.Tensor, hadamard_matrix: torch.Tensor, amax: Optional[torch.Tensor] = None) -> torch.Tensor:
    """max |x @ blockdiag(H)| as a one-element fp32 tensor, folded into `amax` when one is given
    (running maximum over calls).  Same rotation arithmetic as the quantize operators."""
    _require_cuda(x, hadamard_matrix)
    if x.dtype != torch.bfloat16:
        raise ValueError("x must be a bfloat16 tensor")
    x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    if amax is None:
        amax = torch.zeros(1, dtype=torch.float32, device=x.device)
    elif amax.dtype != torch.float32 or amax.numel() != 1 or amax.device != x.device:
        raise ValueError("amax must be a one-element float32 tensor on the device of x")
    kind, norm = classify_rotation(hadamard_matrix)
    h = as_bf16(hadamard_matrix)
    with on_device(x.device):
        st = _engine.lib().fpq_rotated_absmax(x.data_ptr(), rows, cols, kind, hadamard_matrix.shape[0], norm,
                                              h.data_ptr(), amax.data_ptr(), _stream(x))
    _engine.check(st, "fpq_rotated_absmax")
    return amax


### GEMMs

# From these many activation rows on, the MXFP4 GEMM runs on operands re-tiled into the order the
# matrix instructions consume them (bit-identical results, contiguous operand fetch).  The
# re-tiled weights are made once per weight tensor and kept next to it, which doubles the memory
# held by 4-bit weights; FPQ_PACKED_WEIGHTS=0 keeps every call on the row-major kernels.
PACKED_MIN_M = 48          # GEMM operator on row-major operands (pays for re-tiling the activations)
NV_PACKED_MIN_M = 65       # NVFP4 GEMM operator on row-major operands: from here on (and while the 128x128
#                            tiles apply) packed; below, re-tiling the activations costs more than it saves
NV_PACKED_LINEAR_MIN_M = 1 # NVFP4 fused linear (activations quantized straight into the packed layout): the
#                            weight-streaming kernel up to 96 rows (one row is as fast on the row-major split-K
#                            kernel; it stays here so that a layer gives the same bits alone and in a group)
# fused linear: activations are quantized straight into the packed layout; the weight-streaming
# kernel on packed operands serves the few-row (decode) calls; FPQ_PACKED_MIN_ROWS raises the bar
PACKED_LINEAR_MIN_M = int(os.environ.get("FPQ_PACKED_MIN_ROWS", "1"))


def packed_weights_enabled() -> bool:
    return os.environ.get("FPQ_PACKED_WEIGHTS", "1") != "0"


def _pack_buffers(into, codes_bytes: int, scales_bytes: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """Output buffers of a pack: `into` = (codes, scales) of exactly these sizes (written in place, so that
    raw pointers to them stay valid), or new ones."""
    if into is not None:
        pc, ps = into
        if (pc.numel() == codes_bytes and ps.numel() == scales_bytes and pc.device == device and ps.device == device
                and pc.dtype == torch.uint8 and ps.dtype == torch.uint8 and pc.is_contiguous() and ps.is_contiguous()):
            return pc, ps
    return (torch.empty(codes_bytes, dtype=torch.uint8, device=device),
            torch.empty(scales_bytes, dtype=torch.uint8, device=device))


def pack_mxf4(codes: torch.Tensor, scales: torch.Tensor, rows: int, k: int, into=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-major codes [rows, k/2] and E8M0 scales [>=rows, >=k/32] -> the packed layout of
    fpq_gemm_mxf4_packed (rows padded to a multiple of 32)."""
    lib = _engine.lib()
    pc, ps = _pack_buffers(into, lib.fpq_packed_codes_bytes(rows, k), lib.fpq_packed_scales_bytes(rows, k), codes.device)
    st = lib.fpq_pack_mxf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k,
                           pc.data_ptr(), ps.data_ptr(), _stream(codes))
    _engine.check(st, "fpq_pack_mxf4")
    return pc, ps


def pack_nvf4(codes: torch.Tensor, scales: torch.Tensor, rows: int, k: int, into=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-major codes [rows, k/2] and E4M3 scales [>=rows, >=k/16] -> the packed layout of
    fpq_gemm_nvf4_packed."""
    lib = _engine.lib()
    pc, ps = _pack_buffers(into, lib.fpq_packed_codes_bytes(rows, k), lib.fpq_packed_scales_bytes_nv(rows, k),
                           codes.device)
    st = lib.fpq_pack_nvf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k,
                           pc.data_ptr(), ps.data_ptr(), _stream(codes))
    _engine.check(st, "fpq_pack_nvf4")
    return pc, ps


def nv_packed_eligible(m: int, n: int, k: int, fused_linear: bool = False) -> bool:
    """NVFP4: the packed kernels at every row count from the smallest they take (the weight-streaming kernel,
    the tile kernels, whose large tiles convert the operands of the next K step behind the matrix instructions
    of the current one and are 6-7 % faster than the row-major kernel: 4096 x 24576 x 4096 570 against 610 us)."""
    return ((NV_PACKED_LINEAR_MIN_M if fused_linear else NV_PACKED_MIN_M) <= m and k % 256 == 0
            and packed_weights_enabled())


def unpack_fp4(pc: torch.Tensor, ps: torch.Tensor, rows: int, k: int, nvfp4: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Packed operand -> row-major codes [rows, k/2] and scales [rows, k/32] (MXFP4, E8M0) or [rows, k/16]
    (NVFP4, E4M3): the inverse of pack_mxf4 / pack_nvf4."""
    lib = _engine.lib()
    group = 16 if nvfp4 else 32
    codes = torch.empty(rows, k // 2, dtype=torch.uint8, device=pc.device)
    scales = torch.empty(rows, k // group, dtype=torch.uint8, device=pc.device)
    entry = lib.fpq_unpack_nvf4 if nvfp4 else lib.fpq_unpack_mxf4
    with on_device(pc.device):
        st = entry(pc.data_ptr(), ps.data_ptr(), rows, k, codes.data_ptr(), scales.data_ptr(), k // group, _stream(pc))
    _engine.check(st, "fpq_unpack_nvf4" if nvfp4 else "fpq_unpack_mxf4")
    return codes, scales


# A layer may hold its weight in the packed layout ONLY (FPQuantLinear.release_row_major): its
# `qweight` / `scales` are then the 1-D packed buffers themselves.  The number of dimensions is the marker
# (it survives every operator boundary); the row count follows from the inner dimension of the activations.
def is_packed_only(wq: torch.Tensor) -> bool:
    return wq.dim() == 1


def weight_rows(wq: torch.Tensor, k: int) -> int:
    """Output features of a weight given as row-major codes [n, k/2] or as a 1-D packed buffer (n % 32 == 0)."""
    if wq.dim() == 2:
        return wq.shape[0]
    n = wq.numel() * 2 // max(k, 1)
    if k < 256 or k % 256 != 0 or n * k != wq.numel() * 2 or n % 32 != 0:
        raise ValueError(f"a packed weight of {wq.numel()} bytes does not match activations with K={k}")
    return n


def _packed_weight_key(wq: torch.Tensor, ws: torch.Tensor, nvfp4: bool):
    return (wq.data_ptr(), _version(wq), ws.data_ptr(), _version(ws), tuple(wq.shape), nvfp4)


def packed_weight_ready(wq: torch.Tensor, ws: torch.Tensor, nvfp4: bool = False) -> bool:
    """Whether packed_weight would find its cached copy."""
    if wq.dim() == 1:
        return True
    hit = getattr(wq, "_fpq_packed", None)
    return hit is not None and hit[0] == _packed_weight_key(wq, ws, nvfp4)


def packed_weight(wq: torch.Tensor, ws: torch.Tensor, nvfp4: bool = False, into=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Packed copy of a weight, cached on the code tensor until either tensor is written to (a weight
    held in the packed layout only is its own packed copy).  A copy that has gone stale is re-packed into the
    buffers it already has, and a new one into `into` = (codes, scales) if those have the right sizes: the
    addresses a recorded graph holds stay those of the layer's current weight."""
    if wq.dim() == 1:
        return wq, ws
    key = _packed_weight_key(wq, ws, nvfp4)
    hit = getattr(wq, "_fpq_packed", None)
    if hit is not None and hit[0] == key:
        return hit[1], hit[2]
    if hit is not None and into is None and not torch.cuda.is_current_stream_capturing():
        into = (hit[1], hit[2])
    pc, ps = (pack_nvf4 if nvfp4 else pack_mxf4)(wq, ws, wq.shape[0], wq.shape[1] * 2, into)
    try:
        wq._fpq_packed = (key, pc, ps)
    except (AttributeError, RuntimeError):
        pass
    return pc, ps



def adopt_packed_weight(wq: torch.Tensor, ws: torch.Tensor, nvfp4: bool, pc: torch.Tensor, ps: torch.Tensor) -> None:
    """Declare (pc, ps) the packed copy of the row-major weight (wq, ws), as packed_weight would have made it."""
    try:
        wq._fpq_packed = (_packed_weight_key(wq, ws, nvfp4), pc, ps)
    except (AttributeError, RuntimeError):
        pass


_splitk_need = {}   # (n, k, nvfp4) -> workspace bytes with which fpq_gemm_*_packed_splitk splits K at any row count it does
SPLIT_K_ROWS = 128  # the rows the weight-streaming GEMM takes (MXFP4 splits nowhere else)
# NVFP4: beyond them come two passes of that kernel (up to 256 rows) and the tile kernels' K split (a few
# hundred rows on few weight rows and a long K); the row counts probed for the workspace a layer may need,
# and the row count up to which a call hands its workspace to the library
_SPLIT_K_PROBE_ROWS = (32, 64, 96, 128, 192, 256, 384, 512, 768, 1024)
SPLIT_K_MAX_ROWS = 1024
# FPQ_SPLIT_K=0: no split-K workspace anywhere; every GEMM walks the whole of K in one workgroup
SPLIT_K = os.environ.get("FPQ_SPLIT_K", "1") != "0"

# Eager calls: ONE workspace per (device, stream), shared by every layer called on that stream.  Kernels on a
# stream run one after the other and each leaves the workspace zeroed, so layers may share it, while calls of
# one layer on different streams (host threads with a stream each) never meet in one.  Created, and grown, by
# the call that needs it, on the stream it is for; at most _STREAM_WORKSPACES_MAX per device (the oldest goes
# first: PyTorch's allocator hands its memory out again in the order of the stream that used it).
_stream_workspaces = {}
_STREAM_WORKSPACES_MAX = 16


def _stream_workspace(device: torch.device, stream: int, need: int) -> torch.Tensor:
    per_device = _stream_workspaces.setdefault(device.index, {})
    hit = per_device.get(stream)
    if hit is not None and hit.numel() >= need:
        return hit
    per_device.pop(stream, None)
    while len(per_device) >= _STREAM_WORKSPACES_MAX:
        per_device.pop(next(iter(per_device)))
    workspace = per_device[stream] = torch.zeros(need, dtype=torch.uint8, device=device)
    return workspace


def splitk_workspace(wq: torch.Tensor, n: int, k: int, create: bool, stream: Optional[int] = None,
                     nvfp4: bool = False) -> Optional[torch.Tensor]:
    """The workspace with which the packed GEMM of a layer [n, k] (either format) splits K across workgroups at
    up to 128 activation rows (few weight rows and a long K: a Llama down-projection), or None where it would
    not split.  Always zeroed between calls.  Which one:

    * an eager call (`create` and the current stream `stream` given, no capture running): the stream's own
      workspace (_stream_workspace), so calls on different streams share nothing;
    * a call recorded into a graph capture, or a traced call (which may not create anything): the LAYER's
      workspace, kept on its code tensor `wq`, made when the layer is primed (`create` without `stream`) and
      kept for the layer's lifetime, so that a recorded graph's pointers stay valid.  Two graphs that hold the
      same layer must not be replayed at the same time on different streams.

    Either way the layer takes the same kernel and gives the same bits."""
    if not SPLIT_K:
        return None
    need = _splitk_need.get((n, k, nvfp4))
    if need is None:
        lib = _engine.lib()
        size = lib.fpq_gemm_nvf4_packed_workspace_bytes if nvfp4 else lib.fpq_gemm_mxf4_packed_workspace_bytes
        rows = _SPLIT_K_PROBE_ROWS if nvfp4 else _SPLIT_K_PROBE_ROWS[:4]
        need = _splitk_need[(n, k, nvfp4)] = max(int(size(m, n, k)) for m in rows)
    if need == 0:
        return None
    capturing = torch.cuda.is_current_stream_capturing()
    if create and stream is not None and not capturing:
        return _stream_workspace(wq.device, stream, need)
    hit = getattr(wq, "_fpq_splitk", None)
    if hit is not None and hit.numel() >= need and hit.device == wq.device:
        return hit
    if not create or capturing:
        return None
    workspace = torch.zeros(need, dtype=torch.uint8, device=wq.device)
    try:
        wq._fpq_splitk = workspace
    except (AttributeError, RuntimeError):
        return None   # cannot be kept: a workspace per call would cost more than the split gains
    return workspace


def _gemm(entry: str, x, w, xs, ws, alpha, bias: Optional[torch.Tensor], group: int) -> torch.Tensor:
    _require_cuda(x, w, xs, ws, alpha)
    if x.dtype != torch.uint8 or w.dtype != torch.uint8:
        raise ValueError("packed operands must be uint8")
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise ValueError("alpha must be a one-element float32 tensor")
    xq = x.contiguous().view(-1, x.shape[-1])
    wq = w.contiguous()
    m, kb = xq.shape
    k = kb * 2
    xs_b = xs.contiguous().view(torch.uint8)
    xs_b = xs_b.view(-1, xs_b.shape[-1])
    ws_b = ws.contiguous().view(torch.uint8)
    packed_only = is_packed_only(wq)   # a layer that holds its weight in the packed layout only
    if packed_only:
        n = weight_rows(wq, k)
        if ws_b.numel() * (group // 2) != wq.numel():
            raise ValueError("packed scales do not match the packed codes")
    else:
        n = wq.shape[0]
        if wq.shape[1] != kb:
            raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
        ws_b = ws_b.view(-1, ws_b.shape[-1])
        if ws_b.shape[0] < n or ws_b.shape[1] < k // group:
            raise ValueError("scale tensors are smaller than the operands they describe")
    if xs_b.shape[0] < m or xs_b.shape[1] < k // group:
        raise ValueError("scale tensors are smaller than the operands they describe")
    y = torch.empty(*x.shape[:-1], n, dtype=torch.bfloat16, device=x.device)
    b_ptr = None
    if bias is not None:
        if bias.dtype != torch.bfloat16 or bias.numel() != n:
            raise ValueError("bias must be a bfloat16 vector of length N")
        bias = bias.contiguous()
        b_ptr = bias.data_ptr()
    a = alpha.contiguous()
    if entry == "fpq_gemm_mxf4" and (packed_only or (m >= PACKED_MIN_M and k % 256 == 0 and packed_weights_enabled())):
        with on_device(x.device):
            wp, wsp = packed_weight(wq, ws_b)
            xp, xsp = pack_mxf4(xq, xs_b, m, k)
            st = _engine.lib().fpq_gemm_mxf4_packed(
                xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(), b_ptr,
                y.data_ptr(), m, n, k, _stream(x))
        _engine.check(st, "fpq_gemm_mxf4_packed")
        return y
    if entry == "fpq_gemm_nvf4" and (packed_only or nv_packed_eligible(m, n, k)):
        with on_device(x.device):
            wp, wsp = packed_weight(wq, ws_b, True)
            xp, xsp = pack_nvf4(xq, xs_b, m, k)
            st = _engine.lib().fpq_gemm_nvf4_packed(
                xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(), b_ptr,
                y.data_ptr(), m, n, k, _stream(x))
        _engine.check(st, "fpq_gemm_nvf4_packed")
        return y
    with on_device(x.device):
        st = getattr(_engine.lib(), entry)(
            xq.data_ptr(), xs_b.data_ptr(), xs_b.shape[1], wq.data_ptr(), ws_b.data_ptr(),
            ws_b.shape[1], a.data_ptr(), b_ptr, y.data_ptr(), m, n, k, _stream(x))
    _engine.check(st, entry)
    return y


@torch.library.custom_op("fp_quant::matmul_mxf4_bf16_tn_op", mutates_args=())
def matmul_mxf4_bf16_tn_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor
) -> torch.Tensor:
    return _gemm("fpq_gemm_mxf4", x, w, xs, ws, alpha, None, 32)


@matmul_mxf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty(*x.shape[:-1], weight_rows(w, x.shape[-1] * 2), dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_ada_mxf4_bf16_tn_op", mutates_args=())
def matmul_ada_mxf4_bf16_tn_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor
) -> torch.Tensor:
    # The reference's small-M entry takes un-tiled scales; here every entry does, and the
    # library picks the small-M kernel by shape.
    return _gemm("fpq_gemm_mxf4", x, w, xs, ws, alpha, None, 32)


@matmul_ada_mxf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty(*x.shape[:-1], weight_rows(w, x.shape[-1] * 2), dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_nvf4_bf16_tn_op", mutates_args=())
def matmul_nvf4_bf16_tn_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor
) -> torch.Tensor:
    return _gemm("fpq_gemm_nvf4", x, w, xs, ws, alpha, None, 16)


@matmul_nvf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty(*x.shape[:-1], weight_rows(w, x.shape[-1] * 2), dtype=torch.bfloat16)


### Fused epilogue variants (bias added inside the GEMM; not part of the reference op set)


@torch.library.custom_op("fp_quant::matmul_mxf4_bf16_tn_bias_op", mutates_args=())
def matmul_mxf4_bf16_tn_bias_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
    bias: torch.Tensor,
) -> torch.Tensor:
    return _gemm("fpq_gemm_mxf4", x, w, xs, ws, alpha, bias, 32)


@matmul_mxf4_bf16_tn_bias_op.register_fake
def _(x, w, xs, ws, alpha, bias):
    return x.new_empty(*x.shape[:-1], weight_rows(w, x.shape[-1] * 2), dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_nvf4_bf16_tn_bias_op", mutates_args=())
def matmul_nvf4_bf16_tn_bias_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
    bias: torch.Tensor,
) -> torch.Tensor:
    return _gemm("fpq_gemm_nvf4", x, w, xs, ws, alpha, bias, 16)


@matmul_nvf4_bf16_tn_bias_op.register_fake
def _(x, w, xs, ws, alpha, bias):
    return x.new_empty(*x.shape[:-1], weight_rows(w, x.shape[-1] * 2), dtype=torch.bfloat16)
