"""`fp_quant::*` operators of the inference path, backed by libfpq_hip.so.

Same operator names, signatures, output shapes/dtypes and fake (meta) implementations as the
reference's QuTLASS wrappers (inference_lib/src/fp_quant/module/qutlass_ops.py:36-168), so that
`torch.compile(..., fullgraph=True)` keeps working across them.  Differences that stay inside
the boundary: scales are consumed row-major by the GEMMs (no per-call re-tiling), and the
rotation matrix is recognised once (Hadamard / identity / GSR) and applied as butterflies.
"""
from typing import Optional, Tuple

import ctypes
import os
import weakref

import torch

from .. import _engine
from ..utils import FPQuantDtype  # noqa: F401  (re-exported for parity with the reference module)

HAS_HIP_ENGINE = _engine.available()

# zero-nibble policy used by the operators (see include/fpq.h)
ZERO_NIBBLE_POLICY = _engine.ZERO_REFERENCE

def _version(t: torch.Tensor) -> int:
    """The tensor's in-place modification counter, the key of everything cached per tensor.  Tensors
    created under torch.inference_mode() have none: they get a constant (parameters and buffers made
    that way are not written to afterwards; activations made that way are never shared, see
    _sharing_key)."""
    try:
        return t._version
    except RuntimeError:
        return -1


def _sylvester(g: int) -> torch.Tensor:
    idx = torch.arange(g)
    anded = idx[:, None] & idx[None, :]
    pop = torch.zeros_like(anded)
    for b in range(8):
        pop += (anded >> b) & 1
    return (1 - 2 * (pop & 1)).to(torch.float32)


def classify_rotation(h: torch.Tensor) -> Tuple[int, float]:
    """(rotation kind, norm) of a [g, g] matrix.  The result is remembered on the tensor object
    itself (with its version counter), so the one device->host copy it needs happens once per
    matrix and can never be confused with another tensor that later reuses the same memory."""
    hit = getattr(h, "_fpq_rotation", None)
    if hit is not None and hit[0] == _version(h):
        return hit[1], hit[2]
    g = h.shape[0]
    if h.dim() != 2 or h.shape[1] != g:
        raise ValueError(f"rotation matrix must be square, got {tuple(h.shape)}")
    hf = h.detach().to(device="cpu", dtype=torch.float32)
    kind, norm = _engine.ROT_GENERAL, 0.0
    if torch.equal(hf, torch.eye(g)):
        kind, norm = _engine.ROT_IDENTITY, 1.0
    elif g in (16, 32, 64, 128) and float(hf[0, 0]) != 0.0:
        n = float(hf[0, 0])
        signed = _sylvester(g) * n
        if torch.equal(hf, signed):
            kind, norm = _engine.ROT_HADAMARD, n
        else:
            changes = torch.diff(signed, dim=0).ne(0).sum(dim=0)
            if torch.equal(hf, signed[:, torch.argsort(changes)]):
                kind, norm = _engine.ROT_GSR, n
    try:
        h._fpq_rotation = (_version(h), kind, norm)
    except AttributeError:  # objects that refuse attributes: classify again next time
        pass
    return kind, norm


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
    with torch.cuda.device(x.device):
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
        with torch.cuda.device(x.device):
            st = _engine.lib().fpq_quantize_mx_quest(
                x.data_ptr(), rows, cols, kind, g, norm, h.data_ptr(), codes.data_ptr(), scales.data_ptr(),
                prow, pcol, mask.data_ptr() if mask is not None else None, ZERO_NIBBLE_POLICY, _stream(x))
        _engine.check(st, "fused_quantize_mx_op")
        return codes, scales.view(torch.float8_e8m0fnu), mask
    with torch.cuda.device(x.device):
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
    with torch.cuda.device(x.device):
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
    with torch.cuda.device(x.device):
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
NV_PACKED_MIN_M = 65       # NVFP4 fused linear: from here on (and while the 128x128 tiles apply) packed;
#                            below, the split-K weight-streaming kernel on row-major operands is faster
PACKED_LINEAR_MIN_M = 25   # fused linear: activations are quantized straight into the packed layout
#                            (below, the weight-streaming split-K kernel on row-major operands is faster)


def packed_weights_enabled() -> bool:
    return os.environ.get("FPQ_PACKED_WEIGHTS", "1") != "0"


def pack_mxf4(codes: torch.Tensor, scales: torch.Tensor, rows: int, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-major codes [rows, k/2] and E8M0 scales [>=rows, >=k/32] -> the packed layout of
    fpq_gemm_mxf4_packed (rows padded to a multiple of 32)."""
    lib = _engine.lib()
    pc = torch.empty(lib.fpq_packed_codes_bytes(rows, k), dtype=torch.uint8, device=codes.device)
    ps = torch.empty(lib.fpq_packed_scales_bytes(rows, k), dtype=torch.uint8, device=codes.device)
    st = lib.fpq_pack_mxf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k,
                           pc.data_ptr(), ps.data_ptr(), _stream(codes))
    _engine.check(st, "fpq_pack_mxf4")
    return pc, ps


def pack_nvf4(codes: torch.Tensor, scales: torch.Tensor, rows: int, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-major codes [rows, k/2] and E4M3 scales [>=rows, >=k/16] -> the packed layout of
    fpq_gemm_nvf4_packed."""
    lib = _engine.lib()
    pc = torch.empty(lib.fpq_packed_codes_bytes(rows, k), dtype=torch.uint8, device=codes.device)
    ps = torch.empty(lib.fpq_packed_scales_bytes_nv(rows, k), dtype=torch.uint8, device=codes.device)
    st = lib.fpq_pack_nvf4(codes.data_ptr(), scales.data_ptr(), scales.shape[1], rows, k,
                           pc.data_ptr(), ps.data_ptr(), _stream(codes))
    _engine.check(st, "fpq_pack_nvf4")
    return pc, ps


def nv_packed_eligible(m: int, n: int, k: int) -> bool:
    """NVFP4: the packed kernel wins where its 128x128 tiles apply (mid-sized M); large M runs at
    the same speed on row-major operands, tiny M is faster on the direct kernel."""
    return (NV_PACKED_MIN_M <= m and k % 256 == 0 and packed_weights_enabled()
            and ((m + 255) // 256) * ((n + 255) // 256) < 100)


def packed_weight(wq: torch.Tensor, ws: torch.Tensor, nvfp4: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Packed copy of a weight, cached on the code tensor until either tensor is written to."""
    key = (wq.data_ptr(), _version(wq), ws.data_ptr(), _version(ws), tuple(wq.shape), nvfp4)
    hit = getattr(wq, "_fpq_packed", None)
    if hit is not None and hit[0] == key:
        return hit[1], hit[2]
    pc, ps = (pack_nvf4 if nvfp4 else pack_mxf4)(wq, ws, wq.shape[0], wq.shape[1] * 2)
    try:
        wq._fpq_packed = (key, pc, ps)
    except (AttributeError, RuntimeError):
        pass
    return pc, ps



def _gemm(entry: str, x, w, xs, ws, alpha, bias: Optional[torch.Tensor], group: int) -> torch.Tensor:
    _require_cuda(x, w, xs, ws, alpha)
    if x.dtype != torch.uint8 or w.dtype != torch.uint8:
        raise ValueError("packed operands must be uint8")
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise ValueError("alpha must be a one-element float32 tensor")
    xq = x.contiguous().view(-1, x.shape[-1])
    wq = w.contiguous()
    m, kb = xq.shape
    n = wq.shape[0]
    k = kb * 2
    if wq.shape[1] != kb:
        raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
    xs_b = xs.contiguous().view(torch.uint8)
    ws_b = ws.contiguous().view(torch.uint8)
    xs_b = xs_b.view(-1, xs_b.shape[-1])
    ws_b = ws_b.view(-1, ws_b.shape[-1])
    if xs_b.shape[0] < m or ws_b.shape[0] < n or xs_b.shape[1] < k // group or ws_b.shape[1] < k // group:
        raise ValueError("scale tensors are smaller than the operands they describe")
    y = torch.empty(*x.shape[:-1], n, dtype=torch.bfloat16, device=x.device)
    b_ptr = None
    if bias is not None:
        if bias.dtype != torch.bfloat16 or bias.numel() != n:
            raise ValueError("bias must be a bfloat16 vector of length N")
        bias = bias.contiguous()
        b_ptr = bias.data_ptr()
    a = alpha.contiguous()
    if entry == "fpq_gemm_mxf4" and m >= PACKED_MIN_M and k % 256 == 0 and packed_weights_enabled():
        with torch.cuda.device(x.device):
            wp, wsp = packed_weight(wq, ws_b)
            xp, xsp = pack_mxf4(xq, xs_b, m, k)
            st = _engine.lib().fpq_gemm_mxf4_packed(
                xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(), b_ptr,
                y.data_ptr(), m, n, k, _stream(x))
        _engine.check(st, "fpq_gemm_mxf4_packed")
        return y
    if entry == "fpq_gemm_nvf4" and nv_packed_eligible(m, n, k):
        with torch.cuda.device(x.device):
            wp, wsp = packed_weight(wq, ws_b, True)
            xp, xsp = pack_nvf4(xq, xs_b, m, k)
            st = _engine.lib().fpq_gemm_nvf4_packed(
                xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(), a.data_ptr(), b_ptr,
                y.data_ptr(), m, n, k, _stream(x))
        _engine.check(st, "fpq_gemm_nvf4_packed")
        return y
    with torch.cuda.device(x.device):
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
    return x.new_empty(*x.shape[:-1], w.shape[0], dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_ada_mxf4_bf16_tn_op", mutates_args=())
def matmul_ada_mxf4_bf16_tn_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor
) -> torch.Tensor:
    # The reference's small-M entry takes un-tiled scales; here every entry does, and the
    # library picks the small-M kernel by shape.
    return _gemm("fpq_gemm_mxf4", x, w, xs, ws, alpha, None, 32)


@matmul_ada_mxf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty(*x.shape[:-1], w.shape[0], dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_nvf4_bf16_tn_op", mutates_args=())
def matmul_nvf4_bf16_tn_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor
) -> torch.Tensor:
    return _gemm("fpq_gemm_nvf4", x, w, xs, ws, alpha, None, 16)


@matmul_nvf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty(*x.shape[:-1], w.shape[0], dtype=torch.bfloat16)


### Fused epilogue variants (bias added inside the GEMM; not part of the reference op set)


@torch.library.custom_op("fp_quant::matmul_mxf4_bf16_tn_bias_op", mutates_args=())
def matmul_mxf4_bf16_tn_bias_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
    bias: torch.Tensor,
) -> torch.Tensor:
    return _gemm("fpq_gemm_mxf4", x, w, xs, ws, alpha, bias, 32)


@matmul_mxf4_bf16_tn_bias_op.register_fake
def _(x, w, xs, ws, alpha, bias):
    return x.new_empty(*x.shape[:-1], w.shape[0], dtype=torch.bfloat16)


@torch.library.custom_op("fp_quant::matmul_nvf4_bf16_tn_bias_op", mutates_args=())
def matmul_nvf4_bf16_tn_bias_op(
    x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
    bias: torch.Tensor,
) -> torch.Tensor:
    return _gemm("fpq_gemm_nvf4", x, w, xs, ws, alpha, bias, 16)


@matmul_nvf4_bf16_tn_bias_op.register_fake
def _(x, w, xs, ws, alpha, bias):
    return x.new_empty(*x.shape[:-1], w.shape[0], dtype=torch.bfloat16)


### Whole linear, eager fast path


def cached_on(t: torch.Tensor, slot: str, key, make):
    """`make()` remembered on tensor `t` under attribute `slot` while `key` stays the same."""
    hit = getattr(t, slot, None)
    if hit is not None and hit[0] == key:
        return hit[1]
    val = make()
    try:
        setattr(t, slot, (key, val))
    except (AttributeError, RuntimeError):
        pass
    return val


def linear_alpha(weight_global_scale: torch.Tensor, act_global_scale: torch.Tensor) -> torch.Tensor:
    """fp32 one-element `1 / (wgs * ags)` evaluated in the buffers' dtype as the reference does
    (linear_fns.py:505; bf16 buffers round 1/9 to 0.111328125), cached until a buffer changes."""
    key = (_version(weight_global_scale), _version(act_global_scale), act_global_scale.data_ptr(),
           weight_global_scale.data_ptr())
    return cached_on(weight_global_scale, "_fpq_alpha", key,
                     lambda: (1.0 / (weight_global_scale * act_global_scale)).float().reshape(1).contiguous())


def as_f32_scalar(t: torch.Tensor) -> torch.Tensor:
    if t.dtype == torch.float32 and t.is_contiguous():
        return t
    return cached_on(t, "_fpq_f32", (_version(t), t.data_ptr()), lambda: t.detach().float().contiguous())


# Several layers that consume one tensor (q/k/v projections, gate/up projections) would rotate and
# quantize it once each.  The quantized activations of the latest call are kept per device and reused
# while the next call passes the very same tensor object, unmodified (its version counter), with an
# equal rotation and global scale, on the same stream and in the same graph capture (or both outside
# any: work recorded during a capture has not run when the capture ends).  The source is held weakly,
# so a freed tensor whose address is reused can never match.  Producers fused with the quantizer
# (rmsnorm_quantize, silu_mul_quantize) leave their result in the same slot for the layers that
# follow.  FPQ_SHARE_ACT_QUANT=0 turns the sharing off.
SHARE_ACT_QUANT = os.environ.get("FPQ_SHARE_ACT_QUANT", "1") != "0"


class QuantizedActivations:
    """Rotated and quantized activations of one [m, k] tensor, in whichever operand layouts have
    been asked for so far (row-major codes/scales, packed MXFP4, packed NVFP4)."""
    __slots__ = ("m", "k", "nvfp4", "packed_gemm", "ref", "version", "key", "keep", "mx_packed", "row_major",
                 "nv_packed")

    def __init__(self, m: int, k: int, nvfp4: bool, packed_gemm: bool):
        self.m, self.k, self.nvfp4 = m, k, nvfp4
        self.packed_gemm = packed_gemm   # MXFP4: the GEMM runs on packed operands (decided once per call)
        self.ref = self.key = self.keep = None
        self.version = 0
        self.mx_packed = self.row_major = self.nv_packed = None

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


def _sharing_key(x_shape, h, kind: int, norm: float, act_global_scale, stream: int, want_packed: bool):
    """What two calls must agree on, besides the source tensor, to share quantized activations, or
    None when nothing may be shared.  Layers own separate but equal rotation and global-scale
    buffers, so those are compared by value: (kind, norm, size) of a recognised rotation, the host
    copy of the scale (read once per buffer); an unrecognised rotation matrix only matches itself."""
    if not SHARE_ACT_QUANT or torch.is_inference_mode_enabled():
        return None   # in inference mode in-place writes to the source could not be noticed
    capture_id = ctypes.c_ulonglong()   # per call: host threads may run layers concurrently
    _engine.check(_engine.lib().fpq_stream_capture_id(stream, ctypes.byref(capture_id)), "fpq_stream_capture_id")
    rot = (kind, norm, h.shape[0]) if kind != _engine.ROT_GENERAL else (kind, id(h), _version(h))
    gs = None
    if act_global_scale is not None:
        gs = cached_on(act_global_scale, "_fpq_host", (_version(act_global_scale), act_global_scale.data_ptr()),
                       lambda: float(act_global_scale))
    # the operand layout the GEMM will ask for is part of the key: the packed form can be made from the
    # row-major one but not the other way round
    return (rot, gs, stream, capture_id.value, tuple(x_shape), want_packed)


def _publish(qa: QuantizedActivations, src: torch.Tensor, key, keep) -> None:
    qa.ref, qa.version, qa.key, qa.keep = weakref.ref(src), _version(src), key, keep
    _shared_activations[src.device.index] = qa


def _lookup(src: torch.Tensor, key) -> Optional[QuantizedActivations]:
    qa = _shared_activations.get(src.device.index)
    if qa is not None and qa.ref() is src and qa.version == _version(src) and qa.key == key:
        return qa
    return None


def quantize_activations(x_flat: torch.Tensor, h: torch.Tensor, kind: int, norm: float,
                         act_global_scale: Optional[torch.Tensor], nvfp4: bool, stream: int,
                         want_packed: bool) -> QuantizedActivations:
    """Rotate and quantize bf16 [m, k]: MXFP4 straight into the packed layout when the packed GEMM will
    run, row-major otherwise (NVFP4 always; its packed form is made on demand)."""
    lib = _engine.lib()
    m, k = x_flat.shape
    dev = x_flat.device
    g = h.shape[0]
    qa = QuantizedActivations(m, k, nvfp4, want_packed)
    if want_packed:
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
    group = 16 if nvfp4 else 32
    codes = torch.empty(m, k // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(m, k // group, dtype=torch.uint8, device=dev)
    if nvfp4:
        gs = as_f32_scalar(act_global_scale)
        st = lib.fpq_quantize_nv(x_flat.data_ptr(), m, k, kind, g, norm, h.data_ptr(), gs.data_ptr(),
                                 codes.data_ptr(), scales.data_ptr(), m, k // group, ZERO_NIBBLE_POLICY, stream)
        _engine.check(st, "fpq_quantize_nv")
    else:
        st = lib.fpq_quantize_mx(x_flat.data_ptr(), m, k, kind, g, norm, h.data_ptr(), codes.data_ptr(),
                                 scales.data_ptr(), m, k // group, ZERO_NIBBLE_POLICY, stream)
        _engine.check(st, "fpq_quantize_mx")
    qa.row_major = (codes, scales)
    return qa


def linear_on(qa: QuantizedActivations, wq: torch.Tensor, ws: torch.Tensor, alpha: torch.Tensor,
              bias: Optional[torch.Tensor], stream: int) -> torch.Tensor:
    """bf16 [m, n] = alpha * dq(activations) @ dq(w).T (+ bias) on quantized activations, with the
    kernel and operand layout the shape calls for."""
    lib = _engine.lib()
    m, k = qa.m, qa.k
    n = wq.shape[0]
    if wq.shape[1] * 2 != k:
        raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
    y = torch.empty(m, n, dtype=torch.bfloat16, device=wq.device)
    b_ptr = bias.data_ptr() if bias is not None else None
    if qa.nvfp4:
        if nv_packed_eligible(m, n, k):
            xp, xsp = qa.packed()
            wp, wsp = packed_weight(wq, ws, True)
            st = lib.fpq_gemm_nvf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                          alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
            _engine.check(st, "fpq_gemm_nvf4_packed")
            return y
        codes, scales = qa.row_major
        st = lib.fpq_gemm_nvf4(codes.data_ptr(), scales.data_ptr(), scales.shape[-1], wq.data_ptr(), ws.data_ptr(),
                               ws.shape[-1], alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
        _engine.check(st, "fpq_gemm_nvf4")
        return y
    if qa.packed_gemm:
        pc, ps = qa.packed()
        wp, wsp = packed_weight(wq, ws)
        st = lib.fpq_gemm_mxf4_packed(pc.data_ptr(), ps.data_ptr(), wp.data_ptr(), wsp.data_ptr(), alpha.data_ptr(),
                                      b_ptr, y.data_ptr(), m, n, k, stream)
        _engine.check(st, "fpq_gemm_mxf4_packed")
        return y
    codes, scales = qa.row_major
    st = lib.fpq_gemm_mxf4(codes.data_ptr(), scales.data_ptr(), scales.shape[-1], wq.data_ptr(), ws.data_ptr(),
                           ws.shape[-1], alpha.data_ptr(), b_ptr, y.data_ptr(), m, n, k, stream)
    _engine.check(st, "fpq_gemm_mxf4")
    return y


def linear_w4a4(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, wq: torch.Tensor, ws: torch.Tensor,
                alpha: torch.Tensor, act_global_scale: torch.Tensor, bias: Optional[torch.Tensor],
                nvfp4: bool, shared_source: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Activation rotate+quantize and W4A4 GEMM of one linear with as little host work as possible:
    the eager (non-traced) body of FPQuantLinear.forward.  Same kernels and results as the
    fused_quantize_* and matmul_* operators; `x_flat` bf16 [M, K] contiguous on the GPU, `alpha`
    fp32 [1], `bias` bf16 [N] or None.  `shared_source` is the tensor object `x_flat` was derived
    from: consecutive calls with the same, unmodified object reuse its quantized form."""
    if not x_flat.is_cuda:
        raise ValueError("fp_quant HIP operators need tensors on a GPU; there is no CPU path")
    dev = x_flat.device
    if torch.cuda.current_device() != dev.index:
        with torch.cuda.device(dev):
            return linear_w4a4(x_flat, hadamard_matrix, wq, ws, alpha, act_global_scale, bias, nvfp4, shared_source)
    stream = _current_stream(dev.index)
    h = as_bf16(hadamard_matrix)
    kind, norm = classify_rotation(h)
    want_packed = not nvfp4 and packed_linear_eligible(x_flat.shape[0], x_flat.shape[1], "abs_max")
    qa = key = None
    if shared_source is not None:
        key = _sharing_key(x_flat.shape, h, kind, norm, act_global_scale if nvfp4 else None, stream, want_packed)
        if key is not None:
            qa = _lookup(shared_source, key)
    if qa is None:
        qa = quantize_activations(x_flat, h, kind, norm, act_global_scale, nvfp4, stream, want_packed)
        if key is not None:
            _publish(qa, shared_source, key, h)
    return linear_on(qa, wq, ws, alpha, bias, stream)


### Quantizers fused with the producer of their input


def _fused_quantize(entry: str, head: tuple, rows: int, cols: int, h: torch.Tensor, kind: int, norm: float,
                    act_global_scale: Optional[torch.Tensor], nvfp4: bool, out: Optional[torch.Tensor],
                    stream: int, dev) -> Optional[QuantizedActivations]:
    """Common tail of the fused producers: allocate row-major codes/scales and call
    fpq_<entry>_quantize_{mx,nv}; None if the library has no fused kernel for this rotation."""
    lib = _engine.lib()
    group = 16 if nvfp4 else 32
    optr = out.data_ptr() if out is not None else None
    want_packed = not nvfp4 and packed_linear_eligible(rows, cols, "abs_max")
    if want_packed:
        # straight into the operand layout of the packed GEMM (streaming kernel)
        pc = torch.empty(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device=dev)
        ps = torch.empty(lib.fpq_packed_scales_bytes(rows, cols), dtype=torch.uint8, device=dev)
        st = getattr(lib, f"fpq_{entry}_quantize_mx_packed")(*head, rows, cols, kind, h.shape[0], norm, optr,
                                                             pc.data_ptr(), ps.data_ptr(), ZERO_NIBBLE_POLICY, stream)
        if st == _engine.E_UNSUPPORTED:
            return None
        _engine.check(st, f"fpq_{entry}_quantize_mx_packed")
        qa = QuantizedActivations(rows, cols, nvfp4, True)
        qa.mx_packed = (pc, ps)
        return qa
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    scales = torch.empty(rows, cols // group, dtype=torch.uint8, device=dev)
    tail = (optr, codes.data_ptr(), scales.data_ptr(), rows, cols // group, ZERO_NIBBLE_POLICY, stream)
    if nvfp4:
        gs = as_f32_scalar(act_global_scale)
        st = getattr(lib, f"fpq_{entry}_quantize_nv")(*head, rows, cols, kind, h.shape[0], norm, gs.data_ptr(), *tail)
    else:
        st = getattr(lib, f"fpq_{entry}_quantize_mx")(*head, rows, cols, kind, h.shape[0], norm, *tail)
    if st == _engine.E_UNSUPPORTED:
        return None
    _engine.check(st, f"fpq_{entry}_quantize")
    qa = QuantizedActivations(rows, cols, nvfp4, False)
    qa.row_major = (codes, scales)
    return qa


def rmsnorm_quantize(x: torch.Tensor, weight: torch.Tensor, eps: float, hadamard_matrix: torch.Tensor,
                     act_global_scale: Optional[torch.Tensor], nvfp4: bool) -> Optional[torch.Tensor]:
    """RMSNorm of bf16 `x` over its last dimension, y = bf16(weight * bf16(x / rms)), in one pass
    that also leaves y rotated and quantized for the layers that consume it next (they find it
    through the sharing slot when called with the returned tensor).  None if this rotation has no
    fused kernel; the caller then normalises as usual."""
    if not x.is_cuda or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        return None
    x_flat = x.contiguous().view(-1, x.shape[-1])
    rows, cols = x_flat.shape
    if rows == 0 or weight.numel() != cols:
        return None
    dev = x.device
    with torch.cuda.device(dev):
        stream = _current_stream(dev.index)
        h = as_bf16(hadamard_matrix)
        kind, norm = classify_rotation(h)
        if kind not in (_engine.ROT_HADAMARD, _engine.ROT_IDENTITY) or cols % max(h.shape[0], 32) != 0:
            return None
        lib = _engine.lib()
        inv = torch.empty(rows, dtype=torch.float32, device=dev)
        _engine.check(lib.fpq_row_inv_rms(x_flat.data_ptr(), cols, rows, cols, eps, inv.data_ptr(), stream),
                      "fpq_row_inv_rms")
        y = torch.empty_like(x_flat)
        w = weight.contiguous()
        qa = _fused_quantize("rmsnorm", (x_flat.data_ptr(), cols, inv.data_ptr(), w.data_ptr()), rows, cols, h, kind,
                             norm, act_global_scale, nvfp4, y, stream, dev)
        if qa is None:
            return None
        y = y.view(x.shape)
        key = _sharing_key(x_flat.shape, h, kind, norm, act_global_scale if nvfp4 else None, stream, qa.packed_gemm)
        if key is not None:
            _publish(qa, y, key, h)
    return y


def silu_mul_quantize(gate: torch.Tensor, up: torch.Tensor, hadamard_matrix: torch.Tensor,
                      act_global_scale: Optional[torch.Tensor], nvfp4: bool) -> Optional[QuantizedActivations]:
    """Quantized bf16(silu(gate)) * up without materialising the product; gate and up are bf16 with a
    contiguous last dimension (two tensors, or two column halves of one).  None if not fusable."""
    if (not gate.is_cuda or gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16 or gate.shape != up.shape
            or gate.dim() != 2 or gate.stride(1) != 1 or up.stride(1) != 1):
        return None
    rows, cols = gate.shape
    if rows == 0:
        return None
    dev = gate.device
    with torch.cuda.device(dev):
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
                               act_global_scale, nvfp4, None, stream, dev)
