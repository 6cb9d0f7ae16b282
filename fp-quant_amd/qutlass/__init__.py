"""QuTLASS's Python entry points, as FP-Quant's inference path calls them, on the MI355X engine.

FP-Quant reaches its CUDA kernels through the un-vendored package `qutlass`
(inference_lib/src/fp_quant/module/qutlass_ops.py:5-28 imports the names below; the calls are at
:43-48, :80-84, :119-125, :141 and :157-163).  This module answers to that name with the same
functions, arguments and returned tensors, implemented by libfpq_hip.so (include/fpq.h) through
ctypes, so that code written against QuTLASS -- the reference's own `fp_quant` package included --
runs on a gfx950 GPU without a change, and so that callers which only test for the package
(transformers' `is_qutlass_available()` wants version >= 0.2.0) find it.

Differences a caller can see: scales are consumed row-major, so `qutlass.utils.to_blocked` returns
its argument unchanged; the training entry points (MXFP8 GEMMs, the backward quantizers) are not
part of this engine and raise NotImplementedError.  There is no CPU path and no other backend:
without the library every call raises.

It depends on nothing but the engine's loader (fp_quant/_engine.py beside it, read by file path
under a private name, so that whichever package is installed as `fp_quant` is left alone).
"""
import importlib.util
import os
from typing import Optional, Tuple

import torch

__version__ = "0.2.0"

_HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location(
    "_fpq_engine_for_qutlass", os.path.join(_HERE, os.pardir, "fp_quant", "_engine.py"))
_engine = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_engine)

_ZERO_POLICY = _engine.ZERO_REFERENCE   # every zero packs as 0x8, as the reference's exporter packs it
_PACKED_MIN_M = 48   # from here on the MXFP4 GEMM runs on re-tiled operands (weights re-tiled once)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("these kernels need tensors on a GPU; there is no CPU path")


_rotation = _engine.classify_rotation   # (rotation kind, norm) of a [g, g] matrix, remembered per tensor


def _padded(rows: int, groups: int) -> Tuple[int, int]:
    return (rows + 127) // 128 * 128, (groups + 3) // 4 * 4


def _bf16_matrix(h: torch.Tensor) -> torch.Tensor:
    return h if (h.dtype == torch.bfloat16 and h.is_contiguous()) else h.detach().to(torch.bfloat16).contiguous()


def fusedQuantizeMx(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, method: str = "abs_max",
                    return_mask: bool = False):
    """(codes uint8 [R, C/2], scales float8_e8m0fnu [ceil128(R), ceil4(C/32)]) of bf16 `x_flat`
    rotated in blocks by `hadamard_matrix`; with `return_mask` (method "quest") also the clip mask
    uint8 [R, C/8]."""
    if method not in ("abs_max", "quest"):
        raise ValueError(f"Unsupported forward method: {method}")
    if return_mask and method != "quest":
        raise NotImplementedError("clip masks are only produced by the quest method")
    _need_gpu(x_flat, hadamard_matrix)
    if x_flat.dtype != torch.bfloat16 or x_flat.dim() != 2:
        raise ValueError("x_flat must be a 2-D bfloat16 tensor")
    x = x_flat.contiguous()
    rows, cols = x.shape
    h = _bf16_matrix(hadamard_matrix)
    kind, norm = _rotation(h)
    prow, pcol = _padded(rows, cols // 32)
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(prow, pcol, dtype=torch.uint8, device=x.device)
    lib = _engine.lib()
    with _engine.on_device(x.device):
        if method == "quest":
            mask = torch.empty(rows, cols // 8, dtype=torch.uint8, device=x.device) if return_mask else None
            st = lib.fpq_quantize_mx_quest(x.data_ptr(), rows, cols, kind, h.shape[0], norm, h.data_ptr(),
                                           codes.data_ptr(), scales.data_ptr(), prow, pcol,
                                           mask.data_ptr() if mask is not None else None, _ZERO_POLICY, _stream(x))
            _engine.check(st, "fusedQuantizeMx")
            out = (codes, scales.view(torch.float8_e8m0fnu))
            return out + (mask,) if return_mask else out
        st = lib.fpq_quantize_mx(x.data_ptr(), rows, cols, kind, h.shape[0], norm, h.data_ptr(), codes.data_ptr(),
                                 scales.data_ptr(), prow, pcol, _ZERO_POLICY, _stream(x))
    _engine.check(st, "fusedQuantizeMx")
    return codes, scales.view(torch.float8_e8m0fnu)


def fusedQuantizeNv(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor, global_scale: torch.Tensor):
    """(codes uint8 [..., C/2], scales float8_e4m3fn [ceil128(R), ceil4(C/16)]); `global_scale` is a
    one-element fp32 tensor on the GPU (a multiplier, as in the reference)."""
    _need_gpu(x_flat, hadamard_matrix, global_scale)
    if x_flat.dtype != torch.bfloat16:
        raise ValueError("x_flat must be a bfloat16 tensor")
    if global_scale.dtype != torch.float32 or global_scale.numel() != 1:
        raise ValueError("global_scale must be a one-element float32 tensor")
    x = x_flat.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols if cols else 0
    h = _bf16_matrix(hadamard_matrix)
    kind, norm = _rotation(h)
    prow, pcol = _padded(rows, cols // 16)
    codes = torch.empty(*x.shape[:-1], cols // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(prow, pcol, dtype=torch.uint8, device=x.device)
    gs = global_scale.contiguous()
    with _engine.on_device(x.device):
        st = _engine.lib().fpq_quantize_nv(x.data_ptr(), rows, cols, kind, h.shape[0], norm, h.data_ptr(),
                                           gs.data_ptr(), codes.data_ptr(), scales.data_ptr(), prow, pcol,
                                           _ZERO_POLICY, _stream(x))
    _engine.check(st, "fusedQuantizeNv")
    return codes, scales.view(torch.float8_e4m3fn)


def _packed_weight(lib, wq: torch.Tensor, ws: torch.Tensor, n: int, k: int):
    key = (wq.data_ptr(), getattr(wq, "_version", 0), ws.data_ptr(), getattr(ws, "_version", 0), n, k)
    hit = getattr(wq, "_fpq_packed_for_qutlass", None)
    if hit is not None and hit[0] == key:
        return hit[1], hit[2]
    pc = torch.empty(lib.fpq_packed_codes_bytes(n, k), dtype=torch.uint8, device=wq.device)
    ps = torch.empty(lib.fpq_packed_scales_bytes(n, k), dtype=torch.uint8, device=wq.device)
    _engine.check(lib.fpq_pack_mxf4(wq.data_ptr(), ws.data_ptr(), ws.shape[1], n, k, pc.data_ptr(), ps.data_ptr(),
                                    _stream(wq)), "fpq_pack_mxf4")
    try:
        wq._fpq_packed_for_qutlass = (key, pc, ps)
    except (AttributeError, RuntimeError):
        pass
    return pc, ps


def _matmul(entry: str, group: int, x, w, xs, ws, alpha) -> torch.Tensor:
    _need_gpu(x, w, xs, ws, alpha)
    if x.dtype != torch.uint8 or w.dtype != torch.uint8:
        raise ValueError("packed operands must be uint8")
    if alpha.dtype != torch.float32 or alpha.numel() != 1:
        raise ValueError("alpha must be a one-element float32 tensor")
    xq = x.contiguous().view(-1, x.shape[-1])
    wq = w.contiguous()
    m, kb = xq.shape
    n, k = wq.shape[0], kb * 2
    if wq.shape[1] != kb:
        raise ValueError(f"inner dimensions differ: x has K={k}, w has K={wq.shape[1] * 2}")
    xs_b = xs.contiguous().view(torch.uint8)
    ws_b = ws.contiguous().view(torch.uint8)
    xs_b = xs_b.view(-1, xs_b.shape[-1])
    ws_b = ws_b.view(-1, ws_b.shape[-1])
    if xs_b.shape[0] < m or ws_b.shape[0] < n or xs_b.shape[1] < k // group or ws_b.shape[1] < k // group:
        raise ValueError("scale tensors are smaller than the operands they describe")
    y = torch.empty(*x.shape[:-1], n, dtype=torch.bfloat16, device=x.device)
    a = alpha.contiguous()
    lib = _engine.lib()
    with _engine.on_device(x.device):
        if entry == "fpq_gemm_mxf4" and m >= _PACKED_MIN_M and k % 256 == 0 \
                and os.environ.get("FPQ_PACKED_WEIGHTS", "1") != "0":
            wp, wsp = _packed_weight(lib, wq, ws_b, n, k)
            xp = torch.empty(lib.fpq_packed_codes_bytes(m, k), dtype=torch.uint8, device=x.device)
            xsp = torch.empty(lib.fpq_packed_scales_bytes(m, k), dtype=torch.uint8, device=x.device)
            st = lib.fpq_pack_mxf4(xq.data_ptr(), xs_b.data_ptr(), xs_b.shape[1], m, k, xp.data_ptr(), xsp.data_ptr(),
                                   _stream(x))
            st = st or lib.fpq_gemm_mxf4_packed(xp.data_ptr(), xsp.data_ptr(), wp.data_ptr(), wsp.data_ptr(),
                                                a.data_ptr(), None, y.data_ptr(), m, n, k, _stream(x))
        else:
            st = getattr(lib, entry)(xq.data_ptr(), xs_b.data_ptr(), xs_b.shape[1], wq.data_ptr(), ws_b.data_ptr(),
                                     ws_b.shape[1], a.data_ptr(), None, y.data_ptr(), m, n, k, _stream(x))
    _engine.check(st, entry)
    return y


def matmul_mxf4_bf16_tn(x, w, xs, ws, alpha) -> torch.Tensor:
    """bf16 [..., N] = alpha * dq(x) @ dq(w).T for MXFP4 codes x [..., K/2], w [N, K/2] and E8M0
    scales per 32 (row-major; `to_blocked` of this package leaves them so)."""
    return _matmul("fpq_gemm_mxf4", 32, x, w, xs, ws, alpha)


def matmul_ada_mxf4_bf16_tn(x, w, xs, ws, alpha) -> torch.Tensor:
    """The small-batch entry of QuTLASS (un-blocked scales): the same kernels choose by shape here."""
    return _matmul("fpq_gemm_mxf4", 32, x, w, xs, ws, alpha)


def matmul_nvf4_bf16_tn(x, w, xs, ws, alpha) -> torch.Tensor:
    """The NVFP4 counterpart: E4M3 scales per 16."""
    return _matmul("fpq_gemm_nvf4", 16, x, w, xs, ws, alpha)


def _training_only(name: str):
    def stub(*args, **kwargs):
        raise NotImplementedError(f"qutlass.{name} belongs to the quantized backward pass, which this engine does not have")
    stub.__name__ = name
    return stub


# imported by the reference in the same statement as the functions above (qutlass_ops.py:12-20)
matmul_mxf8_bf16_tn = _training_only("matmul_mxf8_bf16_tn")
matmul_mxf8_bf16_nn = _training_only("matmul_mxf8_bf16_nn")
backward_t_bf16 = _training_only("backward_t_bf16")
backward_qt_bf16 = _training_only("backward_qt_bf16")
backward_bf16_square_double_mxfp8 = _training_only("backward_bf16_square_double_mxfp8")
mxfp4_transpose_mxfp8 = _training_only("mxfp4_transpose_mxfp8")

__all__ = [
    "fusedQuantizeMx", "fusedQuantizeNv", "matmul_ada_mxf4_bf16_tn", "matmul_mxf4_bf16_tn", "matmul_nvf4_bf16_tn",
    "matmul_mxf8_bf16_tn", "matmul_mxf8_bf16_nn", "backward_t_bf16", "backward_qt_bf16",
    "backward_bf16_square_double_mxfp8", "mxfp4_transpose_mxfp8",
]
