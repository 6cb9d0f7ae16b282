"""Forward pieces of the quantized linear: activation quantize -> W4A4 GEMM -> bias.

Mirrors `forward_quantize`, `forward_gemm` and `FPQuant4x16NoMasterFn` of the reference
(inference_lib/src/fp_quant/module/linear_fns.py:27-64, 482-534): same argument order, same
returned tuples, same exceptions.
"""
from typing import Optional, Tuple

import torch
from torch.autograd import Function

from ..utils import FPQuantDtype
from .hip_ops import (
    as_bf16,
    fused_quantize_mx_op,
    fused_quantize_nv_op,
    linear_alpha_op,
    matmul_mxf4_bf16_tn_bias_op,
    matmul_mxf4_bf16_tn_op,
    matmul_nvf4_bf16_tn_bias_op,
    matmul_nvf4_bf16_tn_op,
    linear_mxf4_packed_op,
    packed_linear_eligible,
)
from .eager import linear_alpha, linear_w4a4, linear_w4a4_op


def forward_quantize(
    x: torch.Tensor,
    hadamard_matrix: torch.Tensor,
    global_scale: torch.Tensor,
    dtype: FPQuantDtype,
    forward_method: str,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(packed codes, scales, clip mask or None) of x rotated by `hadamard_matrix`."""
    if dtype == FPQuantDtype.MXFP4:
        want_mask = forward_method == "quest" and x.requires_grad
        return fused_quantize_mx_op(x.to(torch.bfloat16), as_bf16(hadamard_matrix), forward_method, want_mask)
    if dtype == FPQuantDtype.NVFP4:
        codes, scales = fused_quantize_nv_op(x.to(torch.bfloat16), as_bf16(hadamard_matrix), global_scale.float())
        return codes, scales, None
    raise ValueError(f"Unsupported forward dtype: {dtype}")


def forward_gemm(x_q, w_q, x_scales, w_scales, alpha, dtype: FPQuantDtype, bias=None):
    """bf16(alpha * dq(x_q) @ dq(w_q).T), optionally followed by the bf16 bias add in the
    same kernel.  The library chooses the small-M kernel by shape."""
    if dtype == FPQuantDtype.MXFP4:
        if bias is None:
            return matmul_mxf4_bf16_tn_op(x_q, w_q, x_scales, w_scales, alpha.float())
        return matmul_mxf4_bf16_tn_bias_op(x_q, w_q, x_scales, w_scales, alpha.float(), bias)
    if dtype == FPQuantDtype.NVFP4:
        if bias is None:
            return matmul_nvf4_bf16_tn_op(x_q, w_q, x_scales, w_scales, alpha.float())
        return matmul_nvf4_bf16_tn_bias_op(x_q, w_q, x_scales, w_scales, alpha.float(), bias)
    raise ValueError(f"Unsupported dtype: {dtype}")


class FPQuant4x16NoMasterFn(Function):
    """Inference-only W4A4 linear on pre-quantized weights (no backward)."""

    @staticmethod
    def forward(
        ctx,
        x: torch.Tensor,
        weight_q: torch.Tensor,
        weight_scales: torch.Tensor,
        weight_global_scale: torch.Tensor,
        act_global_scale: torch.Tensor,
        bias: Optional[torch.Tensor],
        forward_hadamard_matrix: torch.Tensor,
        dtype: FPQuantDtype,
        forward_method: str,
        residual: Optional[torch.Tensor] = None,
    ):
        """`residual` (not in the reference's signature): a tensor of the output's shape added to
        the result as a separate bf16 addition would, inside the GEMM where the kernel can."""
        x_flat = x.contiguous().flatten(end_dim=-2)
        res_flat = residual.contiguous().flatten(end_dim=-2) if residual is not None else None
        # quest (MXFP4 only, validate_config) takes the same road when no clip mask is wanted
        quest = forward_method == "quest" and dtype == FPQuantDtype.MXFP4 and not x.requires_grad
        direct = ((forward_method == "abs_max" and dtype in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4)) or quest)
        plain = weight_q.is_contiguous() and weight_scales.is_contiguous()
        # a bias the kernels can add in their epilogue; any other is added afterwards, like the reference's `y += bias`
        fused_bias = bias if (bias is not None and bias.dtype == torch.bfloat16 and bias.is_contiguous()) else None
        residual_done = False
        if direct and plain and not torch.compiler.is_compiling():
            # eager calls: the kernels of the operators below without operator dispatch, with alpha and the
            # fp32 global scale computed once per layer; the residual rides in the GEMM when nothing has to
            # be added between the GEMM and it
            res_in = res_flat if (bias is None or fused_bias is not None) else None
            y = linear_w4a4(x_flat.to(torch.bfloat16), forward_hadamard_matrix, weight_q, weight_scales,
                            linear_alpha(weight_global_scale, act_global_scale), act_global_scale, fused_bias,
                            dtype == FPQuantDtype.NVFP4, shared_source=x, residual=res_in, quest=quest)
            residual_done = res_in is not None
        elif direct and plain and x_flat.is_cuda:
            # traced callers: the eager body above as one operator
            y = linear_w4a4_op(x_flat.to(torch.bfloat16), forward_hadamard_matrix, weight_q, weight_scales,
                               weight_global_scale, act_global_scale, fused_bias, dtype == FPQuantDtype.NVFP4, quest)
        elif (dtype == FPQuantDtype.MXFP4 and x_flat.is_cuda
                and packed_linear_eligible(x_flat.shape[0], x_flat.shape[1], forward_method)):
            # quantize and multiply on operands in the matrix units' own order
            y = linear_mxf4_packed_op(x_flat.to(torch.bfloat16), as_bf16(forward_hadamard_matrix), weight_q,
                                      weight_scales, linear_alpha_op(weight_global_scale, act_global_scale), fused_bias)
        else:
            # the reference's operator chain (quest with a clip mask, strided weights, CPU tensors raise in the operators)
            x_q, x_scales, _ = forward_quantize(x_flat, forward_hadamard_matrix, act_global_scale, dtype, forward_method)
            # alpha is evaluated in the buffers' dtype, as the reference does (bf16 buffers round 1/9)
            y = forward_gemm(x_q, weight_q, x_scales, weight_scales,
                             linear_alpha_op(weight_global_scale, act_global_scale), dtype, fused_bias)
        y = y.view(*x.shape[:-1], y.shape[-1])
        if bias is not None and fused_bias is None:
            y += bias
        if residual is not None and not residual_done:
            y = y + residual
        return y

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        raise NotImplementedError("Backward pass is not implemented for FPQuant4x16NoMasterFn yet")
