"""FPQuantLinear: the quantized linear layer of the inference path.

Keeps the constructor, parameter/buffer names, shapes and dtypes, `pre_forward()` and the
inference branch of `forward()` of the reference module
(inference_lib/src/fp_quant/module/linear.py:24-368), so state dicts and loaders written for
the reference work unchanged.  Training branches (master weights, quantized backward) and
pseudo-quantization are not part of this engine and raise.
"""
import os
from typing import Optional

import torch
from torch import nn

from ..utils import FPQuantConfig, FPQuantDtype, validate_config
from . import eager, hip_ops
from .linear_fns import FPQuant4x16NoMasterFn, forward_quantize

def _sylvester_signs(n: int) -> torch.Tensor:
    """+-1 Sylvester-Hadamard matrix, entry (i, j) = (-1)^popcount(i & j) (== scipy.linalg.hadamard)."""
    h = torch.ones(1, 1, dtype=torch.float64)
    while h.shape[0] < n:
        h = torch.cat((torch.cat((h, h), dim=1), torch.cat((h, -h), dim=1)), dim=0)
    if h.shape[0] != n:
        raise ValueError(f"Hadamard size must be a power of two, got {n}")
    return h


def get_hadamard_matrix(group_size: int, dtype: torch.dtype, device: torch.device):
    """hadamard(g) * g**-0.5 rounded to `dtype` (linear.py:24-30)."""
    return (_sylvester_signs(group_size) * group_size ** -0.5).to(dtype=dtype, device=device)


def get_identity_matrix(group_size: int, dtype: torch.dtype, device: torch.device):
    return torch.eye(group_size, dtype=dtype, device=device)


def get_gsr_matrix(group_size: int, dtype: torch.dtype, device: torch.device):
    """Hadamard matrix with columns sorted by their number of sign changes (linear.py:37-41)."""
    had = get_hadamard_matrix(group_size, dtype, device)
    order = torch.argsort(torch.diff(had, dim=0).ne(0).sum(dim=0))
    return had[:, order].contiguous()


_TRANSFORMS = {"hadamard": get_hadamard_matrix, "identity": get_identity_matrix, "gsr": get_gsr_matrix}


def _no_master_forward(*args):
    return FPQuant4x16NoMasterFn.forward(None, *args)


class FPQuantLinear(nn.Module):
    def __init__(
        self,
        in_features: int,
        out_features: int,
        config: FPQuantConfig,
        bias: bool = True,
        device: torch.device = None,
        dtype: torch.dtype = None,
    ):
        super().__init__()
        validate_config(config)
        if config.pseudoquantization:
            raise ValueError(
                "pseudoquantization=True is not available: this engine runs real FP4 kernels only"
            )
        if not hip_ops.HAS_HIP_ENGINE:
            raise ValueError(
                "libfpq_hip.so is not built or failed to load; build it with `python fp-quant_amd/build.py`"
            )
        group = config.forward_dtype.scale_group if config.forward_dtype in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4) else None
        if group is None:
            raise ValueError(f"Unsupported forward dtype: {config.forward_dtype}")

        factory = {"device": device, "dtype": dtype}
        self.in_features = in_features
        self.out_features = out_features
        self.config = config
        self.weight = nn.Parameter(torch.empty((out_features, in_features), **factory))
        self.dqweight = nn.Parameter(torch.empty((out_features, in_features), **factory))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features, **factory))
        else:
            self.register_parameter("bias", None)

        dev = self.weight.device
        self.register_buffer("qweight", torch.empty(out_features, in_features // 2, dtype=torch.uint8, device=dev))
        self.register_buffer("scales", torch.empty(out_features, in_features // group, dtype=torch.uint8, device=dev))
        self.register_buffer("weight_global_scale", torch.empty(1, **factory))
        self.register_buffer("act_global_scale", torch.empty(1, **factory))
        g = config.hadamard_group_size
        self.register_buffer("forward_hadamard_matrix", torch.empty(g, g, **factory))
        self.register_buffer("backward_hadamard_matrix", torch.empty(g, g, **factory))
        self._register_load_state_dict_pre_hook(FPQuantLinear._before_load, with_module=True)
        self.register_load_state_dict_post_hook(FPQuantLinear._prime)
        self._register_state_dict_hook(FPQuantLinear._row_major_state)

    @torch.no_grad()
    def pre_forward(self):
        """Build the rotation and global-scale buffers and quantize `weight` into
        `qweight`/`scales` (linear.py:154-248, real-quant branch)."""
        cfg = self.config
        g = cfg.hadamard_group_size
        assert self.weight.shape[1] % g == 0, (
            f"Weight shape must be divisible by hadamard group size: {self.weight.shape[1]} % {g} = "
            f"{self.weight.shape[1] % g}"
        )
        assert self.weight.data.device.type in ("cuda", "xpu"), (
            f"Weight must be on CUDA or XPU, but is on {self.weight.device}"
        )
        try:
            make = _TRANSFORMS[cfg.transform_init]
        except KeyError:
            raise ValueError(f"Invalid transform init: {cfg.transform_init}") from None
        wdtype, wdev = self.weight.dtype, self.weight.device
        self.forward_hadamard_matrix = nn.Buffer(make(g, wdtype, wdev))
        self.backward_hadamard_matrix = nn.Buffer(make(g, wdtype, wdev))

        if cfg.forward_dtype == FPQuantDtype.MXFP4 and cfg.forward_method == "quest":
            global_scale_val = 1.0
        elif cfg.forward_method == "abs_max":
            global_scale_val = 3.0  # abs-max MXFP4 carries an implicit factor 3 per operand
        elif cfg.forward_dtype == FPQuantDtype.NVFP4:
            global_scale_val = 10.0
        self.weight_global_scale = nn.Buffer(torch.tensor([global_scale_val], dtype=wdtype, device=wdev))
        self.act_global_scale = nn.Buffer(torch.tensor([global_scale_val], dtype=wdtype, device=wdev))

        if cfg.store_master_weights:
            self.qweight = None
            self.scales = None
            self.dqweight = None
            return
        weight_q, scales, _ = forward_quantize(
            self.weight, self.forward_hadamard_matrix, self.weight_global_scale,
            cfg.forward_dtype, cfg.forward_method,
        )
        group = cfg.forward_dtype.scale_group
        rows, cols = self.weight.shape[0], self.weight.shape[1] // group
        scales = scales.view(dtype=torch.uint8)[:rows, :cols].contiguous()  # drop the op's padding
        self.qweight = nn.Parameter(weight_q, requires_grad=False)
        self.scales = nn.Parameter(scales, requires_grad=False)
        self.weight = None
        self.dqweight = None
        self._prime()

    def _prime(self, *_):
        """Per-call constants (rotation kind, alpha, fp32 global scale) computed now rather than inside
        the first forward, which may be a traced one or a graph capture; also run after load_state_dict.
        What a recorded graph may point at keeps its address when the weight was rewritten in place: the
        split-K workspace stays, and a packed copy of the old weight is re-packed into its own buffers."""
        h, wgs, ags = self.forward_hadamard_matrix, self.weight_global_scale, self.act_global_scale
        q, s = getattr(self, "qweight", None), getattr(self, "scales", None)
        stale = getattr(q, "_fpq_packed", None) if isinstance(q, torch.Tensor) else None
        # whatever was remembered about the old contents goes (in-place copies under torch.inference_mode()
        # leave no trace in a tensor's modification counter)
        hip_ops.drop_tensor_caches(h, wgs, ags, q, s, keep=("_fpq_splitk", "_fpq_alpha", "_fpq_f32"))
        if all(isinstance(t, torch.Tensor) and t.is_cuda for t in (h, wgs, ags)):
            eager.prime(h, wgs, ags, refresh=True)   # alpha and the fp32 scale: new values in the old tensors
        else:
            hip_ops.drop_tensor_caches(wgs, ags)
        if (stale is not None and isinstance(s, torch.Tensor) and q.is_cuda and q.dim() == 2 and s.dim() == 2
                and q.dtype == torch.uint8 and s.dtype == torch.uint8 and q.is_contiguous() and s.is_contiguous()
                and hip_ops.packed_weights_enabled() and not torch.cuda.is_current_stream_capturing()):
            hip_ops.packed_weight(q, s, self.config.forward_dtype == FPQuantDtype.NVFP4, into=(stale[1], stale[2]))
        if self._fpq_single_copy or os.environ.get("FPQ_SINGLE_WEIGHT_COPY", "0") == "1":
            self.release_row_major()
        self._ensure_splitk_workspace()

    def _ensure_splitk_workspace(self) -> None:
        """The layer's split-K workspace (hip_ops.splitk_workspace) made now, outside any trace or capture,
        so that every later call -- eager, traced, captured -- takes the same kernel."""
        qweight = getattr(self, "qweight", None)
        if (isinstance(qweight, torch.Tensor) and qweight.is_cuda and hip_ops.packed_weights_enabled()
                and self.config.forward_dtype in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4)
                and self.in_features % 256 == 0):
            hip_ops.splitk_workspace(qweight, self.out_features, self.in_features, True,
                                     nvfp4=self.config.forward_dtype == FPQuantDtype.NVFP4)

    # True once release_row_major has been asked for: the layer goes back to the packed layout after
    # every load_state_dict
    _fpq_single_copy = False

    @property
    def weights_packed_only(self) -> bool:
        q = getattr(self, "qweight", None)
        return isinstance(q, torch.Tensor) and hip_ops.is_packed_only(q)

    @torch.no_grad()
    def release_row_major(self) -> bool:
        """Keep the 4-bit weight once: `qweight` and `scales` become the 1-D buffers of the packed
        layout the GEMM kernels read (what is otherwise a second copy next to the row-major tensors of
        the reference, linear.py:87-88), and the row-major tensors are freed.  state_dict() still hands
        out the reference's row-major tensors (re-tiled on demand) and load_state_dict() accepts them.
        MXFP4 or NVFP4 with in_features % 256 == 0 and out_features % 32 == 0 on a GPU; returns whether
        the layer is in that state afterwards."""
        if self.weights_packed_only:
            return True
        q, s = getattr(self, "qweight", None), getattr(self, "scales", None)
        nvfp4 = self.config.forward_dtype == FPQuantDtype.NVFP4
        if not hip_ops.packed_weights_enabled():   # FPQ_PACKED_WEIGHTS=0: every call stays on the row-major kernels
            return False
        if (self.config.forward_dtype not in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4) or q is None or s is None
                or not q.is_cuda or q.dim() != 2 or q.dtype != torch.uint8 or s.dtype != torch.uint8
                or self.in_features % 256 != 0 or self.out_features % 32 != 0
                or tuple(q.shape) != (self.out_features, self.in_features // 2)
                or tuple(s.shape) != (self.out_features, self.in_features // self.config.forward_dtype.scale_group)):
            return False
        pc, ps = hip_ops.packed_weight(q.contiguous(), s.contiguous(), nvfp4)
        workspace = getattr(q, "_fpq_splitk", None)
        hip_ops.drop_tensor_caches(q, s)
        self.qweight = nn.Parameter(pc, requires_grad=False)
        self.scales = nn.Parameter(ps, requires_grad=False)
        if workspace is not None:
            self.qweight._fpq_splitk = workspace   # the layer's, whichever tensor holds its weight
        self._fpq_single_copy = True
        self._ensure_splitk_workspace()
        return True

    @torch.no_grad()
    def restore_row_major(self) -> None:
        """Undo release_row_major: `qweight` [out, in/2] and `scales` [out, in/32] as the reference holds them."""
        if not self.weights_packed_only:
            return
        nvfp4 = self.config.forward_dtype == FPQuantDtype.NVFP4
        pc, ps = self.qweight.detach(), self.scales.detach()
        workspace = getattr(self.qweight, "_fpq_splitk", None)
        codes, scales = hip_ops.unpack_fp4(pc, ps, self.out_features, self.in_features, nvfp4)
        self.qweight = nn.Parameter(codes, requires_grad=False)
        self.scales = nn.Parameter(scales, requires_grad=False)
        # the packed buffers stay the row-major tensors' packed copy (same addresses; re-packed in place when
        # the weight is rewritten)
        hip_ops.adopt_packed_weight(self.qweight, self.scales, nvfp4, pc, ps)
        if workspace is not None:
            self.qweight._fpq_splitk = workspace
        self._fpq_single_copy = False
        self._ensure_splitk_workspace()

    def _row_major_state(self, state_dict, prefix, local_metadata):
        """state_dict() hook: a layer that holds the packed layout only hands out row-major tensors."""
        if self.weights_packed_only and prefix + "qweight" in state_dict and prefix + "scales" in state_dict:
            with torch.no_grad():
                codes, scales = hip_ops.unpack_fp4(self.qweight.detach(), self.scales.detach(), self.out_features,
                                                   self.in_features, self.config.forward_dtype == FPQuantDtype.NVFP4)
            state_dict[prefix + "qweight"], state_dict[prefix + "scales"] = codes, scales

    def _before_load(self, state_dict, prefix, *_):
        """load_state_dict() pre-hook: row-major parameters to load into (the post-hook packs them again)."""
        if self.weights_packed_only and (prefix + "qweight" in state_dict or prefix + "scales" in state_dict):
            self.restore_row_major()
            self._fpq_single_copy = True

    # A tensor of the output's shape that the next forward adds to its result (inside the GEMM
    # where the kernel can) and then clears; set by a fused decoder block around its attention call.
    # It stays set when the forward cannot take it (autograd), and the block then adds it itself.
    # Host-side state of the module: two threads must not run the same fused block at the same time.
    _fpq_residual: Optional[torch.Tensor] = None

    def forward(self, x) -> torch.Tensor:
        cfg = self.config
        if (
            cfg.forward_dtype in (FPQuantDtype.MXFP4, FPQuantDtype.NVFP4)
            and cfg.backward_dtype == FPQuantDtype.BF16
            and not cfg.store_master_weights
            and not cfg.pseudoquantization
        ):
            # no autograd graph to build (inference): call the forward directly
            fn = (FPQuant4x16NoMasterFn.apply if (torch.is_grad_enabled() and x.requires_grad)
                  else _no_master_forward)
            extra = ()
            residual = self._fpq_residual
            if (residual is not None and fn is _no_master_forward and not residual.requires_grad
                    and residual.shape[:-1] == x.shape[:-1] and residual.shape[-1] == self.out_features):
                self._fpq_residual = None
                extra = (residual,)
            return fn(
                x,
                self.qweight,
                self.scales,
                self.weight_global_scale,
                self.act_global_scale,
                self.bias,
                self.forward_hadamard_matrix,
                cfg.forward_dtype,
                cfg.forward_method,
                *extra,
            )
        raise ValueError(
            f"Forward dtype: {cfg.forward_dtype}, backward dtype: {cfg.backward_dtype}, "
            f"store_master_weights: {cfg.store_master_weights}, pseudoquantization: "
            f"{cfg.pseudoquantization} isn't supported yet."
        )

    def forward_quantized(self, activations, leading_shape, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The GEMM (+ bias) of `forward` on activations that a fused producer has already rotated and
        quantized for this layer (`eager.QuantizedActivations`); returns [*leading_shape, out].
        `residual` ([*leading_shape, out], bf16) is added to the result as a separate bf16 addition
        would add it, inside the GEMM where the kernel can."""
        alpha = eager.linear_alpha(self.weight_global_scale, self.act_global_scale)
        bias = self.bias
        fused_bias = bias if (bias is not None and bias.dtype == torch.bfloat16 and bias.is_contiguous()) else None
        in_gemm = residual is not None and (bias is None or fused_bias is not None)
        with hip_ops.on_device(self.qweight.device):
            y = eager.linear_on(activations, self.qweight, self.scales, alpha, fused_bias,
                                  hip_ops._current_stream(self.qweight.device.index),
                                  residual=residual.contiguous().flatten(end_dim=-2) if in_gemm else None,
                                  remember=True)
        y = y.view(*leading_shape, y.shape[-1])
        if bias is not None and fused_bias is None:
            y += bias
        if residual is not None and not in_gemm:
            y += residual
        return y
