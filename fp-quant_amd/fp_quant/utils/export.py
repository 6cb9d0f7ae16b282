"""Round-to-nearest export of a model's linear layers into the *realquant* checkpoint format.

Produces, per converted nn.Linear, the tensors the reference's exporter stores
(src/quantization/rtn.py:159-193): `qweight` (two E2M1 codes per byte), `scales` (E8M0 or E4M3
bytes of group scale x global scale), `forward_hadamard_matrix`, `backward_hadamard_matrix`,
`weight_global_scale`, `act_global_scale`; and writes them the way model_quant.py:39-116 does
(safetensors shards, `model.safetensors.index.json`, `quantization_config` of
src/quantization/qconfig.py:3-21), so that the result loads through
`replace_with_fp_quant_linear` + `load_state_dict` unchanged.

Rules kept from the exporter: MXFP4 uses the fixed global scale 3 (quantizer.py:64-66); NVFP4
tracks 448 * 6 / max|rotated tensor| as a running minimum (quantizer.py:145-150) for weights and,
over calibration batches, for the inputs of each layer; `fuse_global_scale` gives q/k/v and
gate/up of one block the smallest of their weight scales (rtn.py:131-147).  The arithmetic is the
engine's own (fp32 after an exact butterfly rotation, on the GPU), i.e. what `pre_forward`
computes from the same bf16 weights.
"""
import json
import os
import re
from typing import Dict, Iterable, Iterator, List, Optional, Tuple

import torch
from torch import nn

from .config import FPQuantConfig, FPQuantDtype, validate_config
from .replace import _linears, _skipped

FP8_E4M3_MAX = 448.0
FP4_E2M1_MAX = 6.0
MXFP_GLOBAL_SCALE = 3.0

# layers of one block that share a weight global scale under fuse_global_scale (rtn.py:131-147)
FUSED_SCALE_GROUPS = (r"(q|k|v)_proj$", r"(gate|up)_proj$")


def _ops():
    from ..module import hip_ops

    return hip_ops


def _transform_matrix(config: FPQuantConfig, dtype: torch.dtype, device) -> torch.Tensor:
    from ..module.linear import _TRANSFORMS

    try:
        make = _TRANSFORMS[config.transform_init]
    except KeyError:
        raise ValueError(f"Invalid transform init: {config.transform_init}") from None
    return make(config.hadamard_group_size, dtype, device)


def tracked_global_scale(amax: torch.Tensor) -> torch.Tensor:
    """448 * 6 * fl(1 / amax) as a one-element fp32 tensor (quantizer.py:145-150 with the tracker
    starting at +inf).  A tensor of zeros has no such scale and raises, as the reference does."""
    amax = amax.detach().to(torch.float32).reshape(1)
    if not bool(torch.isfinite(amax).all()) or float(amax) == 0.0:
        raise ValueError(f"Global scale is not finite: absolute maximum {float(amax)}")
    return torch.tensor([FP8_E4M3_MAX * FP4_E2M1_MAX], dtype=torch.float32, device=amax.device) * (1.0 / amax)


class ActivationScaleTracker:
    """Tracks, per converted nn.Linear, the maximum |rotated input| over the forward passes run
    while it is attached (the calibration pass of rtn.py:150-155), on the GPU.

        with ActivationScaleTracker(model, config) as tracker:
            for batch in calibration_data:
                model(batch)
        act_scales = tracker.global_scales()
    """

    def __init__(self, model: nn.Module, config: FPQuantConfig):
        self.config = config
        self.amax: Dict[str, torch.Tensor] = {}
        self._handles = []
        self._targets = [(name, parent._modules[child]) for parent, child, name in _linears(model, None)
                         if not _skipped(name, config)]
        self._h = {}

    def _hook(self, name: str):
        def pre_forward(module, args):
            x = args[0]
            h = self._h.get(x.device)
            if h is None:
                h = self._h[x.device] = _transform_matrix(self.config, torch.bfloat16, x.device)
            self.amax[name] = _ops().rotated_absmax(x.detach().to(torch.bfloat16), h, self.amax.get(name))
        return pre_forward

    def __enter__(self):
        for name, module in self._targets:
            self._handles.append(module.register_forward_pre_hook(self._hook(name)))
        return self

    def __exit__(self, *exc):
        for handle in self._handles:
            handle.remove()
        self._handles = []
        return False

    def global_scales(self) -> Dict[str, torch.Tensor]:
        return {name: tracked_global_scale(a) for name, a in self.amax.items()}


def export_linear(
    weight: torch.Tensor,
    config: FPQuantConfig,
    weight_global_scale: Optional[torch.Tensor] = None,
    act_global_scale: Optional[torch.Tensor] = None,
) -> Dict[str, torch.Tensor]:
    """The realquant tensors of one [out, in] weight on a GPU (rtn.py:185-193).

    MXFP4 ignores the scale arguments (both are 3).  NVFP4 tracks the weight scale from the rotated
    weight unless one is given (a fused q/k/v scale) and needs `act_global_scale` from calibration."""
    from ..module.linear_fns import forward_quantize

    validate_config(config)
    if config.forward_method != "abs_max":
        raise ValueError("the round-to-nearest export uses forward_method='abs_max'")
    if not weight.is_cuda:
        raise ValueError("export_linear needs the weight on a GPU; there is no CPU path")
    w = weight.detach().to(torch.bfloat16).contiguous()
    h = _transform_matrix(config, w.dtype, w.device)
    if w.shape[1] % config.hadamard_group_size != 0:
        raise ValueError(f"in_features {w.shape[1]} is not a multiple of the rotation size {config.hadamard_group_size}")
    if config.forward_dtype == FPQuantDtype.MXFP4:
        group = 32
        wgs = torch.tensor([MXFP_GLOBAL_SCALE], dtype=torch.float32, device=w.device)
        ags = wgs.clone()
    elif config.forward_dtype == FPQuantDtype.NVFP4:
        group = 16
        if weight_global_scale is None:
            weight_global_scale = tracked_global_scale(_ops().rotated_absmax(w, h))
        if act_global_scale is None:
            raise ValueError("NVFP4 export needs act_global_scale (see ActivationScaleTracker)")
        wgs = weight_global_scale.detach().to(device=w.device, dtype=torch.float32).reshape(1)
        ags = act_global_scale.detach().to(device=w.device, dtype=torch.float32).reshape(1)
    else:
        raise ValueError(f"Unsupported forward dtype: {config.forward_dtype}")
    codes, scales, _ = forward_quantize(w, h, wgs, config.forward_dtype, "abs_max")
    scales = scales.view(torch.uint8)[: w.shape[0], : w.shape[1] // group].contiguous()
    return {
        "qweight": codes,
        "scales": scales,
        "forward_hadamard_matrix": h,
        "backward_hadamard_matrix": h.clone(),
        "weight_global_scale": wgs.clone(),
        "act_global_scale": ags.clone(),
    }


def _fused_groups(names: Iterable[str]) -> Iterator[List[str]]:
    """Names that share a parent module and match one pattern of FUSED_SCALE_GROUPS."""
    buckets: Dict[Tuple[str, int], List[str]] = {}
    for name in names:
        parent, _, leaf = name.rpartition(".")
        for i, pattern in enumerate(FUSED_SCALE_GROUPS):
            if re.search(pattern, leaf):
                buckets.setdefault((parent, i), []).append(name)
    for members in buckets.values():
        if len(members) > 1:
            yield members


@torch.no_grad()
def rtn_export(
    model: nn.Module,
    config: FPQuantConfig,
    act_global_scales: Optional[Dict[str, torch.Tensor]] = None,
    fuse_global_scale: bool = False,
    device: Optional[torch.device] = None,
) -> Dict[str, torch.Tensor]:
    """State dict of `model` with every convertible nn.Linear's `weight` replaced by its realquant
    tensors (`<name>.qweight`, `<name>.scales`, ...); everything else is passed through, all on the
    CPU (model_quant.py:49-71).  Weights are moved to `device` (default: the current GPU) one layer
    at a time, so the model itself may live on the CPU."""
    validate_config(config)
    device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    nvfp4 = config.forward_dtype == FPQuantDtype.NVFP4
    targets = {name: parent._modules[child] for parent, child, name in _linears(model, None)
               if not _skipped(name, config)}
    weight_scales: Dict[str, torch.Tensor] = {}
    if nvfp4:
        if act_global_scales is None:
            raise ValueError("NVFP4 export needs act_global_scales (see ActivationScaleTracker)")
        missing = [n for n in targets if n not in act_global_scales]
        if missing:
            raise ValueError(f"no activation global scale for: {', '.join(missing[:4])}")
        h = _transform_matrix(config, torch.bfloat16, device)
        for name, layer in targets.items():
            w = layer.weight.detach().to(device=device, dtype=torch.bfloat16)
            weight_scales[name] = tracked_global_scale(_ops().rotated_absmax(w, h))
        if fuse_global_scale:
            for members in _fused_groups(targets):
                shared = torch.stack([weight_scales[m] for m in members]).min(dim=0).values
                for m in members:
                    weight_scales[m] = shared
    out: Dict[str, torch.Tensor] = {}
    converted = {f"{name}.weight": name for name in targets}
    for key, value in model.state_dict().items():
        name = converted.get(key)
        if name is None:
            out[key] = value.detach().cpu()
            continue
        tensors = export_linear(
            targets[name].weight.to(device), config,
            weight_global_scale=weight_scales.get(name),
            act_global_scale=act_global_scales[name] if nvfp4 else None,
        )
        for k, v in tensors.items():
            out[f"{name}.{k}"] = v.cpu()
    return out


def quantization_config_dict(config: FPQuantConfig) -> Dict[str, object]:
    """`quantization_config` entry of the saved model config (src/quantization/qconfig.py:3-21): the
    inference configuration of what was exported."""
    entry = config.to_dict()
    entry.update(backward_dtype="bf16", forward_method="abs_max", store_master_weights=False,
                 pseudoquantization=False)
    if config.transform_init == "hadamard":   # the reference's entry has no such key; only say what differs
        del entry["transform_init"]
    return entry


def save_realquant_checkpoint(
    state_dict: Dict[str, torch.Tensor],
    save_path: str,
    config: Optional[FPQuantConfig] = None,
    model_config=None,
    max_shard_size: int = 5 * 1024 ** 3,
) -> List[str]:
    """Write `state_dict` as safetensors shards plus `model.safetensors.index.json`
    (model_quant.py:73-107); with a Hugging Face `model_config`, also `config.json` carrying the
    quantization config (model_quant.py:109-116).  Returns the shard file names."""
    from safetensors.torch import save_file

    os.makedirs(save_path, exist_ok=True)
    shards: List[Dict[str, torch.Tensor]] = []
    current: Dict[str, torch.Tensor] = {}
    current_size = 0
    for key, value in state_dict.items():
        size = value.numel() * value.element_size()
        if current and current_size + size > max_shard_size:
            shards.append(current)
            current, current_size = {}, 0
        current[key] = value.contiguous()
        current_size += size
    if current:
        shards.append(current)
    digits = len(str(max(len(shards), 1)))
    index: Dict[str, str] = {}
    names = []
    for i, shard in enumerate(shards):
        name = f"model-{str(i + 1).zfill(digits)}-of-{str(len(shards)).zfill(digits)}.safetensors"
        save_file(shard, os.path.join(save_path, name))
        names.append(name)
        for key in shard:
            index[key] = name
    with open(os.path.join(save_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": index}, f)
    if model_config is not None:
        if config is None:
            raise ValueError("saving a model config needs the FPQuantConfig that was exported")
        model_config.quantization_config = quantization_config_dict(config)
        model_config.save_pretrained(save_path)
    return names
