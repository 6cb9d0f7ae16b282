"""Host logic of the round-to-nearest exporter that needs no GPU: the tracked global scale, the
fused-scale grouping, the quantization config entry and the checkpoint writer."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import fpq_oracle as O


def test_tracked_global_scale_matches_oracle_rule():
    from fp_quant.utils import export
    for amax in (4.0, 0.3740234375, 1e-3, 12345.0):
        got = export.tracked_global_scale(torch.tensor([amax]))
        assert got.dtype == torch.float32 and got.shape == (1,)
        assert float(got) == O.nv_tracked_global_scale(torch.tensor([[amax, -amax / 2]]))
    # by hand (quantizer.py:145): 448 * 6 * fl32(1 / 4) = 672
    assert float(export.tracked_global_scale(torch.tensor([4.0]))) == 672.0
    f32 = np.float32
    assert float(export.tracked_global_scale(torch.tensor([3.0]))) == float(f32(2688.0) * (f32(1.0) / f32(3.0)))
    for bad in (0.0, float("inf"), float("nan")):
        with pytest.raises(ValueError):
            export.tracked_global_scale(torch.tensor([bad]))


def test_fused_groups_follow_the_exporter():
    from fp_quant.utils import export
    names = [f"model.layers.{i}.{m}" for i in range(2) for m in
             ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
              "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")]
    groups = sorted(sorted(g) for g in export._fused_groups(names))
    assert groups == sorted(
        [sorted(f"model.layers.{i}.self_attn.{p}_proj" for p in "qkv") for i in range(2)]
        + [sorted(f"model.layers.{i}.mlp.{p}_proj" for p in ("gate", "up")) for i in range(2)])


def test_quantization_config_entry():
    import fp_quant
    from fp_quant.utils import export
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.NVFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=16)
    # keys and values of src/quantization/qconfig.py:9-18 for format "nvfp"
    assert export.quantization_config_dict(cfg) == {
        "forward_dtype": "nvfp4", "backward_dtype": "bf16", "forward_method": "abs_max",
        "hadamard_group_size": 16, "modules_to_not_convert": ["lm_head"], "quant_method": "fp_quant",
        "store_master_weights": False, "pseudoquantization": False}


def test_checkpoint_writer_shards_and_indexes(tmp_path):
    from safetensors.torch import load_file
    from fp_quant.utils import export
    gen = torch.Generator().manual_seed(0)
    state = {f"t{i}": torch.randint(0, 255, (1000,), dtype=torch.uint8, generator=gen) for i in range(5)}
    state["big"] = torch.randn(4000, generator=gen).to(torch.bfloat16)
    names = export.save_realquant_checkpoint(state, str(tmp_path), max_shard_size=2500)
    assert names == [f"model-{i}-of-4.safetensors" for i in range(1, 5)]
    index = json.load(open(os.path.join(tmp_path, "model.safetensors.index.json")))
    assert index["metadata"] == {} and sorted(index["weight_map"]) == sorted(state)
    for key, value in state.items():
        shard = load_file(os.path.join(tmp_path, index["weight_map"][key]))
        assert torch.equal(shard[key], value)
    assert index["weight_map"]["t0"] == index["weight_map"]["t1"] != index["weight_map"]["t2"]
    assert index["weight_map"]["big"] == "model-4-of-4.safetensors"


def test_export_has_no_cpu_path():
    import fp_quant
    from fp_quant.utils import export
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=32)
    with pytest.raises(ValueError):
        export.export_linear(torch.zeros(32, 64, dtype=torch.bfloat16), cfg)
    cfg.forward_method = "quest"
    with pytest.raises(ValueError):
        export.export_linear(torch.zeros(32, 64, dtype=torch.bfloat16), cfg)
