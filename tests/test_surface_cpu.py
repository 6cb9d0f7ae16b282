"""CPU-side checks of the fp_quant surface: exported names, config validation, module
buffers/shapes, replace helpers on the meta device, loud failure without a GPU."""
import pytest
import torch
from torch import nn

import fp_quant
from fp_quant import FPQuantConfig, FPQuantDtype, FPQuantLinear
from fp_quant.utils import validate_config


def test_exports():
    for name in ("FPQuantLinear", "FPQuantConfig", "FPQuantDtype", "replace_with_fp_quant_linear",
                 "replace_quantize_with_fp_quant_linear", "finalize_master_weights"):
        assert hasattr(fp_quant, name)


def test_config_defaults_match_reference_dataclass():
    c = FPQuantConfig()
    assert (c.forward_dtype, c.forward_method, c.backward_dtype) == (FPQuantDtype.MXFP4, "quest", FPQuantDtype.MXFP4)
    assert (c.store_master_weights, c.hadamard_group_size, c.pseudoquantization) == (False, 32, False)
    assert c.transform_init == "hadamard" and c.modules_to_not_convert == ["lm_head"]
    assert [d.value for d in FPQuantDtype] == ["mxfp4", "nvfp4", "mxfp8", "bf16"]


@pytest.mark.parametrize("kw,ok", [
    (dict(forward_dtype=FPQuantDtype.NVFP4, forward_method="quest", backward_dtype=FPQuantDtype.BF16), False),
    (dict(forward_dtype=FPQuantDtype.NVFP4, forward_method="abs_max", backward_dtype=FPQuantDtype.BF16,
          hadamard_group_size=16), True),
    (dict(forward_dtype=FPQuantDtype.NVFP4, forward_method="abs_max", backward_dtype=FPQuantDtype.BF16,
          hadamard_group_size=8), False),
    (dict(forward_dtype=FPQuantDtype.MXFP4, hadamard_group_size=16), False),
    (dict(forward_dtype=FPQuantDtype.MXFP4, hadamard_group_size=128), True),
    (dict(forward_dtype=FPQuantDtype.MXFP8), False),
    (dict(forward_dtype=FPQuantDtype.NVFP4, forward_method="abs_max", backward_dtype=FPQuantDtype.MXFP8,
          hadamard_group_size=16), False),
    (dict(forward_dtype=FPQuantDtype.MXFP4, backward_dtype=FPQuantDtype.MXFP8), True),
    (dict(forward_dtype=FPQuantDtype.NVFP4, forward_method="abs_max", backward_dtype=FPQuantDtype.MXFP4,
          hadamard_group_size=16), False),
])
def test_validate_config(kw, ok):
    cfg = FPQuantConfig(**kw)
    if ok:
        validate_config(cfg)
    else:
        with pytest.raises(ValueError):
            validate_config(cfg)


@pytest.mark.parametrize("fmt,group", [(FPQuantDtype.MXFP4, 32), (FPQuantDtype.NVFP4, 16)])
def test_module_buffers(fmt, group):
    cfg = FPQuantConfig(forward_dtype=fmt, forward_method="abs_max", backward_dtype=FPQuantDtype.BF16,
                        hadamard_group_size=64)
    lin = FPQuantLinear(256, 96, cfg, bias=True, dtype=torch.bfloat16)
    sd = lin.state_dict()
    assert sd["qweight"].shape == (96, 128) and sd["qweight"].dtype == torch.uint8
    assert sd["scales"].shape == (96, 256 // group) and sd["scales"].dtype == torch.uint8
    assert sd["weight_global_scale"].shape == (1,) and sd["act_global_scale"].shape == (1,)
    assert sd["forward_hadamard_matrix"].shape == (64, 64) and sd["backward_hadamard_matrix"].shape == (64, 64)
    assert sd["weight"].shape == (96, 256) and sd["dqweight"].shape == (96, 256) and sd["bias"].shape == (96,)


def test_pre_forward_refuses_cpu_weights():
    cfg = FPQuantConfig(forward_dtype=FPQuantDtype.MXFP4, forward_method="abs_max",
                        backward_dtype=FPQuantDtype.BF16, hadamard_group_size=32)
    lin = FPQuantLinear(64, 32, cfg, bias=False, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        lin.pre_forward()
    bad = FPQuantLinear(48, 32, FPQuantConfig(forward_method="abs_max", backward_dtype=FPQuantDtype.BF16), bias=False)
    with pytest.raises(AssertionError):
        bad.pre_forward()  # 48 % 32 != 0


def test_operators_refuse_cpu_tensors():
    from fp_quant.module import hip_ops
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    h = torch.eye(32, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        hip_ops.fused_quantize_mx_op(x, h, "abs_max", False)


def test_fake_impls_give_reference_shapes():
    from fp_quant.module import hip_ops
    x = torch.empty(130, 4096, dtype=torch.bfloat16, device="meta")
    h = torch.empty(128, 128, dtype=torch.bfloat16, device="meta")
    q, s, m = torch.ops.fp_quant.fused_quantize_mx_op(x, h, "abs_max", False)
    assert q.shape == (130, 2048) and s.shape == (256, 128) and s.dtype == torch.float8_e8m0fnu and m is None
    gs = torch.empty(1, dtype=torch.float32, device="meta")
    q, s = torch.ops.fp_quant.fused_quantize_nv_op(x, h, gs)
    assert q.shape == (130, 2048) and s.shape == (256, 256) and s.dtype == torch.float8_e4m3fn
    w = torch.empty(512, 2048, dtype=torch.uint8, device="meta")
    a = torch.empty(1, dtype=torch.float32, device="meta")
    y = torch.ops.fp_quant.matmul_mxf4_bf16_tn_op(q, w, s, s, a)
    assert y.shape == (130, 512) and y.dtype == torch.bfloat16
    assert torch.ops.fp_quant.matmul_nvf4_bf16_tn_op(q, w, s, s, a).shape == (130, 512)
    assert torch.ops.fp_quant.matmul_ada_mxf4_bf16_tn_op(q, w, s, s, a).shape == (130, 512)


def test_replace_with_meta_init_and_skip_rule():
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(64, 64, bias=False)
            self.mlp = nn.Sequential(nn.Linear(64, 128), nn.Linear(128, 64))

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Block(), Block()])
            self.lm_head = nn.Linear(64, 32, bias=False)

    cfg = FPQuantConfig(forward_method="abs_max", backward_dtype=FPQuantDtype.BF16,
                        modules_to_not_convert=["lm_head", "layers.1.mlp.0"])
    model, replaced = fp_quant.replace_with_fp_quant_linear(Model(), cfg)
    assert replaced
    assert isinstance(model.layers[0].q_proj, FPQuantLinear) and isinstance(model.layers[0].mlp[0], FPQuantLinear)
    assert type(model.layers[1].mlp[0]) is nn.Linear and type(model.lm_head) is nn.Linear
    fl = model.layers[0].mlp[0]
    assert fl.qweight.device.type == "meta" and fl.bias is not None and fl.source_cls is nn.Linear
    assert all(not p.requires_grad for p in fl.parameters())
    model2, replaced2 = fp_quant.replace_with_fp_quant_linear(nn.Sequential(nn.ReLU()), cfg)
    assert not replaced2


def test_config_dict_round_trip_and_scale_groups():
    import fp_quant
    D = fp_quant.FPQuantDtype
    assert D.MXFP4.scale_group == 32 and D.NVFP4.scale_group == 16 and D.BF16.scale_group == 0
    # the entry the reference writes for an exported checkpoint (src/quantization/qconfig.py:9-18)
    entry = {"forward_dtype": "nvfp4", "backward_dtype": "bf16", "forward_method": "abs_max",
             "hadamard_group_size": 16, "modules_to_not_convert": ["lm_head"], "quant_method": "fp_quant",
             "store_master_weights": False, "pseudoquantization": False}
    cfg = fp_quant.FPQuantConfig.from_dict(entry)
    assert cfg.forward_dtype is D.NVFP4 and cfg.backward_dtype is D.BF16 and cfg.hadamard_group_size == 16
    assert cfg.transform_init == "hadamard" and cfg.modules_to_not_convert == ["lm_head"]
    back = cfg.to_dict()
    assert {k: back[k] for k in entry} == entry and back["transform_init"] == "hadamard"
    # enum members pass through, unknown keys are dropped, defaults stay defaults
    cfg2 = fp_quant.FPQuantConfig.from_dict({"forward_dtype": D.MXFP4, "something_else": 1})
    assert cfg2 == fp_quant.FPQuantConfig()
    from fp_quant.utils import export
    assert "transform_init" not in export.quantization_config_dict(cfg)
    cfg.transform_init = "gsr"
    assert export.quantization_config_dict(cfg)["transform_init"] == "gsr"


def test_everything_fails_loudly_without_the_library():
    """No other backend exists: with the shared library missing, the loader, the module constructor
    (the reference raises there when QuTLASS is absent, linear.py:57-60) and the qutlass stand-in all
    raise instead of computing something else."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r"""
import sys
sys.path.insert(0, sys.argv[1])
import torch, fp_quant, qutlass
from fp_quant import _engine
assert not _engine.available()
for what in ("loader", "module", "standin"):
    try:
        if what == "loader":
            _engine.lib()
        elif what == "module":
            fp_quant.FPQuantLinear(64, 32, fp_quant.FPQuantConfig(forward_method="abs_max",
                                   backward_dtype=fp_quant.FPQuantDtype.BF16), device="meta")
        else:
            qutlass._engine.lib()
    except Exception as exc:
        print(what, type(exc).__name__)
    else:
        print(what, "NO ERROR")
"""
    env = dict(os.environ, FPQ_LIBRARY_PATH="/nonexistent/libfpq_hip.so")
    r = subprocess.run([sys.executable, "-c", code, os.path.join(root, "fp-quant_amd")], capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = dict(l.split(" ", 1) for l in r.stdout.strip().splitlines())
    assert lines == {"loader": "FPQEngineError", "module": "ValueError", "standin": "FPQEngineError"}, r.stdout
