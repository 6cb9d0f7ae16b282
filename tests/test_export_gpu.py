"""Round-to-nearest exporter on the GPU: the rotated absolute maximum against the oracle's rotation,
exported tensors against the oracle's quantizers, and a saved checkpoint loaded back through the
loader path (meta-device FPQuantLinear + load_state_dict)."""
import json
import os

import pytest
import torch
from torch import nn

from oracle import fpq_oracle as O
from tests import capi
from tests.conftest import make_outlier_normal, make_student_t

pytestmark = pytest.mark.gpu

ROTS = {"hadamard": O.ROT_HADAMARD, "identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR}


def _cfg(fmt, g, **kw):
    import fp_quant
    return fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype(fmt), forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=g, **kw)


@pytest.mark.parametrize("rot,g", [("hadamard", 16), ("hadamard", 32), ("hadamard", 64), ("hadamard", 128),
                                   ("gsr", 32), ("gsr", 128), ("identity", 16)])
@pytest.mark.parametrize("rows,cols", [(1, 128), (37, 384), (300, 1024)])
def test_rotated_absmax_bit_exact(rot, g, rows, cols):
    x = make_student_t(rows, cols, seed=rows + g)
    norm = float(O.hadamard_matrix(g)[0, 0])
    want = float(O.rotate(x, ROTS[rot], g, norm).abs().max())
    assert capi.rotated_absmax(x, rot, g, norm) == want
    # running maximum: a larger preset value survives, a smaller one is replaced
    assert capi.rotated_absmax(x, rot, g, norm, start=want * 2) == want * 2
    assert capi.rotated_absmax(x, rot, g, norm, start=want / 2) == want


def test_rotated_absmax_general_matrix_and_edges():
    gen = torch.Generator().manual_seed(5)
    g = 32
    h = torch.linalg.qr(torch.randn(g, g, generator=gen))[0].to(torch.bfloat16)
    x = make_outlier_normal(65, 256, seed=2)
    want = float(O.rotate(x, O.ROT_GENERAL, g, 0.0, h).abs().max())
    assert capi.rotated_absmax(x, "general", g, 0.0, h) == want
    # all zeros leave the preset value; a large tensor exercises the grid-stride loop
    assert capi.rotated_absmax(torch.zeros(8, 128, dtype=torch.bfloat16), "hadamard", 128) == 0.0
    big = make_outlier_normal(4096, 4096, seed=9)
    want = float(O.rotate(big, O.ROT_HADAMARD, 128, float(O.hadamard_matrix(128)[0, 0])).abs().max())
    assert capi.rotated_absmax(big, "hadamard", 128) == want
    # the operator wrapper folds several tensors into one maximum
    from fp_quant.module import hip_ops
    hm = O.hadamard_matrix(128).cuda()
    amax = hip_ops.rotated_absmax(x.cuda(), hm)
    amax = hip_ops.rotated_absmax(big.cuda(), hm, amax)
    small = float(O.rotate(x, O.ROT_HADAMARD, 128, float(hm[0, 0])).abs().max())
    assert float(amax) == max(want, small)


@pytest.mark.parametrize("g,init", [(32, "hadamard"), (128, "hadamard"), (64, "gsr")])
def test_export_linear_mxfp4_matches_oracle(g, init):
    from fp_quant.utils import export
    n, k = 200, 512
    w = make_outlier_normal(n, k, seed=g) * 0.02
    out = export.export_linear(w.cuda(), _cfg("mxfp4", g, transform_init=init))
    kind = O.ROT_HADAMARD if init == "hadamard" else O.ROT_GSR
    wq, ws, _ = O.quantize_mx(w, kind, g, float(O.hadamard_matrix(g)[0, 0]))
    assert out["qweight"].dtype == torch.uint8 and torch.equal(out["qweight"].cpu(), wq)
    assert out["scales"].dtype == torch.uint8 and out["scales"].shape == (n, k // 32)
    assert torch.equal(out["scales"].cpu(), ws)
    hm = O.hadamard_matrix(g) if init == "hadamard" else O.gsr_matrix(g)
    assert torch.equal(out["forward_hadamard_matrix"].cpu(), hm)
    assert torch.equal(out["backward_hadamard_matrix"].cpu(), hm)
    for key in ("weight_global_scale", "act_global_scale"):   # quantizer.py:64-66
        assert out[key].dtype == torch.float32 and out[key].tolist() == [3.0]


@pytest.mark.parametrize("g", [16, 64])
def test_export_linear_nvfp4_tracks_the_global_scale(g):
    from fp_quant.utils import export
    n, k = 136, 384
    w = make_student_t(n, k, seed=g) * 0.05
    norm = float(O.hadamard_matrix(g)[0, 0])
    gs = O.nv_tracked_global_scale(O.rotate(w, O.ROT_HADAMARD, g, norm))
    ags = torch.tensor([77.5])
    out = export.export_linear(w.cuda(), _cfg("nvfp4", g), act_global_scale=ags)
    assert out["weight_global_scale"].dtype == torch.float32 and float(out["weight_global_scale"]) == gs
    assert float(out["act_global_scale"]) == 77.5
    wq, ws, _ = O.quantize_nv(w, gs, O.ROT_HADAMARD, g, norm)
    assert torch.equal(out["qweight"].cpu(), wq) and torch.equal(out["scales"].cpu(), ws)
    # a given (fused) weight scale is used as is
    out2 = export.export_linear(w.cuda(), _cfg("nvfp4", g), weight_global_scale=torch.tensor([gs / 2]),
                                act_global_scale=ags)
    wq2, ws2, _ = O.quantize_nv(w, gs / 2, O.ROT_HADAMARD, g, norm)
    assert torch.equal(out2["qweight"].cpu(), wq2) and torch.equal(out2["scales"].cpu(), ws2)
    with pytest.raises(ValueError):
        export.export_linear(w.cuda(), _cfg("nvfp4", g))


class _Attn(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.q_proj = nn.Linear(d, d, bias=False)
        self.k_proj = nn.Linear(d, d // 2, bias=False)
        self.v_proj = nn.Linear(d, d // 2, bias=True)
        self.o_proj = nn.Linear(d, d, bias=False)

    def forward(self, x):
        return self.o_proj(self.q_proj(x) + torch.cat([self.k_proj(x), self.v_proj(x)], dim=-1))


class _Mlp(nn.Module):
    def __init__(self, d, i):
        super().__init__()
        self.gate_proj = nn.Linear(d, i, bias=False)
        self.up_proj = nn.Linear(d, i, bias=False)
        self.down_proj = nn.Linear(i, d, bias=False)

    def forward(self, x):
        return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class _Block(nn.Module):
    def __init__(self, d, i):
        super().__init__()
        self.norm = nn.LayerNorm(d)
        self.self_attn = _Attn(d)
        self.mlp = _Mlp(d, i)

    def forward(self, x):
        x = x + self.self_attn(self.norm(x))
        return x + self.mlp(x)


class _Tiny(nn.Module):
    def __init__(self, d=256, i=512, layers=2, vocab=64):
        super().__init__()
        self.embed = nn.Embedding(vocab, d)
        self.layers = nn.ModuleList(_Block(d, i) for _ in range(layers))
        self.lm_head = nn.Linear(d, vocab, bias=False)

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.layers:
            x = layer(x)
        return self.lm_head(x)


def _tiny(seed=0):
    torch.manual_seed(seed)
    return _Tiny().to(torch.bfloat16)


@pytest.mark.parametrize("fmt,g", [("mxfp4", 32), ("nvfp4", 16)])
def test_exported_checkpoint_loads_and_runs(fmt, g, tmp_path):
    """export -> save -> meta-device replacement -> load_state_dict gives the model that quantizing
    in place gives (same buffers bit for bit; same logits when the global scales agree)."""
    import fp_quant
    from safetensors.torch import load_file
    from fp_quant.utils import export
    cfg = _cfg(fmt, g)
    model = _tiny().cuda()
    ids = torch.randint(0, 64, (2, 24), generator=torch.Generator().manual_seed(1)).cuda()
    act = None
    if fmt == "nvfp4":
        with export.ActivationScaleTracker(model, cfg) as tracker:
            model(ids)
            model(ids.flip(1))
        act = tracker.global_scales()
        assert sorted(act) == sorted(n for n, m in model.named_modules()
                                     if isinstance(m, nn.Linear) and n != "lm_head")
        # one layer by hand: the inputs of q_proj over both calibration batches
        xs = []
        hook = model.layers[0].self_attn.q_proj.register_forward_pre_hook(lambda m, a: xs.append(a[0].detach().cpu()))
        model(ids), model(ids.flip(1))
        hook.remove()
        norm = float(O.hadamard_matrix(g)[0, 0])
        amax = max(float(O.rotate(x.reshape(-1, x.shape[-1]), O.ROT_HADAMARD, g, norm).abs().max()) for x in xs)
        want = O.nv_tracked_global_scale(torch.tensor([[amax]]))
        assert float(act["layers.0.self_attn.q_proj"]) == want
    state = export.rtn_export(model, cfg, act_global_scales=act, fuse_global_scale=(fmt == "nvfp4"))
    assert "lm_head.weight" in state and "layers.0.self_attn.q_proj.weight" not in state
    assert "layers.0.self_attn.v_proj.bias" in state and "embed.weight" in state
    assert all(not v.is_cuda for v in state.values())
    if fmt == "nvfp4":
        # rtn.py:131-147: q/k/v and gate/up share the smallest tracked weight scale
        norm = float(O.hadamard_matrix(g)[0, 0])
        attn = model.layers[1].self_attn
        each = [O.nv_tracked_global_scale(O.rotate(m.weight.detach().cpu(), O.ROT_HADAMARD, g, norm))
                for m in (attn.q_proj, attn.k_proj, attn.v_proj)]
        for p in "qkv":
            assert float(state[f"layers.1.self_attn.{p}_proj.weight_global_scale"]) == min(each)
        own = O.nv_tracked_global_scale(O.rotate(attn.o_proj.weight.detach().cpu(), O.ROT_HADAMARD, g, norm))
        assert float(state["layers.1.self_attn.o_proj.weight_global_scale"]) == own
        wq, ws, _ = O.quantize_nv(attn.k_proj.weight.detach().cpu(), min(each), O.ROT_HADAMARD, g, norm)
        assert torch.equal(state["layers.1.self_attn.k_proj.qweight"], wq)
        assert torch.equal(state["layers.1.self_attn.k_proj.scales"], ws)

    class _HfConfig:   # stand-in with the two members the writer uses
        def save_pretrained(self, path):
            json.dump({"quantization_config": self.quantization_config}, open(os.path.join(path, "config.json"), "w"))

    export.save_realquant_checkpoint(state, str(tmp_path), cfg, _HfConfig(), max_shard_size=300_000)
    saved_cfg = json.load(open(os.path.join(tmp_path, "config.json")))["quantization_config"]
    assert saved_cfg["quant_method"] == "fp_quant" and saved_cfg["forward_dtype"] == fmt
    index = json.load(open(os.path.join(tmp_path, "model.safetensors.index.json")))["weight_map"]
    assert len(set(index.values())) > 1
    loaded = {}
    for shard in sorted(set(index.values())):
        loaded.update(load_file(os.path.join(tmp_path, shard)))

    # the loader path: empty FPQuantLinear modules, filled from the checkpoint.  Loaders build the model
    # under the checkpoint's dtype, which the new modules' buffers take (alpha is evaluated in it).
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("meta"):
            fresh = _Tiny()
        fresh, replaced = fp_quant.replace_with_fp_quant_linear(fresh, cfg)
    finally:
        torch.set_default_dtype(prev)
    assert replaced
    for module in fresh.modules():
        if isinstance(module, fp_quant.FPQuantLinear):
            module.weight = None
            module.dqweight = None
    fresh = fresh.to_empty(device="cuda")
    missing, unexpected = fresh.load_state_dict(loaded, strict=False)
    assert not unexpected and not missing
    got = fresh(ids)

    if fmt == "mxfp4":
        # quantizing in place gives the same buffers and therefore the same logits
        inplace = fp_quant.replace_quantize_with_fp_quant_linear(_tiny().cuda(), cfg)
        for (na, a), (nb, b) in zip(sorted(inplace.state_dict().items()), sorted(fresh.state_dict().items())):
            assert na == nb and a.dtype == b.dtype and torch.equal(a.cpu(), b.cpu()), na
        assert torch.equal(got, inplace(ids))
    else:
        # NVFP4: tracked scales differ from pre_forward's fixed 3.0, so compare with the float model
        with torch.no_grad():
            want = model(ids).float()
        err = (got.detach().float() - want).norm() / want.norm()
        assert float(err) < 0.2, float(err)
