"""The `qutlass` stand-in (fp-quant_amd/qutlass): the names FP-Quant imports from QuTLASS, implemented on
the C ABI, and the Hugging Face loading route that is gated on that package being present."""
import pytest
import torch

from oracle import fpq_oracle as O

# the names of `from qutlass import (...)` and `from qutlass.utils import to_blocked`
# (inference_lib/src/fp_quant/module/qutlass_ops.py:5-23)
REFERENCE_IMPORTS = [
    "fusedQuantizeMx", "fusedQuantizeNv", "matmul_ada_mxf4_bf16_tn", "matmul_mxf4_bf16_tn", "matmul_nvf4_bf16_tn",
    "matmul_mxf8_bf16_tn", "matmul_mxf8_bf16_nn", "backward_t_bf16", "backward_qt_bf16",
    "backward_bf16_square_double_mxfp8", "mxfp4_transpose_mxfp8",
]


def test_names_versions_and_availability_checks():
    import fp_quant
    import qutlass
    import qutlass.utils
    from packaging import version
    for name in REFERENCE_IMPORTS:
        assert callable(getattr(qutlass, name)), name
    assert version.parse(qutlass.__version__) >= version.parse("0.2.0")
    assert version.parse(fp_quant.__version__) >= version.parse("0.3.2")
    t = torch.arange(12, dtype=torch.uint8).view(3, 4)
    assert qutlass.utils.to_blocked(t, use_triton_kernel=True) is t
    with pytest.raises(NotImplementedError):
        qutlass.backward_t_bf16(t)
    with pytest.raises(ValueError):                      # no CPU path
        qutlass.fusedQuantizeMx(torch.zeros(2, 64, dtype=torch.bfloat16), torch.eye(32, dtype=torch.bfloat16))
    from transformers.utils import import_utils
    assert import_utils.is_qutlass_available() and import_utils.is_fp_quant_available()


@pytest.mark.gpu
@pytest.mark.parametrize("m", [3, 70])
def test_entry_points_equal_the_operators(m):
    """Same bits as the fp_quant::* operators, through the call sequences of qutlass_ops.py."""
    import qutlass
    from qutlass.utils import to_blocked
    from fp_quant.module import hip_ops
    gen = torch.Generator().manual_seed(m)
    x = (torch.randn(m, 512, generator=gen) * 2).to(torch.bfloat16).cuda()
    w = (torch.randn(96, 512, generator=gen) * 0.05).to(torch.bfloat16).cuda()
    alpha = torch.tensor([0.111328125], dtype=torch.float32, device="cuda")
    h = O.hadamard_matrix(128).cuda()
    xq, xs = qutlass.fusedQuantizeMx(x, h, method="abs_max", return_mask=False)
    oq, os_, _ = hip_ops.fused_quantize_mx_op(x, h, "abs_max", False)
    assert xs.dtype == torch.float8_e8m0fnu and xs.shape == os_.shape
    assert torch.equal(xq, oq) and torch.equal(xs.view(torch.uint8), os_.view(torch.uint8))
    wq, ws = qutlass.fusedQuantizeMx(w, h)
    y = qutlass.matmul_mxf4_bf16_tn(xq, wq, to_blocked(xs, use_triton_kernel=True),
                                    to_blocked(ws, use_triton_kernel=True).view(torch.float8_e8m0fnu), alpha)
    assert torch.equal(y, hip_ops.matmul_mxf4_bf16_tn_op(xq, wq, xs, ws, alpha))
    assert torch.equal(qutlass.matmul_ada_mxf4_bf16_tn(xq, wq, xs, ws.view(torch.float8_e8m0fnu), alpha), y)
    q3 = qutlass.fusedQuantizeMx(x, h, method="quest", return_mask=True)
    o3 = hip_ops.fused_quantize_mx_op(x, h, "quest", True)
    assert len(q3) == 3 and all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(q3, o3))

    h16 = O.hadamard_matrix(16).cuda()
    gs = torch.tensor([7.5], dtype=torch.float32, device="cuda")
    nq, ns = qutlass.fusedQuantizeNv(x, h16, gs)
    oq, os_ = hip_ops.fused_quantize_nv_op(x, h16, gs)
    assert ns.dtype == torch.float8_e4m3fn and torch.equal(nq, oq) and torch.equal(ns.view(torch.uint8), os_.view(torch.uint8))
    wq, ws = qutlass.fusedQuantizeNv(w, h16, gs)
    y = qutlass.matmul_nvf4_bf16_tn(nq, wq, to_blocked(ns), to_blocked(ws.view(torch.float8_e4m3fn)), alpha)
    assert torch.equal(y, hip_ops.matmul_nvf4_bf16_tn_op(nq, wq, ns, ws, alpha))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_transformers_loads_and_quantizes_through_its_own_fp_quant_route(tmp_path, fmt, g):
    """transformers' FP-Quant quantizer (quantizers/quantizer_fp_quant.py, integrations/fp_quant.py) with this
    package answering to `fp_quant` and `qutlass`: (1) a bf16 checkpoint quantized while loading,
    (2) the realquant checkpoint exported from it loaded as is.  Both give the logits of
    replace_quantize_with_fp_quant_linear on the same weights."""
    import fp_quant
    import transformers
    from transformers import AutoModelForCausalLM, LlamaConfig, LlamaForCausalLM
    from fp_quant.utils import export
    torch.manual_seed(3)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=128, max_position_embeddings=128)
    dense = LlamaForCausalLM(cfg).to(torch.bfloat16)
    dense_dir = str(tmp_path / "dense")
    dense.save_pretrained(dense_dir)
    ids = torch.randint(0, 128, (2, 40), generator=torch.Generator().manual_seed(1)).cuda()

    qcfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype(fmt), forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=g)
    mine = fp_quant.replace_quantize_with_fp_quant_linear(
        LlamaForCausalLM.from_pretrained(dense_dir, dtype=torch.bfloat16).cuda().eval(), qcfg)
    with torch.no_grad():
        want = mine(ids).logits

    hf_cfg = transformers.FPQuantConfig(forward_dtype=fmt, forward_method="abs_max", backward_dtype="bf16",
                                        hadamard_group_size=g)
    loaded = AutoModelForCausalLM.from_pretrained(dense_dir, quantization_config=hf_cfg, device_map="cuda",
                                                  dtype=torch.bfloat16).eval()
    assert sum(isinstance(m, fp_quant.FPQuantLinear) for m in loaded.modules()) == 14
    with torch.no_grad():
        assert torch.equal(loaded(ids).logits, want)

    # the exported realquant checkpoint (weights as qweight / scales, quantization_config in config.json)
    real_dir = str(tmp_path / "realquant")
    state = {k: v.detach().cpu() for k, v in mine.state_dict().items()}
    export.save_realquant_checkpoint(state, real_dir, qcfg, dense.config)
    again = AutoModelForCausalLM.from_pretrained(real_dir, device_map="cuda", dtype=torch.bfloat16).eval()
    assert sum(isinstance(m, fp_quant.FPQuantLinear) for m in again.modules()) == 14
    with torch.no_grad():
        assert torch.equal(again(ids).logits, want)
