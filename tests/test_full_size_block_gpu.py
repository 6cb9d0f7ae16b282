"""One decoder layer at the sizes of the end-to-end benchmark configuration (Llama-3.1-8B: hidden 4096, 32 query / 8 key-value
heads, intermediate 14336) on 4 x 2048 = 8192 tokens, every linear an MXFP4 FPQuantLinear with Hadamard 128.
Drives the kernels FPQuantLinear dispatches at prefill size (packed quantizer, 256 x 128 tile GEMM, fused
producers, residual epilogues) through the module surface."""
import pytest
import torch

from oracle import fpq_oracle as O
from tests.conftest import row_major_weights

pytestmark = pytest.mark.gpu

HIDDEN, INTER, TOKENS = 4096, 14336, 8192


def _block(seed=0):
    import fp_quant
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer, LlamaRotaryEmbedding
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=HIDDEN, intermediate_size=INTER, num_hidden_layers=1, num_attention_heads=32,
                      num_key_value_heads=8, vocab_size=128, max_position_embeddings=4096, rms_norm_eps=1e-5,
                      rope_theta=500000.0, attn_implementation="sdpa")
    holder = torch.nn.Module()
    holder.self_attn_holder = None
    layer = LlamaDecoderLayer(cfg, 0).to(device="cuda", dtype=torch.bfloat16).eval()
    for p in layer.parameters():
        if p.dim() == 1:
            p.data.add_(0.1 * torch.randn_like(p))
    wrapper = torch.nn.ModuleDict({"layers": torch.nn.ModuleList([layer])})
    qcfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=128)
    fp_quant.replace_quantize_with_fp_quant_linear(wrapper, qcfg)
    rope = LlamaRotaryEmbedding(config=cfg).to("cuda")
    return wrapper, layer, rope


def _run(layer, rope, x):
    b, s, _ = x.shape
    pos = torch.arange(s, device="cuda").unsqueeze(0).expand(b, -1)
    cos_sin = rope(x, pos)
    out = layer(x, position_embeddings=cos_sin, position_ids=pos, attention_mask=None)
    return out[0] if isinstance(out, tuple) else out


def _check_linear(lin, x2d, rows=24, cols=160, seed=0):
    """Output of one FPQuantLinear on [tokens, K] against the oracle on a seeded sample of rows and columns."""
    y = lin(x2d)
    gen = torch.Generator().manual_seed(seed)
    ri = torch.randperm(x2d.shape[0], generator=gen)[:rows].sort().values
    ci = torch.randperm(lin.out_features, generator=gen)[:cols].sort().values
    wq, ws = row_major_weights(lin)      # (never index `lin.qweight` by output feature: a layer may hold 1-D packed buffers)
    xq, xs, _ = O.quantize_mx(x2d[ri.cuda()].cpu(), O.ROT_HADAMARD, 128)
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    ref, mag = O.gemm_ref(xq, xs, wq[ci], ws[ci], alpha, "mxfp4")
    got = y[ri.cuda()][:, ci.cuda()].cpu()
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
    assert ((got.double() - ref).abs() <= tol).all()
    assert (got == ref.to(torch.bfloat16)).float().mean() > 0.98
    return y


def test_every_linear_of_a_full_size_block_matches_the_oracle():
    _, layer, _ = _block()
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(TOKENS, HIDDEN, generator=gen).to(torch.bfloat16).cuda()
    h = (torch.randn(TOKENS, INTER, generator=gen) * 0.5).to(torch.bfloat16).cuda()
    with torch.no_grad():
        for i, name in enumerate(("q_proj", "k_proj", "v_proj", "o_proj")):
            _check_linear(getattr(layer.self_attn, name), x, seed=i)
        _check_linear(layer.mlp.gate_proj, x, seed=10)
        _check_linear(layer.mlp.up_proj, x, seed=11)
        _check_linear(layer.mlp.down_proj, h, seed=12)


def test_full_size_block_fused_against_unfused():
    from fp_quant.utils import fuse
    wrapper, layer, rope = _block(seed=1)
    gen = torch.Generator().manual_seed(6)
    x = torch.randn(4, 2048, HIDDEN, generator=gen).to(torch.bfloat16).cuda()
    with torch.no_grad():
        want = _run(layer, rope, x)
        # producers fused into the quantizers: this library's RMSNorm / SiLU arithmetic against PyTorch's,
        # a few bf16 flips per million inputs, each of which can move a 4-bit code
        assert fuse.fuse_rmsnorm(layer.input_layernorm, layer.self_attn.q_proj)
        assert fuse.fuse_rmsnorm(layer.post_attention_layernorm, layer.mlp.gate_proj)
        assert fuse.fuse_gated_mlp(layer.mlp)
        got = _run(layer, rope, x)
        err = (got.float() - want.float()).norm() / want.float().norm()
        assert float(err) < 0.02, float(err)     # same bound as the whole-model test on the small model
        # the residual additions inside the o_proj / down_proj GEMMs change no bit
        assert fuse.fuse_residual_adds(layer)
        with_adds = _run(layer, rope, x)
        assert torch.equal(with_adds, got)
        fuse.unfuse_producers(wrapper)
        assert torch.equal(_run(layer, rope, x), want)
