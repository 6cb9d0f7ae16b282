"""Quantizers fused with the producer of their input (RMSNorm, SiLU*up): codes, scales and the
optional bf16 by-product must be bit-identical to the oracle's producer followed by its quantizer."""
import pytest
import torch

from oracle import fpq_oracle as O
from tests import capi
from tests.conftest import make_outlier_normal, make_student_t, needs_packed, packed_copy

pytestmark = pytest.mark.gpu


def _oracle_quantize(v_bf16, fmt, rot, g, gs):
    kind = O.ROT_HADAMARD if rot == "hadamard" else O.ROT_IDENTITY
    norm = float(O.hadamard_matrix(g)[0, 0])
    if fmt == "mxfp4":
        q, s, _ = O.quantize_mx(v_bf16, kind, g, norm)
    else:
        q, s, _ = O.quantize_nv(v_bf16, gs, kind, g, norm)
    return q, s


@pytest.mark.parametrize("rows,cols,ld", [(1, 128, None), (37, 384, 512), (300, 4096, None)])
def test_row_inv_rms_bit_exact(rows, cols, ld):
    x = make_student_t(rows, cols, seed=rows)
    x[0, :8] = 0
    got = capi.row_inv_rms(x, 1e-5, ld)
    assert torch.equal(got, O.row_inv_rms(x, 1e-5))
    z = torch.zeros(3, cols, dtype=torch.bfloat16)
    assert torch.equal(capi.row_inv_rms(z, 1e-6), O.row_inv_rms(z, 1e-6))


CASES = [("mxfp4", "hadamard", 32), ("mxfp4", "hadamard", 128), ("mxfp4", "identity", 32),
         ("nvfp4", "hadamard", 16), ("nvfp4", "hadamard", 64), ("nvfp4", "identity", 16)]


@pytest.mark.parametrize("fmt,rot,g", CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (45, 384), (260, 1024)])
def test_rmsnorm_quantize_bit_exact(fmt, rot, g, rows, cols):
    x = make_outlier_normal(rows, cols, seed=rows + g) * 1.7
    gen = torch.Generator().manual_seed(cols)
    w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
    eps = 1e-5
    want_v = O.rmsnorm(x, w, eps)
    gs = 1234.5 if fmt == "nvfp4" else None
    wq, ws = _oracle_quantize(want_v, fmt, rot, g, gs)
    codes, scales, out = capi.fused_quantize("rmsnorm", fmt, x, w, g=g, rot=rot, global_scale=gs, eps=eps,
                                             ld_a=cols + 64 if rows == 45 else None)
    assert torch.equal(out, want_v)
    assert torch.equal(codes, wq) and torch.equal(scales, ws)
    # without the by-product
    codes2, scales2, none = capi.fused_quantize("rmsnorm", fmt, x, w, g=g, rot=rot, global_scale=gs, eps=eps,
                                                want_out=False)
    assert none is None and torch.equal(codes2, wq) and torch.equal(scales2, ws)


@pytest.mark.parametrize("fmt,rot,g", CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (45, 384), (260, 1024)])
def test_silu_mul_quantize_bit_exact(fmt, rot, g, rows, cols):
    gate = make_student_t(rows, cols, seed=rows + g) * 2
    up = make_outlier_normal(rows, cols, seed=cols + g)
    # extremes of the activation: saturated both ways, zeros, the last finite binade of exp
    gate[0, :8] = torch.tensor([-300.0, 300.0, 0.0, -0.0, -88.5, 88.5, -20.0, 20.0]).to(torch.bfloat16)
    want_v = O.silu_mul(gate, up)
    gs = 777.0 if fmt == "nvfp4" else None
    wq, ws = _oracle_quantize(want_v, fmt, rot, g, gs)
    # gate and up as the two halves of one [rows, 2 * cols] tensor (a fused gate/up projection)
    both = torch.cat((gate, up), dim=1).cuda()
    if rows == 45:
        lib_args = dict(ld_a=2 * cols, ld_b=cols + 8)
    else:
        lib_args = {}
    codes, scales, out = capi.fused_quantize("silu_mul", fmt, gate, up, g=g, rot=rot, global_scale=gs, **lib_args)
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))   # bit pattern: keeps -0 apart from +0
    assert torch.equal(codes, wq) and torch.equal(scales, ws)
    del both


PACKED_CASES = [("hadamard", 16), ("hadamard", 32), ("hadamard", 64), ("hadamard", 128), ("identity", 32)]


@pytest.mark.parametrize("rot,g", PACKED_CASES)
@pytest.mark.parametrize("kind", ["rmsnorm", "silu_mul"])
@pytest.mark.parametrize("rows,cols", [(1, 256), (20, 768), (70, 512), (300, 1024)])
def test_fused_quantize_packed_bit_exact(kind, rot, g, rows, cols):
    """The streaming kernel with a prologue: packed codes and scales (ragged last row tile, strided
    inputs, extreme exponents that take the slow path) and the bf16 by-product."""
    from tests.test_packed_gpu import pack_by_definition
    a = make_student_t(rows, cols, seed=rows + g) * 2
    if kind == "rmsnorm":
        gen = torch.Generator().manual_seed(cols)
        b = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
        if rows > 8:
            b[64:96] = 0.0                           # a zero group in every row
            a[5] *= 2.0 ** -60                       # (normalisation undoes the row's magnitude)
        want_v = O.rmsnorm(a, b, 1e-5)
    else:
        b = make_outlier_normal(rows, cols, seed=cols + g)
        a[0, :8] = torch.tensor([-300.0, 300.0, 0.0, -0.0, -88.5, 88.5, -20.0, 1e-30]).to(torch.bfloat16)
        if rows > 8:
            b[3, 64:96] = 0.0
            b[7] *= 2.0 ** -110                      # exponents outside the fast range
            b[9] *= 2.0 ** 100
        want_v = O.silu_mul(a, b)
    okind = O.ROT_HADAMARD if rot == "hadamard" else O.ROT_IDENTITY
    wc, ws, _ = O.quantize_mx(want_v, okind, g, float(O.hadamard_matrix(g)[0, 0]))
    want_c, want_s = pack_by_definition(wc, ws, cols)
    lds = dict(ld_a=cols + 64, ld_b=2 * cols) if rows in (20, 70) else {}
    pc, ps, out = capi.fused_quantize_packed(kind, a, b, g=g, rot=rot, **lds)
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)
    pc2, ps2, none = capi.fused_quantize_packed(kind, a, b, g=g, rot=rot, want_out=False)
    assert none is None and torch.equal(pc2, want_c) and torch.equal(ps2, want_s)


@pytest.mark.parametrize("rot,g", PACKED_CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (1, 4096), (5, 768), (33, 4096), (64, 1024), (20, 16384)])
def test_rmsnorm_rows_in_one_launch_bit_exact(rot, g, rows, cols):
    """fpq_rmsnorm_rows_quantize_mx_packed: the row statistic, the normalised bf16 tensor and the packed codes
    and scales of the oracle (and so of fpq_row_inv_rms + fpq_rmsnorm_quantize_mx_packed), zero padding rows,
    a strided input, both optional outputs absent."""
    from tests.test_packed_gpu import pack_by_definition
    x = make_student_t(rows, cols, seed=rows + g) * 2
    gen = torch.Generator().manual_seed(cols)
    w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
    if rows > 4:
        w[64:96] = 0.0
        x[3] *= 2.0 ** -60
        x[4] = 0.0                                    # an all-zero row: 1 / sqrt(eps)
    want_v = O.rmsnorm(x, w, 1e-5)
    okind = O.ROT_HADAMARD if rot == "hadamard" else O.ROT_IDENTITY
    wc, ws, _ = O.quantize_mx(want_v, okind, g, float(O.hadamard_matrix(g)[0, 0]))
    want_c, want_s = pack_by_definition(wc, ws, cols)
    ld = cols + 64 if rows in (5, 33) else None
    pc, ps, out, inv = capi.rmsnorm_rows_quantize_packed(x, w, g=g, rot=rot, ld=ld)
    assert torch.equal(inv, O.row_inv_rms(x, 1e-5))
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)
    pc2, ps2, none, none2 = capi.rmsnorm_rows_quantize_packed(x, w, g=g, rot=rot, want_out=False, want_inv=False)
    assert none is None and none2 is None and torch.equal(pc2, want_c) and torch.equal(ps2, want_s)


NV_PACKED_CASES = [("hadamard", 16), ("hadamard", 32), ("hadamard", 128), ("identity", 16)]


@pytest.mark.parametrize("rot,g", NV_PACKED_CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (1, 4096), (5, 768), (33, 4096), (64, 1024)])
def test_rmsnorm_rows_in_one_launch_nvfp4_bit_exact(rot, g, rows, cols):
    """fpq_rmsnorm_rows_quantize_nv_packed: as the MXFP4 entry, with E4M3 scales under a global scale."""
    from tests.test_packed_gpu import pack_nv_by_definition
    x = make_student_t(rows, cols, seed=rows + g) * 2
    gen = torch.Generator().manual_seed(cols)
    w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
    if rows > 4:
        w[64:96] = 0.0
        x[3] *= 2.0 ** -60
        x[4] = 0.0
    want_v = O.rmsnorm(x, w, 1e-5)
    wc, ws = _oracle_quantize(want_v, "nvfp4", rot, g, 777.0)
    want_c, want_s = pack_nv_by_definition(wc, ws, cols)
    ld = cols + 64 if rows in (5, 33) else None
    pc, ps, out, inv = capi.rmsnorm_rows_quantize_packed(x, w, g=g, rot=rot, ld=ld, global_scale=777.0)
    assert torch.equal(inv, O.row_inv_rms(x, 1e-5))
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)
    pc2, ps2, none, none2 = capi.rmsnorm_rows_quantize_packed(x, w, g=g, rot=rot, want_out=False, want_inv=False,
                                                              global_scale=777.0)
    assert none is None and none2 is None and torch.equal(pc2, want_c) and torch.equal(ps2, want_s)


@pytest.mark.parametrize("rot,g", NV_PACKED_CASES)
@pytest.mark.parametrize("kind", ["rmsnorm", "silu_mul"])
@pytest.mark.parametrize("rows,cols", [(1, 256), (20, 768), (64, 512), (70, 512), (300, 1024)])
def test_fused_quantize_packed_nvfp4_bit_exact(kind, rot, g, rows, cols):
    """The NVFP4 fused producers writing the packed layout (generic kernel up to 64 rows, streaming kernel
    beyond): codes, E4M3 scales and the bf16 by-product of the oracle."""
    from fp_quant import _engine
    from tests.test_packed_gpu import pack_nv_by_definition
    a = make_student_t(rows, cols, seed=rows + g) * 2
    if kind == "rmsnorm":
        gen = torch.Generator().manual_seed(cols)
        b = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
        if rows > 8:
            b[64:96] = 0.0
            a[5] *= 2.0 ** -60
        want_v = O.rmsnorm(a, b, 1e-5)
    else:
        b = make_outlier_normal(rows, cols, seed=cols + g)
        a[0, :8] = torch.tensor([-300.0, 300.0, 0.0, -0.0, -88.5, 88.5, -20.0, 1e-30]).to(torch.bfloat16)
        if rows > 8:
            b[3, 64:96] = 0.0
            b[7] *= 2.0 ** -110
            b[9] *= 2.0 ** 100
        want_v = O.silu_mul(a, b)
    wc, ws = _oracle_quantize(want_v, "nvfp4", rot, g, 777.0)
    want_c, want_s = pack_nv_by_definition(wc, ws, cols)
    lds = dict(ld_a=cols + 64, ld_b=2 * cols) if rows in (20, 70) else {}
    pc, ps, out = capi.fused_quantize_packed(kind, a, b, g=g, rot=rot, global_scale=777.0, **lds)
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)
    pc2, ps2, none = capi.fused_quantize_packed(kind, a, b, g=g, rot=rot, want_out=False, global_scale=777.0)
    assert none is None and torch.equal(pc2, want_c) and torch.equal(ps2, want_s)


@pytest.mark.parametrize("gs", [None, 777.0])
def test_rmsnorm_rows_in_one_launch_non_finite_rows_are_data(gs):
    """A row holding NaN (its 1 / rms is NaN) or infinity (1 / rms = 0) goes through the one-launch kernel as
    data, as the reference's RMSNorm propagates it: every byte equals what fpq_row_inv_rms followed by
    fpq_rmsnorm_quantize_*_packed writes, the NaN row's by-product is NaN, and the finite rows keep the
    oracle's bits."""
    rows, cols, g = 6, 1024, 128 if gs is None else 16
    x = make_student_t(rows, cols, seed=11) * 2
    x[1, 100] = float("nan")
    x[4, 7] = float("inf")
    gen = torch.Generator().manual_seed(cols)
    w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
    pc, ps, out, inv = capi.rmsnorm_rows_quantize_packed(x, w, g=g, global_scale=gs)
    pc2, ps2, out2 = capi.fused_quantize_packed("rmsnorm", x, w, g=g, global_scale=gs)
    assert torch.equal(pc, pc2) and torch.equal(ps, ps2)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    assert torch.isnan(inv[1]) and inv[4] == 0.0
    assert torch.isnan(out[1]).all() and torch.isnan(out[4, 7])
    finite = [0, 2, 3, 5]
    want_v = O.rmsnorm(x[finite], w, 1e-5)
    assert torch.equal(out[finite], want_v)
    assert torch.equal(inv[finite], O.row_inv_rms(x[finite], 1e-5))


def test_fused_quantize_packed_nvfp4_needs_a_global_scale():
    from fp_quant import _engine
    lib = _engine.lib()
    rows, cols = 4, 256
    x = torch.zeros(rows, cols, dtype=torch.bfloat16, device="cuda")
    pc = torch.zeros(lib.fpq_packed_codes_bytes(rows, cols), dtype=torch.uint8, device="cuda")
    ps = torch.zeros(lib.fpq_packed_scales_bytes_nv(rows, cols), dtype=torch.uint8, device="cuda")
    assert lib.fpq_silu_mul_quantize_nv_packed(x.data_ptr(), cols, x.data_ptr(), cols, rows, cols, 1, 16, 0.25, None,
                                               None, pc.data_ptr(), ps.data_ptr(), 0,
                                               torch.cuda.current_stream().cuda_stream) == -1


def test_rmsnorm_rows_limits():
    from fp_quant import _engine
    lib = _engine.lib()
    assert lib.fpq_rmsnorm_rows_max_rows() == 64
    x = torch.zeros(65, 256, dtype=torch.bfloat16, device="cuda")
    w = torch.ones(256, dtype=torch.bfloat16, device="cuda")
    pc = torch.zeros(96 * 128, dtype=torch.uint8, device="cuda")
    ps = torch.zeros(96 * 8, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (x.data_ptr(), 256, w.data_ptr())
    tail = (1e-5, 1, 32, 0.177, None, None, pc.data_ptr(), ps.data_ptr(), 0, st)
    assert lib.fpq_rmsnorm_rows_quantize_mx_packed(*args, 65, 256, *tail) == _engine.E_LIMIT
    assert lib.fpq_rmsnorm_rows_quantize_mx_packed(*args, 4, 200, *tail) == -2
    assert lib.fpq_rmsnorm_rows_quantize_mx_packed(*args, 4, 256, 1e-5, _engine.ROT_GSR, 32, 0.177, None, None,
                                                   pc.data_ptr(), ps.data_ptr(), 0, st) == _engine.E_UNSUPPORTED
    assert lib.fpq_rmsnorm_rows_quantize_mx_packed(*args, 0, 256, *tail) == 0


def test_fused_quantize_packed_full_size_matches_generic_kernel():
    """A down_proj-sized input: the streaming fused kernel equals the generic fused kernel re-tiled."""
    from tests.test_packed_gpu import pack_by_definition
    rows, cols = 512, 14336
    gate = make_student_t(rows, cols, seed=1) * 2
    up = make_outlier_normal(rows, cols, seed=2)
    codes, scales, _ = capi.fused_quantize("silu_mul", "mxfp4", gate, up, g=128, want_out=False)
    want_c, want_s = pack_by_definition(codes, scales, cols)
    pc, ps, _ = capi.fused_quantize_packed("silu_mul", gate, up, g=128, want_out=False)
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)


def test_fused_quantize_argument_checks():
    from fp_quant import _engine
    lib = _engine.lib()
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda")
    w = torch.ones(128, dtype=torch.bfloat16, device="cuda")
    inv = torch.ones(4, dtype=torch.float32, device="cuda")
    c = torch.zeros(4, 64, dtype=torch.uint8, device="cuda")
    s = torch.zeros(4, 4, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    ok = lib.fpq_rmsnorm_quantize_mx(x.data_ptr(), 128, inv.data_ptr(), w.data_ptr(), 4, 128, 0, 32, 0.177, None,
                                     c.data_ptr(), s.data_ptr(), 4, 4, 0, st)
    assert ok == 0
    # sequency-ordered and general rotations are not fused
    assert lib.fpq_rmsnorm_quantize_mx(x.data_ptr(), 128, inv.data_ptr(), w.data_ptr(), 4, 128, _engine.ROT_GSR, 32,
                                       0.177, None, c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == _engine.E_UNSUPPORTED
    # row stride smaller than the row, or not a multiple of 8
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 64, x.data_ptr(), 128, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -2
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 128, x.data_ptr(), 132, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -2
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 128, None, 128, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -1
    assert lib.fpq_row_inv_rms(x.data_ptr(), 128, 4, 100, 1e-5, inv.data_ptr(), st) == -2
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------
# Module level: fuse_producers on Llama-style blocks


def _cfg(fmt, g):
    import fp_quant
    return fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype(fmt), forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=g)


def _tiny_llama(fmt, g, seed=0):
    import fp_quant
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=128, max_position_embeddings=256, rms_norm_eps=1e-5)
    model = LlamaForCausalLM(cfg).to(device="cuda", dtype=torch.bfloat16).eval()
    for p in model.parameters():        # norm weights away from 1 so that the weight product matters
        if p.dim() == 1:
            p.data.add_(0.1 * torch.randn_like(p))
    return fp_quant.replace_quantize_with_fp_quant_linear(model, _cfg(fmt, g))


@pytest.mark.parametrize("fmt,g", [("mxfp4", 32), ("mxfp4", 128), ("nvfp4", 16)])
@pytest.mark.parametrize("tokens", [3, 40])
def test_fused_norm_and_mlp_match_the_oracle_composition(fmt, g, tokens):
    """A fused RMSNorm returns the oracle's bf16 tensor and its consumers give what they give when
    handed that tensor unfused; the fused MLP equals down_proj on the oracle's silu*up."""
    from fp_quant.module import eager, hip_ops
    from fp_quant.utils import fuse_producers, unfuse_producers
    model = _tiny_llama(fmt, g)
    block = model.model.layers[1]
    x = (torch.randn(2, tokens, 256, device="cuda") * 1.5).to(torch.bfloat16)
    with torch.no_grad():
        want_y = O.rmsnorm(x.cpu().view(-1, 256), block.input_layernorm.weight.cpu(), 1e-5).view(x.shape).cuda()
        want_q = block.self_attn.q_proj(want_y)
        want_k = block.self_attn.k_proj(want_y.clone())
        gate, up = block.mlp.gate_proj(x), block.mlp.up_proj(x)
        h = O.silu_mul(gate.cpu().view(-1, 512), up.cpu().view(-1, 512)).view(gate.shape).cuda()
        want_mlp = block.mlp.down_proj(h)

        assert fuse_producers(model) == 10                    # two norms, the MLP, the additions, q/k/v per block
        assert sorted(model.state_dict()) == sorted(_tiny_llama(fmt, g).state_dict())
        eager._shared_activations.clear()
        y = block.input_layernorm(x)
        assert torch.equal(y, want_y)
        slot = eager._shared_activations[0]
        assert slot.ref() is y and slot.serves(True)
        assert torch.equal(block.self_attn.q_proj(y), want_q)
        assert torch.equal(block.self_attn.k_proj(y), want_k)
        assert eager._shared_activations[0] is slot         # both projections used the norm's quantization
        assert torch.equal(block.mlp(x), want_mlp)

        # a consumer that does not match (other tensor) still computes its own quantization
        assert torch.equal(block.self_attn.q_proj(want_y.clone()), want_q)

        unfuse_producers(model)
        eager._shared_activations.clear()
        block.input_layernorm(x)
        assert 0 not in eager._shared_activations


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_fused_llama_matches_unfused(fmt, g):
    """Whole model: fused and unfused logits agree up to the rare bf16 flips between this library's
    RMSNorm / SiLU arithmetic and PyTorch's, for prefill-sized and decode-sized batches."""
    from fp_quant.utils import fuse_producers
    model = _tiny_llama(fmt, g, seed=1)
    ids = torch.randint(0, 128, (2, 48), generator=torch.Generator().manual_seed(2)).cuda()
    with torch.no_grad():
        want = model(ids).logits.float()
        want1 = model(ids[:, :1]).logits.float()
        assert fuse_producers(model) == 10
        got = model(ids).logits.float()
        got1 = model(ids[:, :1]).logits.float()
    for a, b in ((got, want), (got1, want1)):
        err = (a - b).norm() / b.norm()
        assert float(err) < 0.02, float(err)
    # generation through the fused model runs (KV cache, single-token steps)
    out = model.generate(ids[:, :8], max_new_tokens=4, do_sample=False)
    assert out.shape == (2, 12)


@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 4), ("mxfp4", 128, 64), ("nvfp4", 16, 4)])
def test_fused_block_is_graph_capturable(fmt, g, m):
    """Inside a capture the norm's quantization is shared with the projections recorded after it;
    replays follow new input contents, and eager calls afterwards never use captured results."""
    from fp_quant.utils import fuse_producers
    model = _tiny_llama(fmt, g, seed=3)
    fuse_producers(model)
    block = model.model.layers[0]

    def step(x):
        y = block.input_layernorm(x)
        return block.self_attn.q_proj(y) + block.self_attn.o_proj(y), block.mlp(x)

    static_x = torch.randn(m, 256, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        step(static_x)                                   # warm-up: tables, caches, packed weights
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = step(static_x)
        for seed in range(3):
            fresh = torch.randn(m, 256, device="cuda", generator=torch.Generator("cuda").manual_seed(seed)).to(torch.bfloat16)
            eager = step(fresh.clone())                  # eager work between replays
            static_x.copy_(fresh)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out[0], eager[0]) and torch.equal(static_out[1], eager[1])
        # an eager call on the captured input object right after a capture must quantize for itself
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2):
            step(static_x)
        eager = step(static_x)
        again = step(static_x.clone())
        assert torch.equal(eager[0], again[0]) and torch.equal(eager[1], again[1])


def test_fused_llama_in_inference_mode():
    """Under torch.inference_mode() the fused modules still run (the MLP hands its quantized input
    over directly; the norm's quantization is not shared) and give the no_grad logits."""
    from fp_quant.utils import fuse_producers
    model = _tiny_llama("mxfp4", 128, seed=5)
    fuse_producers(model)
    ids = torch.randint(0, 128, (2, 40), generator=torch.Generator().manual_seed(3)).cuda()
    with torch.no_grad():
        want = model(ids).logits
    with torch.inference_mode():
        got = model(ids).logits
    assert torch.equal(got, want)


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
@pytest.mark.parametrize("shape", [(2, 48), (1, 200), (2, 3)])
def test_residual_adds_in_the_gemm_change_nothing(fmt, g, shape):
    """Moving the block's two additions into the o_proj / down_proj GEMMs (or, where the GEMM cannot
    take them, adding afterwards) gives bit for bit the block with PyTorch's additions."""
    from fp_quant.utils import fuse
    model = _tiny_llama(fmt, g, seed=7)
    for block in model.model.layers:
        assert fuse.fuse_rmsnorm(block.input_layernorm, block.self_attn.q_proj)
        assert fuse.fuse_rmsnorm(block.post_attention_layernorm, block.mlp.gate_proj)
        assert fuse.fuse_gated_mlp(block.mlp)
    ids = torch.randint(0, 128, shape, generator=torch.Generator().manual_seed(4)).cuda()
    with torch.no_grad():
        want = model(ids, output_hidden_states=True)
        want_tokens = model.generate(ids[:, :3], max_new_tokens=5, do_sample=False)
        for block in model.model.layers:
            assert fuse.fuse_residual_adds(block)
        got = model(ids, output_hidden_states=True)
        for a, b in zip(got.hidden_states, want.hidden_states):
            assert torch.equal(a, b)
        assert torch.equal(got.logits, want.logits)
        assert all(b.self_attn.o_proj._fpq_residual is None for b in model.model.layers)
        # generation (KV cache, one-token steps) takes the same tokens
        assert torch.equal(model.generate(ids[:, :3], max_new_tokens=5, do_sample=False), want_tokens)
        fuse.unfuse_producers(model)
        assert all("forward" not in vars(b) for b in model.model.layers)
        assert fuse.fuse_producers(model) == 10


def test_pending_residual_of_a_linear():
    """A tensor left in `_fpq_residual` is added by the next forward and cleared; a forward that
    builds an autograd graph leaves it alone; a shape that does not fit is not taken."""
    import fp_quant
    torch.manual_seed(11)
    lin = torch.nn.Linear(512, 384, bias=True, device="cuda", dtype=torch.bfloat16)
    layer = fp_quant.FPQuantLinear(512, 384, bias=True, config=_cfg("mxfp4", 128), device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(lin.weight)
        layer.bias.copy_(lin.bias)
    layer.pre_forward()
    for m in (4, 96):
        x = torch.randn(m, 512, device="cuda", dtype=torch.bfloat16)
        res = torch.randn(m, 384, device="cuda", dtype=torch.bfloat16)
        with torch.no_grad():
            plain = layer(x)
            layer._fpq_residual = res
            got = layer(x)
            assert layer._fpq_residual is None
            assert torch.equal(got, plain + res)
            assert torch.equal(layer(x), plain)
            layer._fpq_residual = res[:, :100]
            assert torch.equal(layer(x), plain) and layer._fpq_residual is not None
            layer._fpq_residual = None
    # the fused block's forward falls back to the original one when a graph is being built
    model = _tiny_llama("mxfp4", 128, seed=8)
    from fp_quant.utils import fuse_producers
    fuse_producers(model)
    emb = torch.randn(1, 8, 256, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    with pytest.raises(NotImplementedError):
        model(inputs_embeds=emb).logits.sum().backward()


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_compiled_static_cache_decode_matches_eager(fmt, g):
    """The reference README's recipe for fast generation: model.forward under
    torch.compile(mode="reduce-overhead", fullgraph=True) over a static KV cache, i.e. every decode step one
    replayed HIP graph holding this library's operators.  With the compiler told to keep PyTorch's bf16
    roundings between elementwise operators (emulate_precision_casts) the logits of every step equal the
    eager model's bit for bit."""
    import torch._inductor.config as inductor_config
    from transformers import StaticCache
    model = _tiny_llama(fmt, g, seed=9)
    cfg = model.config
    ids = torch.randint(0, 128, (2, 24), generator=torch.Generator().manual_seed(6)).cuda()
    toks = torch.randint(0, 128, (5, 2, 1), generator=torch.Generator().manual_seed(7)).cuda()

    def fresh_cache():
        cache = StaticCache(config=cfg, max_cache_len=64)
        model(input_ids=ids, past_key_values=cache, use_cache=True)
        return cache

    with torch.no_grad():
        cache = fresh_cache()
        want = [model(input_ids=t, past_key_values=cache, use_cache=True).logits.clone() for t in toks]
        cache = fresh_cache()
        torch._dynamo.reset()
        with inductor_config.patch(emulate_precision_casts=True):
            step = torch.compile(model.forward, mode="reduce-overhead", fullgraph=True)
            got = [step(input_ids=t, past_key_values=cache, use_cache=True).logits.clone() for t in toks]
    torch._dynamo.reset()
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), i


@pytest.mark.parametrize("arch", ["qwen3", "mistral"])
def test_fuse_producers_on_other_llama_layout_models(arch):
    """Qwen3 (the reference's headline family) and Mistral blocks have the Llama layout: every norm,
    MLP and residual addition is patched, and the fused model follows the unfused one."""
    import fp_quant
    from fp_quant.utils import fuse_producers, unfuse_producers
    if arch == "qwen3":
        from transformers import Qwen3Config as Cfg, Qwen3ForCausalLM as Model
    else:
        from transformers import MistralConfig as Cfg, MistralForCausalLM as Model
    torch.manual_seed(12)
    cfg = Cfg(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=256)
    model = Model(cfg).to(device="cuda", dtype=torch.bfloat16).eval()
    fp_quant.replace_quantize_with_fp_quant_linear(model, _cfg("mxfp4", 128))
    ids = torch.randint(0, 128, (2, 48), generator=torch.Generator().manual_seed(2)).cuda()
    with torch.no_grad():
        want = model(ids).logits.float()
        assert fuse_producers(model) == 10
        got = model(ids).logits.float()
        assert float((got - want).norm() / want.norm()) < 0.02
        assert model.generate(ids[:, :8], max_new_tokens=3, do_sample=False).shape == (2, 11)
        unfuse_producers(model)
        assert torch.equal(model(ids).logits.float(), want)


@pytest.mark.parametrize("tokens", [4, 64])
def test_fused_decoder_block_with_residual_epilogues_is_graph_capturable(tokens):
    """The whole patched block (norm+quantize, attention, o_proj with the residual in its GEMM, fused MLP with
    the residual in down_proj's GEMM) recorded into a HIP graph and replayed on new inputs."""
    from fp_quant.utils import fuse_producers
    model = _tiny_llama("mxfp4", 128, seed=13)
    assert fuse_producers(model) == 10
    block = model.model.layers[1]
    pos = torch.arange(tokens, device="cuda").unsqueeze(0)
    static_x = torch.randn(1, tokens, 256, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        emb = model.model.rotary_emb(static_x, position_ids=pos)

        def step(x):
            return block(x, position_embeddings=emb, attention_mask=None)

        step(static_x)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = step(static_x)
        for seed in range(3):
            fresh = torch.randn(1, tokens, 256, device="cuda",
                                generator=torch.Generator("cuda").manual_seed(seed)).to(torch.bfloat16)
            want = step(fresh.clone())
            static_x.copy_(fresh)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), seed
    assert block.self_attn.o_proj._fpq_residual is None


@pytest.mark.parametrize("fmt,g,arch,held_once", [("mxfp4", 128, "llama", False), ("nvfp4", 16, "llama", False),
                                                  ("mxfp4", 128, "qwen3", False), ("nvfp4", 16, "qwen3", False),
                                                  pytest.param("mxfp4", 128, "llama", True, marks=needs_packed)])
def test_compiled_decode_with_grouped_operators_matches_eager(fmt, g, arch, held_once):
    """fuse_producers before torch.compile: the traced attention calls one operator for q/k/v and the
    traced MLP two (gate/up; SiLU*up -> down) instead of seven layer operators and an elementwise kernel.
    Reference: the eager model with only its MLPs fused (the fused SiLU*up arithmetic is this library's, the
    norms and additions are PyTorch's in both), under the compiler's emulate_precision_casts."""
    import fp_quant
    import torch._inductor.config as inductor_config
    from torch._dynamo.utils import counters
    from transformers import StaticCache
    from fp_quant.utils import fuse
    if arch == "llama":
        model = _tiny_llama(fmt, g, seed=21)
    else:
        from transformers import Qwen3Config, Qwen3ForCausalLM
        torch.manual_seed(21)
        cfg = Qwen3Config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                          num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=256)
        model = Qwen3ForCausalLM(cfg).to(device="cuda", dtype=torch.bfloat16).eval()
        fp_quant.replace_quantize_with_fp_quant_linear(model, _cfg(fmt, g))
    cfg = model.config
    for block in model.model.layers:
        assert fuse.fuse_gated_mlp(block.mlp)
    ids = torch.randint(0, 128, (2, 24), generator=torch.Generator().manual_seed(6)).cuda()
    toks = torch.randint(0, 128, (4, 2, 1), generator=torch.Generator().manual_seed(7)).cuda()

    def fresh_cache():
        cache = StaticCache(config=cfg, max_cache_len=64)
        model(input_ids=ids, past_key_values=cache, use_cache=True)
        return cache

    with torch.no_grad():
        cache = fresh_cache()
        want = [model(input_ids=t, past_key_values=cache, use_cache=True).logits.clone() for t in toks]
        assert fuse.fuse_producers(model) == 10
        assert all(b.self_attn._fpq_qkv_alike for b in model.model.layers)
        eager_again = fresh_cache()      # the patched attention forward, called eagerly, changes nothing
        assert torch.equal(model(input_ids=toks[0], past_key_values=eager_again, use_cache=True).logits, want[0])
        fuse.unfuse_producers(model)
        for block in model.model.layers:     # back to the reference configuration for the prefill
            assert fuse.fuse_gated_mlp(block.mlp)
        cache = fresh_cache()
        assert fuse.fuse_producers(model) == 10
        if held_once:    # every operator of the traced model on weights held in the packed layout only
            from fp_quant.utils import release_row_major_weights
            assert release_row_major_weights(model) == 14
        torch._dynamo.reset()
        counters.clear()
        with inductor_config.patch(emulate_precision_casts=True):
            step = torch.compile(model.forward, mode="reduce-overhead", fullgraph=True)
            got = [step(input_ids=t, past_key_values=cache, use_cache=True).logits.clone() for t in toks]
    torch._dynamo.reset()
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), i


@needs_packed
@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
@pytest.mark.parametrize("tokens", [1, 3, 40, 300])
def test_grouped_projections_run_as_one_gemm_on_concatenated_packed_weights(tokens, fmt, g):
    """After fuse_producers q/k/v (and gate/up) of an MXFP4 block are one GEMM on the layers' packed weights
    laid end to end: same bits as the three (two) layers called one by one, the layers' own packed copies
    are views into the concatenated buffers, and a load_state_dict is followed."""
    from fp_quant.module import eager
    from fp_quant.utils import fuse_producers
    model = _tiny_llama(fmt, g, seed=3)
    other = _tiny_llama(fmt, g, seed=4)
    grouped = True      # both formats, every row count
    block, block2 = model.model.layers[0], other.model.layers[0]
    attn, mlp = block.self_attn, block.mlp
    x = (torch.randn(1, tokens, 256, device="cuda") * 1.5).to(torch.bfloat16)
    with torch.no_grad():
        want = [l(x.clone()) for l in (attn.q_proj, attn.k_proj, attn.v_proj)]
        want_mlp = [l(x.clone()) for l in (mlp.gate_proj, mlp.up_proj)]
        want2 = [l(x.clone()) for l in (block2.self_attn.q_proj, block2.self_attn.k_proj, block2.self_attn.v_proj)]
        assert fuse_producers(model) == 10
        group = attn._fpq_weight_group
        assert group is not None and group.n == sum(w.shape[-1] for w in want) and mlp._fpq_weight_group is not None
        lo, hi = group.wp.data_ptr(), group.wp.data_ptr() + group.wp.numel()
        for layer in (attn.q_proj, attn.k_proj, attn.v_proj):
            assert lo <= packed_copy(layer)[0].data_ptr() < hi        # no further copy of the weights
        got = attn._fpq_qkv(x)
        # k and v have 128 output features here: column ranges of one output matrix
        assert (got[0].data_ptr() + 2 * want[0].shape[-1] == got[1].data_ptr()) == grouped
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        gate, up = want_mlp
        # gate and up have 512 each (multiples of 256): the one GEMM writes a dense matrix per layer
        from fp_quant.utils import fuse
        pair = fuse._eager_group_linear(mlp, (mlp.gate_proj, mlp.up_proj), x)
        assert (pair is not None) == grouped
        if grouped:
            assert all(t.is_contiguous() for t in pair) and torch.equal(pair[0], gate) and torch.equal(pair[1], up)
        assert torch.equal(block.mlp(x), block.mlp.down_proj(O.silu_mul(
            gate.cpu().view(-1, gate.shape[-1]), up.cpu().view(-1, up.shape[-1])).view(gate.shape).cuda()))
        # traced callers: the same through the operator
        outs = eager.linear_cat_w4a4_op(x.view(-1, 256), attn.q_proj.forward_hadamard_matrix, group.wp, group.wsp,
                                        group.splits, attn.q_proj.weight_global_scale, attn.q_proj.act_global_scale,
                                        group.bias, fmt == "nvfp4")
        for a, b in zip(outs, want):
            assert a.is_contiguous() and torch.equal(a.reshape(b.shape), b)
        # new weights: the hook rebuilds the group
        attn.load_state_dict(block2.self_attn.state_dict())
        assert attn._fpq_weight_group is not group
        assert attn._fpq_weight_group.wp.data_ptr() == lo      # ... in the buffers of the one it replaces
        for a, b in zip(attn._fpq_qkv(x), want2):
            assert torch.equal(a, b)


@needs_packed
@pytest.mark.parametrize("order,fmt,g", [("fuse_then_release", "mxfp4", 128), ("release_then_fuse", "mxfp4", 128),
                                         ("fuse_then_release", "nvfp4", 16), ("release_then_fuse", "nvfp4", 16)])
def test_model_with_weights_held_once_keeps_its_logits(order, fmt, g):
    """release_row_major_weights on a whole model, before or after fuse_producers: every layer holds the
    packed layout only (the groups of projections included: their members are views into the group's
    buffers), logits keep their bits eagerly and compiled, the state dict is the reference's, and loading
    another model's state dict is followed."""
    import fp_quant
    from fp_quant.utils import fuse_producers, release_row_major_weights, restore_row_major_weights
    model = _tiny_llama(fmt, g, seed=11)
    other = _tiny_llama(fmt, g, seed=12)
    ids = torch.randint(0, 128, (2, 40), generator=torch.Generator().manual_seed(3)).cuda()
    one = ids[:, :1].contiguous()
    n_layers = sum(isinstance(m, fp_quant.FPQuantLinear) for m in model.modules())
    with torch.no_grad():
        fuse_producers(other)
        want_other = other(input_ids=ids).logits
        reference_state = {k: v.clone() for k, v in model.state_dict().items()}
        if order == "fuse_then_release":
            assert fuse_producers(model) == 10
            want, want_one = model(input_ids=ids).logits, model(input_ids=one).logits
            assert release_row_major_weights(model) == n_layers
        else:
            assert release_row_major_weights(model) == n_layers
            assert fuse_producers(model) == 10
            restore_row_major_weights(model)
            want, want_one = model(input_ids=ids).logits, model(input_ids=one).logits
            assert release_row_major_weights(model) == n_layers
        for block in model.model.layers:
            attn, group = block.self_attn, block.self_attn._fpq_weight_group
            assert group is not None and block.mlp._fpq_weight_group is not None
            lo, hi = group.wp.data_ptr(), group.wp.data_ptr() + group.wp.numel()
            for layer in (attn.q_proj, attn.k_proj, attn.v_proj):
                assert layer.weights_packed_only and lo <= layer.qweight.data_ptr() < hi
        assert torch.equal(model(input_ids=ids).logits, want)
        assert torch.equal(model(input_ids=one).logits, want_one)
        state = model.state_dict()
        assert list(sorted(state)) == list(sorted(reference_state))
        for k, v in reference_state.items():
            assert state[k].shape == v.shape and torch.equal(state[k], v), k
        model.load_state_dict(other.state_dict())
        assert all(m.weights_packed_only for m in model.modules() if isinstance(m, fp_quant.FPQuantLinear))
        assert torch.equal(model(input_ids=ids).logits, want_other)
