"""MXFP4 "quest" quantizer on the GPU: codes, scale bytes and clip mask bit-exact against the oracle,
and the operator / module surface for forward_method="quest"."""
import pytest
import torch

from oracle import fpq_oracle as O
from fp_quant import _engine
import capi
from conftest import make_outlier_normal, make_student_t, row_major_weights

pytestmark = pytest.mark.gpu

OK = {"hadamard": O.ROT_HADAMARD, "identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR}


@pytest.mark.parametrize("rot,g", [("hadamard", 128), ("hadamard", 64), ("hadamard", 32), ("hadamard", 16),
                                   ("identity", 32), ("gsr", 128), ("gsr", 32)])
@pytest.mark.parametrize("policy", [_engine.ZERO_REFERENCE, _engine.ZERO_SIGNED])
def test_quest_bit_exact(rot, g, policy):
    rows, cols = 37, 384
    x = make_outlier_normal(rows, cols, 5 * g + len(rot), frac=0.02, mult=40.0)
    x[3, 64:96] = 0.0
    x[4, 32:64] = 1.5            # a constant group: variance rounds to ~0
    x[6] *= 2.0 ** -60
    x[8] *= 2.0 ** 40           # (beyond about 2^60 the sum of squares overflows fp32, as in the reference)
    norm = float(O.hadamard_matrix(g)[0, 0])
    wc, ws, wm, _ = O.quantize_mx_quest(x, OK[rot], g, norm, zero_nibble=policy)
    codes, scales, mask = capi.quantize_quest(x, rot=rot, g=g, norm=norm, zero_policy=policy)
    assert torch.equal(scales, ws)
    assert torch.equal(mask, wm)
    assert torch.equal(codes, wc)
    assert (wm != 0xff).any()    # something clipped, so the mask is not trivially all ones


def test_quest_general_matrix_and_padded_scales():
    gen = torch.Generator().manual_seed(12)
    q, _ = torch.linalg.qr(torch.randn(32, 32, generator=gen))
    h = q.to(torch.bfloat16)
    x = make_student_t(20, 256, 3)
    wc, ws, wm, _ = O.quantize_mx_quest(x, O.ROT_GENERAL, 32, h=h)
    codes, scales, mask = capi.quantize_quest(x, rot="general", g=32, h=h, pad=True)
    assert torch.equal(codes, wc) and torch.equal(mask, wm)
    assert torch.equal(scales[:20, :8], ws)
    assert (scales[20:] == 0).all() and (scales[:, 8:] == 0).all()
    c2, s2, none = capi.quantize_quest(x, rot="general", g=32, h=h, want_mask=False)
    assert none is None and torch.equal(c2, wc) and torch.equal(s2, ws)


def test_quest_full_size_block():
    x = make_outlier_normal(2048, 4096, 0)
    wc, ws, wm, _ = O.quantize_mx_quest(x, O.ROT_HADAMARD, 128)
    codes, scales, mask = capi.quantize_quest(x, g=128)
    assert torch.equal(codes, wc) and torch.equal(scales, ws) and torch.equal(mask, wm)


def test_quest_operator_and_linear():
    import fp_quant
    from fp_quant.module import hip_ops
    x = make_outlier_normal(40, 256, 4).cuda()
    h = O.hadamard_matrix(64).cuda()
    codes, scales, mask = hip_ops.fused_quantize_mx_op(x, h, "quest", True)
    wc, ws, wm, _ = O.quantize_mx_quest(x.cpu(), O.ROT_HADAMARD, 64)
    assert mask.shape == (40, 32) and mask.dtype == torch.uint8
    assert scales.shape == (128, 8) and scales.dtype == torch.float8_e8m0fnu
    assert torch.equal(codes.cpu(), wc) and torch.equal(mask.cpu(), wm)
    assert torch.equal(scales.view(torch.uint8).cpu()[:40], ws)
    _, _, none = hip_ops.fused_quantize_mx_op(x, h, "quest", False)
    assert none is None

    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="quest",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=64)
    gen = torch.Generator().manual_seed(8)
    w = (torch.randn(96, 256, generator=gen) * 0.02).to(torch.bfloat16)
    lin = fp_quant.FPQuantLinear(256, 96, cfg, bias=False, device="cuda", dtype=torch.bfloat16)
    lin.weight.data = w.cuda()
    lin.pre_forward()
    assert float(lin.weight_global_scale) == 1.0 and float(lin.act_global_scale) == 1.0   # linear.py:190-192
    wq, wsc, _, _ = O.quantize_mx_quest(w, O.ROT_HADAMARD, 64)
    got_q, got_s = row_major_weights(lin)
    assert torch.equal(got_q, wq) and torch.equal(got_s, wsc)
    y = lin(x).cpu()
    ref, mag = O.gemm_ref(wc, ws, wq, wsc, 1.0, "mxfp4")
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag).all()
    dense = x.cpu().double() @ w.double().T
    assert (y.double() - dense).norm() / dense.norm() < 0.3


@pytest.mark.parametrize("m", [1, 30, 70, 300])
def test_quest_module_equals_the_operator_chain(m):
    """FPQuantLinear with forward_method="quest" (direct calls into the library, activations re-tiled
    for the packed GEMM from 25 rows on) gives the bits of fused_quantize_mx_op followed by
    matmul_mxf4_bf16_tn_op, eagerly, under torch.compile, and for layers sharing one input."""
    import fp_quant
    from fp_quant.module import hip_ops
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="quest",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=128)
    torch.manual_seed(31)
    layers = []
    for n in (192, 320):
        lin = fp_quant.FPQuantLinear(512, n, cfg, bias=(n == 320), device="cuda", dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.normal_(0, 0.05)
            if lin.bias is not None:
                lin.bias.normal_(0, 1)
        lin.pre_forward()
        layers.append(lin)
    x = make_outlier_normal(m, 512, 9).cuda()
    with torch.no_grad():
        codes, scales, _ = hip_ops.fused_quantize_mx_op(x, layers[0].forward_hadamard_matrix, "quest", False)
        alpha = torch.ones(1, dtype=torch.float32, device="cuda")
        for lin in layers:                      # called one after the other with the same tensor: shared
            wq, ws = (t.cuda() for t in row_major_weights(lin))
            want = hip_ops.matmul_mxf4_bf16_tn_op(codes, wq, scales, ws.view(torch.float8_e8m0fnu), alpha)
            if lin.bias is not None:
                want = want + lin.bias
            assert torch.equal(lin(x), want)
            torch._dynamo.reset()
            assert torch.equal(torch.compile(lin, fullgraph=True)(x), want)
    torch._dynamo.reset()
    # a forward that needs the clip mask (autograd) still goes through the operators and has no backward
    xg = x.clone().requires_grad_(True)
    with pytest.raises(NotImplementedError):
        layers[0](xg).sum().backward()


def _quest_input(rows, cols, seed):
    x = make_outlier_normal(rows, cols, seed, frac=0.02, mult=40.0)
    x[0, 64:96] = 0.0
    x[0, 32:64] = 1.5            # a constant group: variance rounds to ~0
    if rows > 8:
        x[6] *= 2.0 ** -60
        x[8] *= 2.0 ** 40
        x[5, :128] = -x[5, :128].abs() * 2.0 ** -120     # negative values far below every scale
    return x


STREAM_CASES = [("hadamard", 128), ("hadamard", 64), ("hadamard", 32), ("hadamard", 16), ("identity", 32),
                ("gsr", 64), ("gsr", 16)]


@pytest.mark.parametrize("rot,g", STREAM_CASES)
@pytest.mark.parametrize("policy", [_engine.ZERO_REFERENCE, _engine.ZERO_SIGNED])
def test_quest_streaming_kernel_bit_exact(rot, g, policy):
    """Inputs of 2^21 elements and more without a clip mask take the streaming kernel: same codes and scale
    bytes as the oracle (the last tile is ragged: 1030 rows of 2048)."""
    rows, cols = 1030, 2048
    x = _quest_input(rows, cols, 7 * g + len(rot))
    norm = float(O.hadamard_matrix(g)[0, 0])
    wc, ws, _, _ = O.quantize_mx_quest(x, OK[rot], g, norm, zero_nibble=policy)
    codes, scales, none = capi.quantize_quest(x, rot=rot, g=g, norm=norm, zero_policy=policy, want_mask=False)
    assert none is None
    assert torch.equal(scales, ws)
    assert torch.equal(codes, wc)
    # with a mask the generic kernel runs: same codes
    codes2, scales2, _ = capi.quantize_quest(x, rot=rot, g=g, norm=norm, zero_policy=policy)
    assert torch.equal(codes2, wc) and torch.equal(scales2, ws)


@pytest.mark.parametrize("rot,g", [("hadamard", 128), ("hadamard", 32), ("gsr", 64)])
def test_quest_streaming_kernel_from_two_to_the_24_elements(rot, g):
    """From 2^24 elements on a lane of the streaming kernel owns 64 elements instead of 32."""
    rows, cols = 4100, 4096
    x = _quest_input(rows, cols, 11 * g + len(rot))
    norm = float(O.hadamard_matrix(g)[0, 0])
    wc, ws, _, _ = O.quantize_mx_quest(x, OK[rot], g, norm)
    codes, scales, _ = capi.quantize_quest(x, rot=rot, g=g, norm=norm, want_mask=False)
    assert torch.equal(scales, ws) and torch.equal(codes, wc)
    from test_packed_gpu import pack_by_definition
    want_c, want_s = pack_by_definition(wc, ws, cols)
    pc, ps = capi.quantize_quest_packed(x, rot=rot, g=g, norm=norm)
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)


@pytest.mark.parametrize("rot,g", STREAM_CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (20, 768), (64, 512), (70, 512), (300, 1024), (2100, 256)])
def test_quest_packed_bit_exact(rot, g, rows, cols):
    """fpq_quantize_mx_quest_packed (generic kernel up to 64 rows, streaming kernel beyond): the oracle's
    codes and scales in the packed layout, zero padding rows."""
    from test_packed_gpu import pack_by_definition
    x = _quest_input(rows, cols, rows + g)
    norm = float(O.hadamard_matrix(g)[0, 0])
    wc, ws, _, _ = O.quantize_mx_quest(x, OK[rot], g, norm)
    want_c, want_s = pack_by_definition(wc, ws, cols)
    pc, ps = capi.quantize_quest_packed(x, rot=rot, g=g, norm=norm)
    assert torch.equal(ps, want_s)
    assert torch.equal(pc, want_c)


def test_quest_packed_declines_rotations_it_cannot_take():
    lib = _engine.lib()
    x = torch.zeros(64, 256, dtype=torch.bfloat16, device="cuda")
    pc = torch.zeros(64 * 128, dtype=torch.uint8, device="cuda")
    ps = torch.zeros(64 * 8, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.fpq_quantize_mx_quest_packed(x.data_ptr(), 64, 256, _engine.ROT_GSR, 128, 0.088, pc.data_ptr(),
                                            ps.data_ptr(), 0, st) == _engine.E_UNSUPPORTED
    assert lib.fpq_quantize_mx_quest_packed(x.data_ptr(), 64, 256, _engine.ROT_GENERAL, 32, 0.088, pc.data_ptr(),
                                            ps.data_ptr(), 0, st) == _engine.E_UNSUPPORTED
    assert lib.fpq_quantize_mx_quest_packed(x.data_ptr(), 64, 200, 0, 32, 0.088, pc.data_ptr(), ps.data_ptr(), 0,
                                            st) == -2
