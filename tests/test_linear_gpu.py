"""FPQuantLinear end to end on the GPU: pre_forward weight quantization, forward through the
operators, replace helpers, torch.compile friendliness of the operators."""
import pytest
import torch
from torch import nn

from oracle import fpq_oracle as O
from tests.conftest import (PACKED_WEIGHTS, SINGLE_WEIGHT_COPY, needs_packed, needs_row_major_parameters, packed_copy,
                            row_major_weights)

pytestmark = pytest.mark.gpu


def _cfg(fmt, g, **kw):
    import fp_quant
    return fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype(fmt), forward_method="abs_max",
                                  backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=g, **kw)


@pytest.mark.parametrize("fmt,g", [("mxfp4", 32), ("mxfp4", 128), ("nvfp4", 16), ("nvfp4", 64)])
@pytest.mark.parametrize("bias", [False, True])
def test_linear_matches_oracle_pipeline(fmt, g, bias):
    import fp_quant
    gen = torch.Generator().manual_seed(3)
    k, n = 512, 384
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    b = torch.randn(n, generator=gen).to(torch.bfloat16) if bias else None
    x = torch.randn(2, 9, k, generator=gen).to(torch.bfloat16)
    lin = fp_quant.FPQuantLinear(k, n, _cfg(fmt, g), bias=bias, device="cuda", dtype=torch.bfloat16)
    lin.weight.data = w.cuda()
    if bias:
        lin.bias.data = b.cuda()
    lin.pre_forward()
    assert lin.weight is None and lin.dqweight is None
    group = 32 if fmt == "mxfp4" else 16
    if not SINGLE_WEIGHT_COPY:
        assert lin.qweight.dtype == torch.uint8 and lin.qweight.shape == (n, k // 2)
        assert lin.scales.dtype == torch.uint8 and lin.scales.shape == (n, k // group)
    got_q, got_s = row_major_weights(lin)
    assert got_q.dtype == torch.uint8 and got_q.shape == (n, k // 2) and got_s.shape == (n, k // group)
    # linear.py:190-200: the abs_max branch (3.0) is tested before the NVFP4 branch (10.0), and
    # NVFP4 only validates with abs_max, so every real-quant layer gets 3.0
    gsv = 3.0
    assert float(lin.weight_global_scale) == gsv and float(lin.act_global_scale) == gsv
    assert torch.equal(lin.forward_hadamard_matrix.cpu(), O.hadamard_matrix(g))

    # weights: bit-exact against the oracle quantizer
    norm = float(O.hadamard_matrix(g)[0, 0])
    if fmt == "mxfp4":
        wq, ws, _ = O.quantize_mx(w, O.ROT_HADAMARD, g, norm)
        xq, xs, _ = O.quantize_mx(x.view(-1, k), O.ROT_HADAMARD, g, norm)
    else:
        wq, ws, _ = O.quantize_nv(w, gsv, O.ROT_HADAMARD, g, norm)
        xq, xs, _ = O.quantize_nv(x.view(-1, k), gsv, O.ROT_HADAMARD, g, norm)
    assert torch.equal(got_q, wq) and torch.equal(got_s, ws)

    y = lin(x.cuda())
    assert y.shape == (2, 9, n) and y.dtype == torch.bfloat16
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, fmt)
    yb = ref.to(torch.bfloat16)
    if bias:
        yb = yb + b
    got = y.cpu().view(-1, n)
    close = (got.double() - yb.double()).abs() <= 2.0 ** -7 * yb.double().abs() + 1e-5 * mag + 1e-6
    assert close.all()
    # and it approximates the unquantized linear
    dense = x.view(-1, k).double() @ w.double().T + (b.double() if bias else 0)
    rel = (got.double() - dense).norm() / dense.norm()
    assert rel < 0.25, rel


@needs_packed
@pytest.mark.parametrize("m", [9, 100, 200])
def test_nvfp4_layer_with_a_long_k_owns_a_split_k_workspace(m):
    """The NVFP4 counterpart of the test below, in short: workspace made at priming, oracle values, eager ==
    traced operator == C entry point with a workspace of its own -- at one and at four activation row tiles and
    at 200 rows, which run as two passes of the kernel that splits K."""
    import capi
    from fp_quant.module import eager
    from test_packed_gpu import pack_nv_by_definition
    k, n = 8192, 256
    lin = _quantized_linear("nvfp4", 16, k, n, seed=22, bias=True)
    wsk = getattr(lin.qweight, "_fpq_splitk", None)
    assert wsk is not None and wsk.numel() > 16384
    norm = float(O.hadamard_matrix(16)[0, 0])
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    xq, xs, _ = O.quantize_nv(x, float(lin.act_global_scale), O.ROT_HADAMARD, 16, norm)
    wq, ws = row_major_weights(lin)
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "nvfp4")
    want = ref.to(torch.bfloat16) + lin.bias.detach().cpu()
    with torch.no_grad():
        y = lin(x.cuda())
        op = eager.linear_w4a4_op(x.cuda(), lin.forward_hadamard_matrix, lin.qweight, lin.scales,
                                  lin.weight_global_scale, lin.act_global_scale, lin.bias, True)
    assert torch.equal(op, y)
    assert ((y.cpu().double() - want.double()).abs() <= 2.0 ** -6 * want.double().abs() + 1e-5 * mag + 1e-6).all()
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    own = torch.zeros(wsk.numel(), dtype=torch.uint8, device="cuda")
    direct = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=lin.bias.detach().cpu(), workspace=own,
                                     nv=True)
    assert torch.equal(y.cpu(), direct) and not wsk[:16384].any()
    # the split is really taken: K whole (no workspace) sums in another order
    whole = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=lin.bias.detach().cpu())
    assert ((whole.double() - want.double()).abs() <= 2.0 ** -6 * want.double().abs() + 1e-5 * mag + 1e-6).all()


@needs_packed
@pytest.mark.parametrize("bias", [False, True])
def test_decode_rows_on_a_long_k_split_k_across_workgroups(bias):
    """A layer with few output features and a long K (a down-projection) owns a workspace with which its GEMM
    splits K at up to 128 rows: oracle values, the same bits as the C entry point with a workspace of its own,
    the same bits eagerly, under a graph capture on another stream and through the traced operator, the
    residual taken inside the kernel, counters left at zero; more rows run the tile kernel, which does not split."""
    import capi
    from fp_quant import _engine
    from fp_quant.module import eager, hip_ops
    from test_packed_gpu import pack_by_definition
    k, n = 8192, 256
    lin = _quantized_linear("mxfp4", 128, k, n, seed=21, bias=bias)
    wsk = getattr(lin.qweight, "_fpq_splitk", None)
    assert wsk is not None and wsk.numel() == _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes(128, n, k) > 16384
    norm = float(O.hadamard_matrix(128)[0, 0])
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    wq, ws = row_major_weights(lin)
    wp, wsp = pack_by_definition(wq, ws, k)
    b = lin.bias.detach().cpu() if bias else None
    for m in (1, 20, 32, 50, 128):
        x = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).to(torch.bfloat16)
        xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, 128, norm)
        ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "mxfp4")
        want = ref.to(torch.bfloat16) + b if bias else ref.to(torch.bfloat16)
        with torch.no_grad():
            y = lin(x.cuda())
        close = (y.cpu().double() - want.double()).abs() <= 2.0 ** -7 * want.double().abs() + 1e-5 * mag + 1e-6
        assert close.all()
        xp, xsp = pack_by_definition(xq, xs, k)
        own = torch.zeros(wsk.numel(), dtype=torch.uint8, device="cuda")
        direct = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, workspace=own)
        assert torch.equal(y.cpu(), direct)
        assert not wsk[:16384].any()
        # the traced operator and a capture on a side stream take the same kernel
        xd = x.cuda()
        with torch.no_grad():
            op = eager.linear_w4a4_op(xd, lin.forward_hadamard_matrix, lin.qweight, lin.scales, lin.weight_global_scale,
                                      lin.act_global_scale, lin.bias, False)
            assert torch.equal(op, y)
            graph = torch.cuda.CUDAGraph()
            static_x = xd.clone()
            with torch.cuda.graph(graph):
                static_y = lin(static_x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, y)
            res = torch.randn(m, n, device="cuda").to(torch.bfloat16)
            lin._fpq_residual = res
            assert torch.equal(lin(xd), y + res) and lin._fpq_residual is None
    with torch.no_grad():
        x = torch.randn(129, k, generator=torch.Generator().manual_seed(33)).to(torch.bfloat16)
        xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, 128, norm)
        xp, xsp = pack_by_definition(xq, xs, k)
        assert torch.equal(lin(x.cuda()).cpu(), capi.gemm_packed(xp, xsp, wp, wsp, 129, n, k, alpha, bias=b))
        # the layer keeps a workspace when its weight changes hands (packed layout only and back)
        x = torch.randn(7, k, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).cuda()
        want = lin(x)
        assert lin.release_row_major() and getattr(lin.qweight, "_fpq_splitk", None) is not None
        assert torch.equal(lin(x), want)
        lin.restore_row_major()
        assert getattr(lin.qweight, "_fpq_splitk", None) is not None and torch.equal(lin(x), want)


@pytest.mark.parametrize("init", ["identity", "gsr"])
def test_other_transform_inits(init):
    """transform_init identity / gsr go through the same operators (matrix recognised on the host)."""
    import fp_quant
    from fp_quant.module import eager, hip_ops
    from fp_quant import _engine
    gen = torch.Generator().manual_seed(5)
    w = (torch.randn(64, 256, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(8, 256, generator=gen).to(torch.bfloat16)
    lin = fp_quant.FPQuantLinear(256, 64, _cfg("mxfp4", 64, transform_init=init), bias=False, device="cuda",
                                 dtype=torch.bfloat16)
    lin.weight.data = w.cuda()
    lin.pre_forward()
    kind = {"identity": _engine.ROT_IDENTITY, "gsr": _engine.ROT_GSR}[init]
    assert hip_ops.classify_rotation(lin.forward_hadamard_matrix)[0] == kind
    okind = {"identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR}[init]
    wq, ws, _ = O.quantize_mx(w, okind, 64)
    got_q, got_s = row_major_weights(lin)
    assert torch.equal(got_q, wq) and torch.equal(got_s, ws)
    xq, xs, _ = O.quantize_mx(x, okind, 64)
    ref, mag = O.gemm_ref(xq, xs, wq, ws, 0.111328125, "mxfp4")
    y = lin(x.cuda()).cpu()
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag).all()


def test_general_matrix_through_the_operator():
    from fp_quant.module import eager, hip_ops
    gen = torch.Generator().manual_seed(6)
    q, _ = torch.linalg.qr(torch.randn(32, 32, generator=gen))
    h = q.to(torch.bfloat16)
    x = torch.randn(16, 128, generator=gen).to(torch.bfloat16)
    codes, scales, _ = hip_ops.fused_quantize_mx_op(x.cuda(), h.cuda(), "abs_max", False)
    wc, wsc, _ = O.quantize_mx(x, O.ROT_GENERAL, 32, h=h)
    assert torch.equal(codes.cpu(), wc) and torch.equal(scales.view(torch.uint8).cpu()[:16, :4], wsc)


def test_replace_quantize_and_skip_rule():
    import fp_quant

    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.body = nn.Sequential(nn.Linear(128, 256, bias=True), nn.ReLU(), nn.Linear(256, 128, bias=False))
            self.lm_head = nn.Linear(128, 64, bias=False)

        def forward(self, x):
            return self.lm_head(self.body(x))

    torch.manual_seed(0)
    model = Tiny().to(device="cuda", dtype=torch.bfloat16)
    x = torch.randn(4, 128, device="cuda", dtype=torch.bfloat16)
    want = model(x)
    out = fp_quant.replace_quantize_with_fp_quant_linear(model, _cfg("mxfp4", 128))
    assert out is model
    assert isinstance(model.body[0], fp_quant.FPQuantLinear) and isinstance(model.body[2], fp_quant.FPQuantLinear)
    assert type(model.lm_head) is nn.Linear
    keys = set(model.body[0].state_dict().keys())
    assert keys == {"bias", "qweight", "scales", "weight_global_scale", "act_global_scale",
                    "forward_hadamard_matrix", "backward_hadamard_matrix"}
    got = model(x)
    assert (got.float() - want.float()).norm() / want.float().norm() < 0.3


def test_state_dict_roundtrip_without_pre_forward():
    """A checkpoint written by one layer loads into a freshly replaced (never pre_forward-ed)
    layer and gives identical outputs: what a realquant checkpoint loader relies on."""
    import fp_quant
    torch.manual_seed(1)
    cfg = _cfg("nvfp4", 16)
    src = fp_quant.FPQuantLinear(256, 128, cfg, bias=True, device="cuda", dtype=torch.bfloat16)
    src.weight.data.normal_(0, 0.02)
    src.bias.data.normal_()
    src.pre_forward()
    sd = {k: v.clone() for k, v in src.state_dict().items()}
    dst = fp_quant.FPQuantLinear(256, 128, cfg, bias=True, device="cuda", dtype=torch.bfloat16)
    dst.weight = None
    dst.dqweight = None
    dst.load_state_dict(sd)
    x = torch.randn(7, 256, device="cuda", dtype=torch.bfloat16)
    assert torch.equal(src(x), dst(x))


def test_operators_have_fake_impls_and_compile():
    from fp_quant.module import eager, hip_ops
    x = torch.randn(32, 256, device="cuda", dtype=torch.bfloat16)
    h = O.hadamard_matrix(32).cuda()

    def f(x):
        q, s, _ = hip_ops.fused_quantize_mx_op(x, h, "abs_max", False)
        return q, s

    q0, s0 = f(x)
    q1, s1 = torch.compile(f, fullgraph=True, backend="eager")(x)
    assert torch.equal(q0, q1) and torch.equal(s0.view(torch.uint8), s1.view(torch.uint8))
    assert s0.shape == (128, 8) and s0.dtype == torch.float8_e8m0fnu


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_inductor_compiled_layers_match_eager(fmt, g):
    """torch.compile(fullgraph=True) with the default (inductor) backend, which the reference's README
    recommends for speed: chained layers, a residual addition, strided intermediates.  Every
    elementwise step here is exact (relu, doubling, one addition), so compiled and eager outputs must
    be bit-identical -- which also needs alpha to keep eager's bf16 roundings inside the compiled graph."""
    import fp_quant

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.up = nn.Linear(256, 512, bias=False)
            self.down = nn.Linear(512, 256, bias=True)

        def forward(self, x):
            h = torch.relu(self.up(x)).view(x.shape[0], 4, 128).transpose(0, 1)
            h = (h * 2.0).transpose(0, 1).reshape(x.shape[0], 512)      # reaches `down` through a strided view
            return x + self.down(h)

    torch.manual_seed(21)
    net = Net().to(device="cuda", dtype=torch.bfloat16)
    fp_quant.replace_quantize_with_fp_quant_linear(net, _cfg(fmt, g))
    with torch.no_grad():
        for rows in (1, 40, 300):       # split-K, packed 128x128 and packed-linear operator paths
            x = torch.randn(rows, 256, device="cuda", dtype=torch.bfloat16)
            want = net(x)
            torch._dynamo.reset()
            got = torch.compile(net, fullgraph=True)(x)
            assert torch.equal(got, want), rows
    torch._dynamo.reset()


def test_unsupported_branches_raise():
    import fp_quant
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.MXFP4, hadamard_group_size=32)
    lin = fp_quant.FPQuantLinear(64, 32, cfg, bias=False, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        lin(torch.zeros(1, 64, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        fp_quant.FPQuantLinear(64, 32, fp_quant.FPQuantConfig(pseudoquantization=True), device="cuda")


def test_meta_replacement_then_realquant_checkpoint(tmp_path):
    """The loader route (replace.py:7-71): every nn.Linear becomes an empty meta-device FPQuantLinear,
    then the tensors of a realquant checkpoint (qweight / scales / *_global_scale / *_hadamard_matrix,
    rtn.py:185-193) are loaded from a safetensors file and the model runs without pre_forward."""
    import fp_quant
    from safetensors.torch import load_file, save_file

    class Tiny(nn.Module):
        def __init__(self):
            super().__init__()
            self.up = nn.Linear(256, 512, bias=False)
            self.down = nn.Linear(512, 256, bias=True)
            self.lm_head = nn.Linear(256, 32, bias=False)

        def forward(self, x):
            return self.lm_head(self.down(torch.relu(self.up(x))))

    cfg = _cfg("mxfp4", 128)
    torch.manual_seed(4)
    src = Tiny().to(device="cuda", dtype=torch.bfloat16)
    fp_quant.replace_quantize_with_fp_quant_linear(src, cfg)
    x = torch.randn(70, 256, device="cuda", dtype=torch.bfloat16)
    want = src(x)
    path = str(tmp_path / "realquant.safetensors")
    save_file({k: v.contiguous().cpu() for k, v in src.state_dict().items()}, path)

    # loaders build the model under the checkpoint's default dtype, so the new modules' buffers get it
    # (alpha = 1 / (wgs * ags) is evaluated in the buffers' dtype, linear_fns.py:505)
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("meta"):
            dst = Tiny()
        dst, replaced = fp_quant.replace_with_fp_quant_linear(dst, cfg)
    finally:
        torch.set_default_dtype(torch.float32)
    assert replaced
    assert isinstance(dst.up, fp_quant.FPQuantLinear) and dst.up.qweight.is_meta and type(dst.lm_head) is nn.Linear
    assert dst.up.source_cls is nn.Linear and not any(p.requires_grad for p in dst.up.parameters())
    for m in dst.modules():
        if isinstance(m, fp_quant.FPQuantLinear):
            m.weight = None       # a realquant checkpoint holds no dense weights
            m.dqweight = None
    dst.to_empty(device="cuda")
    missing, unexpected = dst.load_state_dict(load_file(path, device="cuda"), strict=True)
    assert not missing and not unexpected
    assert torch.equal(dst(x), want)


@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 1), ("mxfp4", 128, 200), ("nvfp4", 16, 8), ("nvfp4", 16, 100)])
def test_forward_is_graph_capturable(fmt, g, m):
    """After one eager warm-up call (rotation classified, alpha and packed weights cached) a forward
    records into a HIP graph: no host synchronisation, no allocation outside torch's capture pool.
    Replays, interleaved with eager work, must equal eager results on the new input contents."""
    import fp_quant
    torch.manual_seed(11)
    lin = fp_quant.FPQuantLinear(512, 256, _cfg(fmt, g), bias=True, device="cuda", dtype=torch.bfloat16)
    lin.weight.data.normal_(0, 0.02)
    lin.bias.data.normal_()
    lin.pre_forward()
    static_x = torch.randn(m, 512, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        lin(static_x)                                  # warm-up outside the capture
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            lin(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = lin(static_x)
        for rep in range(3):
            fresh = torch.randn(m, 512, device="cuda", dtype=torch.bfloat16)
            want = lin(fresh)                          # eager work between replays
            torch.cuda.synchronize()
            static_x.copy_(fresh)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), rep


def _quantized_linear(fmt, g, k, n, seed, bias=False):
    import fp_quant
    torch.manual_seed(seed)
    lin = fp_quant.FPQuantLinear(k, n, _cfg(fmt, g), bias=bias, device="cuda", dtype=torch.bfloat16)
    lin.weight.data.normal_(0, 0.02)
    if bias:
        lin.bias.data.normal_()
    lin.pre_forward()
    return lin


@needs_packed
@needs_row_major_parameters
@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 5), ("mxfp4", 32, 200), ("nvfp4", 16, 8), ("nvfp4", 16, 300)])
def test_activations_quantized_into_one_layout_serve_the_other(fmt, g, m):
    """Quantized activations held in the packed layout only feed a GEMM on row-major operands (they are
    re-tiled back, exactly) and the other way round: same output bits as quantizing for that layout."""
    from fp_quant import _engine
    from fp_quant.module import eager, hip_ops
    k, n = 512, 384
    lin = _quantized_linear(fmt, g, k, n, seed=11, bias=True)
    nv = fmt == "nvfp4"
    x = torch.randn(m, k, device="cuda", dtype=torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    h = hip_ops.as_bf16(lin.forward_hadamard_matrix)
    kind, norm = _engine.classify_rotation(h)
    alpha = eager.linear_alpha(lin.weight_global_scale, lin.act_global_scale)
    ags = lin.act_global_scale if nv else None
    with torch.no_grad():
        packed = eager.quantize_activations(x, h, kind, norm, ags, nv, stream, True)
        rows = eager.quantize_activations(x, h, kind, norm, ags, nv, stream, False)
        assert packed.row_major is None and rows.row_major is not None
        assert rows.mx_packed is None and rows.nv_packed is None
        want_rows = eager.linear_on(rows, lin.qweight, lin.scales, alpha, lin.bias, stream, False)
        want_packed = eager.linear_on(packed, lin.qweight, lin.scales, alpha, lin.bias, stream, True)
        assert torch.equal(eager.linear_on(packed, lin.qweight, lin.scales, alpha, lin.bias, stream, False), want_rows)
        assert torch.equal(eager.linear_on(rows, lin.qweight, lin.scales, alpha, lin.bias, stream, True), want_packed)
        assert torch.equal(packed.rows()[0], rows.row_major[0]) and torch.equal(packed.rows()[1], rows.row_major[1])


@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 1), ("mxfp4", 32, 200), ("nvfp4", 16, 8), ("nvfp4", 16, 100),
                                     ("nvfp4", 64, 700)])
def test_layers_sharing_an_input_share_its_quantization(fmt, g, m):
    """q/k/v-style layers called with the same tensor object reuse the quantized activations of the
    first call; outputs are bit-identical to unshared calls, and any change of the input (in-place
    write, another tensor, another rotation or global scale) quantizes again."""
    from fp_quant.module import eager, hip_ops
    k = 512
    layers = [_quantized_linear(fmt, g, k, n, seed) for seed, n in enumerate((256, 128, 384))]
    x = torch.randn(2, m, k, device="cuda", dtype=torch.bfloat16)

    def unshared(inp, lins):
        eager.SHARE_ACT_QUANT = False
        try:
            return [lin(inp) for lin in lins]
        finally:
            eager.SHARE_ACT_QUANT = True

    want = unshared(x, layers)
    eager._shared_activations.clear()
    got0 = layers[0](x)
    slot = eager._shared_activations[0]
    filled = [f for f in ("mx_packed", "row_major", "nv_packed") if getattr(slot, f) is not None]
    assert filled
    got = [got0] + [lin(x) for lin in layers[1:]]
    assert eager._shared_activations[0] is slot          # the later calls found the first call's entry
    for a, b in zip(got, want):
        assert torch.equal(a, b)

    # in-place write: same object, new version -> quantized again
    x.mul_(-1.5)
    want2 = unshared(x, layers[:2])
    assert torch.equal(layers[0](x), want2[0]) and eager._shared_activations[0] is not slot
    assert torch.equal(layers[1](x), want2[1])

    # a new tensor (very likely at the freed address) never matches the dead one
    shape = x.shape
    del x, want, got, got0, want2
    x2 = torch.randn(shape, device="cuda", dtype=torch.bfloat16)
    want3 = unshared(x2, layers[:1])[0]
    assert torch.equal(layers[0](x2), want3)

    # same tensor into a layer with another rotation size: not shared, still right
    other_g = 64 if g != 64 else 32
    other = _quantized_linear(fmt, other_g, k, 256, 7)
    want4 = unshared(x2, [other])[0]
    layers[0](x2)
    assert torch.equal(other(x2), want4)

    if fmt == "nvfp4":
        # another activation global scale quantizes differently and must not reuse the entry
        scaled = _quantized_linear(fmt, g, k, 256, 8)
        scaled.act_global_scale.fill_(5.0)
        want5 = unshared(x2, [scaled])[0]
        layers[0](x2)
        got5 = scaled(x2)
        assert torch.equal(got5, want5) and not torch.equal(got5, unshared(x2, [_quantized_linear(fmt, g, k, 256, 8)])[0])


@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 3), ("mxfp4", 32, 200), ("nvfp4", 16, 70)])
def test_inference_mode(fmt, g, m):
    """torch.inference_mode(): tensors made there carry no version counter, so nothing is cached on or
    shared through them; results equal the no_grad ones, also for a layer built inside the mode."""
    from fp_quant.module import eager, hip_ops
    lin = _quantized_linear(fmt, g, 512, 256, 21, bias=True)
    other = _quantized_linear(fmt, g, 512, 128, 22)
    x = torch.randn(m, 512, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        want, want_other = lin(x), other(x)
    with torch.inference_mode():
        eager._shared_activations.clear()
        xi = x * 1.0                                   # an inference tensor
        assert xi.is_inference()
        got, got_other = lin(xi), other(xi)
        assert not eager._shared_activations         # nothing shared: writes to xi could not be noticed
        xi.mul_(2.0)
        twice = lin(xi)
    assert torch.equal(got, want) and torch.equal(got_other, want_other)
    with torch.no_grad():
        assert torch.equal(twice, lin(x * 2.0))
    with torch.inference_mode():
        import fp_quant
        torch.manual_seed(21)
        inner = fp_quant.FPQuantLinear(512, 256, _cfg(fmt, g), bias=True, device="cuda", dtype=torch.bfloat16)
        inner.weight.data.normal_(0, 0.02)
        inner.bias.data.normal_()
        inner.pre_forward()
        assert inner.qweight.is_inference()
        assert torch.equal(inner(x), want) and torch.equal(inner(x), want)


def test_layers_called_from_two_threads_on_their_own_streams():
    """Every call runs on the calling thread's current stream and shares nothing it should not:
    two host threads, each with its own stream and inputs, calling the same layers concurrently,
    get what a single thread gets."""
    import threading
    import fp_quant
    torch.manual_seed(17)
    lins = []
    for fmt, g in (("mxfp4", 128), ("nvfp4", 16)):
        lin = fp_quant.FPQuantLinear(512, 256, _cfg(fmt, g), bias=True, device="cuda", dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.normal_(0, 0.05)
            lin.bias.normal_(0, 1)
        lin.pre_forward()
        lins.append(lin)
    inputs = [[torch.randn(m, 512, device="cuda", dtype=torch.bfloat16) for m in (1, 30, 70, 300)] for _ in range(2)]
    _run_on_two_streams(lins, inputs)


@needs_packed
def test_layers_that_split_k_called_from_two_threads_on_their_own_streams():
    """The same with layers whose GEMM splits K through a workspace (few output features, K = 8192) at 1 and 70
    rows: the two threads' calls of ONE layer overlap on the GPU, each stream has a workspace of its own, and
    both get the single-stream bits (FPQ_SPLIT_K at its default)."""
    from fp_quant.module import hip_ops
    assert hip_ops.SPLIT_K
    lins = [_quantized_linear(fmt, g, 8192, 1024, seed=31, bias=True) for fmt, g in (("mxfp4", 128), ("nvfp4", 16))]
    for lin in lins:
        assert getattr(lin.qweight, "_fpq_splitk", None) is not None       # the shape splits
    inputs = [[torch.randn(m, 8192, device="cuda", dtype=torch.bfloat16) for m in (1, 70)] for _ in range(2)]
    before = {k: v.data_ptr() for k, v in hip_ops._stream_workspaces.get(torch.cuda.current_device(), {}).items()}
    _run_on_two_streams(lins, inputs, rounds=60, sync_every_call=False)
    after = hip_ops._stream_workspaces[torch.cuda.current_device()]
    assert len(set(v.data_ptr() for v in after.values()) - set(before.values())) >= 2   # one per worker stream
    torch.cuda.synchronize()
    assert not any(bool(v[:16384].any()) for v in after.values())      # counters left at zero


def _run_on_two_streams(lins, inputs, rounds=25, sync_every_call=True):
    import threading
    with torch.no_grad():
        want = [[[lin(x) for x in xs] for lin in lins] for xs in inputs]
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream), torch.no_grad():
                for _ in range(rounds):
                    got = []
                    for li, lin in enumerate(lins):
                        for xi, x in enumerate(inputs[t]):
                            got.append((li, xi, lin(x)))
                            if sync_every_call:
                                stream.synchronize()
                    stream.synchronize()
                    for li, xi, y in got:
                        if not torch.equal(y, want[t][li][xi]):
                            errors.append((t, li, xi))
        except Exception as exc:   # surfaced below
            errors.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads)
    assert not errors, errors[:5]


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_group_operators_equal_separate_layers(fmt, g):
    """linear_group_w4a4_op (one quantization, one GEMM per layer) and silu_mul_linear_w4a4_op give the
    bits of the layers called one by one -- with biases, for row-major and packed operand paths, and
    whether or not a packed copy of a weight exists yet (a traced call may not create one)."""
    import fp_quant
    from fp_quant.module import eager
    torch.manual_seed(41)
    layers = []
    for n, bias in ((256, True), (128, False), (384, True)):
        lin = fp_quant.FPQuantLinear(512, n, _cfg(fmt, g), bias=bias, device="cuda", dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.normal_(0, 0.05)
            if bias:
                lin.bias.normal_(0, 1)
        lin.pre_forward()
        layers.append(lin)
    down = fp_quant.FPQuantLinear(256, 512, _cfg(fmt, g), bias=True, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        down.weight.normal_(0, 0.05)
        down.bias.normal_(0, 1)
    down.pre_forward()
    nv = fmt == "nvfp4"

    def group(x):
        return eager.linear_group_w4a4_op(x, layers[0].forward_hadamard_matrix, [l.qweight for l in layers],
                                          [l.scales for l in layers], [l.weight_global_scale for l in layers],
                                          [l.act_global_scale for l in layers], [l.bias for l in layers], nv)

    def mlp(gate, up):
        return eager.silu_mul_linear_w4a4_op(gate, up, down.forward_hadamard_matrix, down.qweight, down.scales,
                                             down.weight_global_scale, down.act_global_scale, down.bias, nv)

    with torch.no_grad():
        for round_ in range(2):          # second round: after eager calls have made the packed weights
            for m in (3, 70, 300):
                x = torch.randn(m, 512, device="cuda", dtype=torch.bfloat16)
                got = group(x)
                want = [l(x.clone()) for l in layers]
                assert all(torch.equal(a, b) for a, b in zip(got, want)), (round_, m)
                gate, up = torch.randn(2, m, 256, device="cuda", dtype=torch.bfloat16).unbind(0)
                qa = eager.silu_mul_quantize(gate, up, down.forward_hadamard_matrix, down.act_global_scale, nv)
                assert torch.equal(mlp(gate, up), down.forward_quantized(qa, (m,))), (round_, m)


@pytest.mark.parametrize("fmt,g,m", [("mxfp4", 128, 4), ("mxfp4", 128, 200), ("nvfp4", 16, 100)])
def test_load_state_dict_onto_tensors_without_a_modification_counter(fmt, g, m):
    """A layer built under torch.inference_mode() holds tensors without a modification counter; a
    load_state_dict into it (an in-place copy nothing records) must still reach the packed weights,
    alpha and the other per-tensor copies the layer keeps."""
    import fp_quant
    gen = torch.Generator().manual_seed(77)
    k, n = 512, 256
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16).cuda()

    def make(scale):
        lin = fp_quant.FPQuantLinear(k, n, _cfg(fmt, g), bias=False, device="cuda", dtype=torch.bfloat16)
        lin.weight.data = (torch.randn(n, k, generator=gen) * scale).to(torch.bfloat16).cuda()
        lin.pre_forward()
        return lin

    with torch.inference_mode():
        a, b = make(0.02), make(0.05)
        ya, yb = a(x), b(x)                       # both now hold their packed weights and alpha
        assert not torch.equal(ya, yb)
        sd = {key: v.clone() for key, v in b.state_dict().items()}
        sd["act_global_scale"] = sd["act_global_scale"] * 2   # a different alpha as well: exactly half of b's
        a.load_state_dict(sd)
        if fmt == "mxfp4":
            assert torch.equal(a(x), yb * 0.5)                # same codes, alpha halved (a power of two: exact)
        else:
            assert not torch.equal(a(x), ya)                  # NVFP4 activations are scaled by it before rounding
            c = make(0.02)
            c.load_state_dict(sd)
            assert torch.equal(a(x), c(x))


@needs_packed
@needs_row_major_parameters
@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
@pytest.mark.parametrize("released", [False, True])
def test_recorded_graph_follows_an_in_place_load_state_dict(fmt, g, released):
    """A HIP graph recorded around a layer holds raw pointers to the packed weight and the layer's split-K
    workspace.  load_state_dict (in place) keeps both where they are -- the packed copy is re-packed into its own
    buffers -- so a replay afterwards multiplies by the NEW weights, as the reference, which reads `qweight` in
    place, would."""
    k, n = 8192, 256
    lin = _quantized_linear(fmt, g, k, n, seed=51, bias=True)
    other = _quantized_linear(fmt, g, k, n, seed=52, bias=True)
    sd = {key: v.clone() for key, v in other.state_dict().items()}
    sd["act_global_scale"] = sd["act_global_scale"] * 2          # another alpha (and NVFP4 activation scale) too
    other.load_state_dict(sd)
    if released:
        assert lin.release_row_major()
    x = torch.randn(5, k, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        y_old, y_new = lin(x), other(x)
        assert not torch.equal(y_old, y_new)
        graph = torch.cuda.CUDAGraph()
        static_x = x.clone()
        with torch.cuda.graph(graph):
            static_y = lin(static_x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, y_old)
        workspace = lin.qweight._fpq_splitk.data_ptr()
        packed = (lin.qweight if released else lin.qweight._fpq_packed[1]).data_ptr()
        lin.load_state_dict(other.state_dict())
        assert lin.weights_packed_only == released
        assert lin.qweight._fpq_splitk.data_ptr() == workspace
        assert (lin.qweight if released else lin.qweight._fpq_packed[1]).data_ptr() == packed
        for _ in range(2):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, y_new)
        assert torch.equal(lin(x), y_new)


def test_prepare_device_entry_point():
    from fp_quant import _engine
    lib = _engine.lib()
    s = torch.cuda.Stream()
    assert lib.fpq_prepare_device(s.cuda_stream) == 0
    assert lib.fpq_prepare_device(s.cuda_stream) == 0          # idempotent
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        assert lib.fpq_prepare_device(s.cuda_stream) == _engine.E_UNSUPPORTED   # must run, not be recorded


@needs_packed
@needs_row_major_parameters
@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
@pytest.mark.parametrize("bias", [False, True])
def test_release_row_major_keeps_results_and_the_reference_state_dict(bias, fmt, g):
    """FPQuantLinear.release_row_major: the packed buffers become the only copy of the weight; outputs keep
    their bits on every kernel path (1, 40, 300 and 2100 rows), state_dict() still holds the reference's
    row-major tensors, load_state_dict() accepts them and the layer goes back to the packed layout, and
    restore_row_major gives the original tensors back."""
    k, n = 512, 384
    group = 32 if fmt == "mxfp4" else 16
    lin = _quantized_linear(fmt, g, k, n, seed=5, bias=bias)
    other = _quantized_linear(fmt, g, k, n, seed=6, bias=bias)
    xs = [torch.randn(m, k, device="cuda", dtype=torch.bfloat16) for m in (1, 40, 300, 2100)]
    with torch.no_grad():
        want = [lin(x) for x in xs]
        want_other = [other(x) for x in xs]
        q0, s0 = lin.qweight.detach().clone(), lin.scales.detach().clone()
        keys = list(lin.state_dict().keys())
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        assert lin.release_row_major() and lin.weights_packed_only
        assert lin.qweight.dim() == 1 and lin.qweight.numel() == n * k // 2 and lin.scales.numel() == n * k // group
        torch.cuda.synchronize()
        assert before - torch.cuda.memory_allocated() >= n * k // 2        # the row-major codes are gone
        for x, w in zip(xs, want):
            assert torch.equal(lin(x), w)
        sd = {key: v.clone() for key, v in lin.state_dict().items()}   # (entries alias the live parameters)
        assert sorted(sd.keys()) == sorted(keys)
        assert torch.equal(sd["qweight"], q0) and torch.equal(sd["scales"], s0)
        # traced callers
        torch._dynamo.reset()
        assert torch.equal(torch.compile(lin, fullgraph=True)(xs[1]), want[1])
        torch._dynamo.reset()
        # a checkpoint in the reference's layout loads, and the layer is packed-only again afterwards
        lin.load_state_dict(other.state_dict())
        assert lin.weights_packed_only
        for x, w in zip(xs, want_other):
            assert torch.equal(lin(x), w)
        lin.load_state_dict(sd)
        lin.restore_row_major()
        assert not lin.weights_packed_only
        assert torch.equal(lin.qweight, q0) and torch.equal(lin.scales, s0)
        for x, w in zip(xs, want):
            assert torch.equal(lin(x), w)


def test_release_row_major_declines_what_the_packed_layout_cannot_hold():
    nv = _quantized_linear("nvfp4", 16, 256, 48, seed=1)
    assert not nv.release_row_major() and nv.qweight.dim() == 2
    ragged = _quantized_linear("mxfp4", 32, 256, 48, seed=2)        # 48 output features: not whole 32-row tiles
    assert not ragged.release_row_major() and ragged.qweight.dim() == 2
    short = _quantized_linear("mxfp4", 32, 128, 64, seed=3)         # K = 128: below one 256-K block
    assert not short.release_row_major()
    x = torch.randn(5, 256, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        assert nv(x).shape == (5, 48) and ragged(x).shape == (5, 48)


@needs_packed
def test_single_weight_copy_by_environment(monkeypatch):
    """FPQ_SINGLE_WEIGHT_COPY=1: every eligible layer releases its row-major tensors as soon as it is quantized."""
    monkeypatch.setenv("FPQ_SINGLE_WEIGHT_COPY", "1")
    lin = _quantized_linear("mxfp4", 128, 256, 64, seed=8)
    assert lin.weights_packed_only
    monkeypatch.delenv("FPQ_SINGLE_WEIGHT_COPY")
    plain = _quantized_linear("mxfp4", 128, 256, 64, seed=8)
    assert not plain.weights_packed_only
    x = torch.randn(7, 256, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        assert torch.equal(lin(x), plain(x))
    assert torch.equal(lin.state_dict()["qweight"], plain.qweight)


@pytest.mark.parametrize("fmt,g", [("mxfp4", 128), ("nvfp4", 16)])
def test_empty_batch(fmt, g):
    """No rows: every path returns an empty tensor of the right shape (the C entry points accept zero rows)."""
    lin = _quantized_linear(fmt, g, 256, 96, seed=3, bias=True)
    with torch.no_grad():
        for shape in ((0, 256), (2, 0, 256), (0, 5, 256)):
            y = lin(torch.empty(*shape, device="cuda", dtype=torch.bfloat16))
            assert y.shape == (*shape[:-1], 96) and y.dtype == torch.bfloat16
        if fmt == "mxfp4" and PACKED_WEIGHTS:
            assert lin.release_row_major()
            assert lin(torch.empty(0, 256, device="cuda", dtype=torch.bfloat16)).shape == (0, 96)
