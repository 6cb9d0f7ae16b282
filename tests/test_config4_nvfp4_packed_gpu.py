"""NVFP4 linears of the Qwen3-8B shapes (qkv 6144x4096, o 4096x4096, gate_up 24576x4096, down 4096x12288) at
1, 64, 512 and 4096 rows ON THE KERNELS FPQuantLinear DISPATCHES THERE: the packed-operand kernels
(fpq_gemm_nvf4_packed, and fpq_gemm_nvf4_packed_splitk on the long-K down-projection) at every row
count.  Reference contract: matmul_nvf4_bf16_tn_op
(inference_lib/src/fp_quant/module/qutlass_ops.py:149-168) as forward_gemm calls it (linear_fns.py:53-64).

Every case is checked against the oracle (quantizers + fp64 dequantize-then-matmul, tolerance of
tests/test_gemm_gpu.py) on a seeded sample of rows and columns that contains the corners of the first and
last tiles; the tests name the entry point each case must go through, so a change of dispatch has to be
acknowledged here.
"""
import pytest
import torch

from oracle import fpq_oracle as O
import capi
from conftest import PACKED_WEIGHTS, SINGLE_WEIGHT_COPY, needs_packed, row_major_weights

pytestmark = pytest.mark.gpu

SHAPES = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (24576, 4096), "down": (4096, 12288)}
G = 16
NORM = 0.25   # bf16(16 ** -0.5), exact


def _sample(gen, m, n, rows=20, cols=200):
    ri = torch.cat([torch.tensor([0, m - 1, min(31, m - 1), min(32, m - 1), min(127, m - 1), min(128, m - 1),
                                  min(255, m - 1), min(256, m - 1)]), torch.randperm(m, generator=gen)[:rows]])
    ci = torch.cat([torch.tensor([0, n - 1, 31, 32, 255, 256, n - 257, n - 256, n - 33, n - 32]),
                    torch.randperm(n, generator=gen)[:cols]])
    return ri.unique(), ci.unique()


def _assert_close(y, ref, mag, what):
    err = (y.double() - ref).abs()
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance"
    assert (y == ref.to(torch.bfloat16)).double().mean() > 0.98, what


_weights = {}


def _weight(name):
    """bf16 weight of the shape, seeded; kept for the module's lifetime of this test file."""
    if name not in _weights:
        n, k = SHAPES[name]
        gen = torch.Generator().manual_seed(400 + len(name))
        _weights[name] = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    return _weights[name]


def _layer(name, scales_kind):
    """An NVFP4 FPQuantLinear of the shape.  `default`: what pre_forward gives every abs_max layer (global scales
    3.0).  `ten`: the 10.0 the reference intends for NVFP4 (linear.py:198-200).  `calibrated`: a weight scale
    tracked as the exporter tracks it, 2688 / max|rotated w|, and an activation scale of that form for N(0, 1)
    activations, both rounded to the bf16 buffers as the loader does -- loaded through load_state_dict like a
    realquant checkpoint."""
    import fp_quant
    n, k = SHAPES[name]
    w = _weight(name)
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.NVFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=G)
    lin = fp_quant.FPQuantLinear(k, n, cfg, bias=False, device="cuda", dtype=torch.bfloat16)
    lin.weight.data = w.cuda()
    lin.pre_forward()
    if scales_kind == "default":
        return lin
    if scales_kind == "ten":
        wgs = ags = torch.tensor([10.0], dtype=torch.bfloat16)
    else:
        wgs = torch.tensor([2688.0 / capi.rotated_absmax(w, "hadamard", G)], dtype=torch.bfloat16)
        ags = torch.tensor([2688.0 / 5.25], dtype=torch.bfloat16)
    wq, ws = capi.quantize(w, "nvfp4", "hadamard", G, global_scale=float(wgs))
    sd = lin.state_dict()
    sd = dict(sd, qweight=wq, scales=ws, weight_global_scale=wgs, act_global_scale=ags)
    lin.load_state_dict(sd)
    return lin


class _Calls:
    """Counts the calls FPQuantLinear makes into the library's GEMM entry points."""
    NAMES = ("fpq_gemm_nvf4", "fpq_gemm_nvf4_packed", "fpq_gemm_nvf4_packed_splitk", "fpq_gemm_nvf4_packed_residual")

    def __init__(self, monkeypatch):
        from fp_quant import _engine
        self.seen = []
        lib = _engine.lib()
        for name in self.NAMES:
            real = getattr(lib, name)

            def counted(*args, _real=real, _name=name):
                self.seen.append(_name)
                return _real(*args)

            monkeypatch.setattr(lib, name, counted)


def _expected_entry(name, m, released):
    n, k = SHAPES[name]
    if not PACKED_WEIGHTS:
        return "fpq_gemm_nvf4"
    if name == "down" and m <= 1024:
        # few weight tiles, K = 12288: the entry that may split K through a workspace (the weight-streaming kernel up
        # to 128 rows, its two passes up to 256, the tile kernels beyond)
        return "fpq_gemm_nvf4_packed_splitk"
    return "fpq_gemm_nvf4_packed"


@pytest.mark.parametrize("scales_kind", ["default", "ten", "calibrated"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_module_on_config4_shapes(name, scales_kind, monkeypatch):
    """FPQuantLinear.forward at M = 1, 64, 200, 512 and 4096: weights bit-exact against the oracle, outputs within
    tolerance of the oracle's pipeline, through the entry point the dispatch is documented to take."""
    n, k = SHAPES[name]
    lin = _layer(name, scales_kind)
    released = SINGLE_WEIGHT_COPY
    wgs, ags = float(lin.weight_global_scale), float(lin.act_global_scale)
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    got_q, got_s = row_major_weights(lin)
    w = _weight(name)
    calls = _Calls(monkeypatch)
    for m in (1, 64, 200, 512, 4096):
        gen = torch.Generator().manual_seed(1000 * m + n // 256 + k // 1024)
        x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
        ri, ci = _sample(gen, m, n)
        owq, ows, _ = O.quantize_nv(w[ci], wgs, O.ROT_HADAMARD, G, NORM)
        assert torch.equal(got_q[ci], owq) and torch.equal(got_s[ci], ows)
        oxq, oxs, _ = O.quantize_nv(x[ri], ags, O.ROT_HADAMARD, G, NORM)
        calls.seen.clear()
        with torch.no_grad():
            y = lin(x.cuda())
        assert calls.seen == [_expected_entry(name, m, released)], (name, m, calls.seen)
        assert y.shape == (m, n) and not torch.isnan(y.float()).any()
        ref, mag = O.gemm_ref(oxq, oxs, owq, ows, alpha, "nvfp4")
        _assert_close(y.cpu()[ri][:, ci], ref, mag, f"{name} M={m} {scales_kind}")


@needs_packed
@pytest.mark.parametrize("name,m", [("qkv", 4096), ("gate_up", 512), ("down", 4096)])
def test_released_layer_runs_the_packed_kernels_at_every_row_count(name, m, monkeypatch):
    """A layer that holds its weight in the packed layout only has no row-major operand to fall back on: the
    packed tile kernels take the large batches too (256 x 256 tiles)."""
    n, k = SHAPES[name]
    lin = _layer(name, "ten")
    w = _weight(name)
    gen = torch.Generator().manual_seed(7 * m + n)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    with torch.no_grad():
        want = lin(x.cuda())
        assert lin.release_row_major()
        calls = _Calls(monkeypatch)
        y = lin(x.cuda())
    assert calls.seen == ["fpq_gemm_nvf4_packed"]
    ri, ci = _sample(gen, m, n)
    owq, ows, _ = O.quantize_nv(w[ci], 10.0, O.ROT_HADAMARD, G, NORM)
    oxq, oxs, _ = O.quantize_nv(x[ri], 10.0, O.ROT_HADAMARD, G, NORM)
    ref, mag = O.gemm_ref(oxq, oxs, owq, ows, 0.010009765625, "nvfp4")
    _assert_close(y.cpu()[ri][:, ci], ref, mag, f"released {name} M={m}")
    # (the same kernel ran before the release: the same bits)
    assert torch.equal(want, y)


@pytest.fixture(scope="module")
def packed_operands():
    """Weights of the four shapes quantized (global scale 10) and packed by the parity-checked kernels."""
    out = {}
    for name in SHAPES:
        wq, ws = capi.quantize(_weight(name), "nvfp4", "hadamard", G, global_scale=10.0)
        out[name] = (wq, ws) + capi.pack_nv(wq, ws)
    return out


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("m", [1, 64, 200, 512, 4096])
def test_c_entry_points_on_config4_shapes(name, m, packed_operands):
    """fpq_gemm_nvf4_packed at all sixteen points of the configuration (and 200 rows: the two-pass range), with a
    bias; fpq_gemm_nvf4_packed_splitk with a workspace of the advertised size wherever the library asks for
    one (the down-projection up to 256 rows), leaving its counters at zero and repeating its bits."""
    from fp_quant import _engine
    n, k = SHAPES[name]
    wq, ws, wp, wsp = packed_operands[name]
    gen = torch.Generator().manual_seed(31 * m + n // 128)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    bias = torch.randn(n, generator=gen).to(torch.bfloat16)
    alpha = 0.010009765625
    xq, xs = capi.quantize(x, "nvfp4", "hadamard", G, global_scale=10.0)
    xp, xsp = capi.quantize_nv_packed(x, 10.0, "hadamard", G)
    ri, ci = _sample(gen, m, n)
    oxq, oxs, _ = O.quantize_nv(x[ri], 10.0, O.ROT_HADAMARD, G, NORM)
    assert torch.equal(xq[ri], oxq) and torch.equal(xs[ri], oxs)
    ref, mag = O.gemm_ref(oxq, oxs, wq[ci], ws[ci], alpha, "nvfp4")
    want = (ref.to(torch.bfloat16) + bias[ci]).double()

    def check(y, what):
        got = y[ri][:, ci].double()
        tol = 2.0 ** -7 * torch.maximum(want.abs(), ref.abs()) + 1e-5 * mag + 1e-6
        assert ((got - want).abs() <= tol).all(), what
        assert (got == want).double().mean() > 0.97, what

    y = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=bias)
    assert not torch.isnan(y.float()).any()
    check(y, f"{name} M={m} fpq_gemm_nvf4_packed")
    need = int(_engine.lib().fpq_gemm_nvf4_packed_workspace_bytes(m, n, k))
    if need > 0:
        workspace = torch.zeros(need, dtype=torch.uint8, device="cuda")
        ys = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=bias, workspace=workspace, nv=True)
        check(ys, f"{name} M={m} fpq_gemm_nvf4_packed_splitk")
        assert not workspace[:16384].any()
        again = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=bias, workspace=workspace, nv=True)
        assert torch.equal(ys.view(torch.int16), again.view(torch.int16))
    elif name == "down" and m <= 256:
        # (beyond 256 rows the tile kernel halves this K inside its workgroups and needs no workspace)
        raise AssertionError("the down-projection shape is expected to split K")
