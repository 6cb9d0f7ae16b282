"""Parity of the packed GEMM instantiations that only large problems reach.

fpq_gemm_mxf4_packed / fpq_gemm_nvf4_packed pick their big-tile kernels (256-row weight tiles, the
short operand ring with its own prologue and drain) once the problem has at least 100 tiles of
256 x 256; FPQuantLinear.forward runs exactly that kernel on the Llama MLP shape at 2048 rows.  Every
case here is above that threshold and is checked against the oracle's fp64 dequantize-then-matmul
(tolerance of tests/test_gemm_gpu.py) and, for MXFP4, bit for bit against the row-major kernel, which
issues the same matrix instructions per output in the same K order.
"""
import pytest
import torch

from oracle import fpq_oracle as O
import capi
from conftest import needs_packed, packed_copy, row_major_weights
from test_packed_gpu import pack_by_definition, pack_nv_by_definition

pytestmark = pytest.mark.gpu

TOL_REL = 2.0 ** -8
TOL_MAG = 1e-5
ALPHA_MX = 0.111328125  # bf16(1/9)


def big_tiles(m, n):
    return ((m + 255) // 256) * ((n + 255) // 256)


def _assert_close(y, ref, mag, what="", rel=TOL_REL):
    err = (y.double() - ref).abs()
    tol = rel * ref.abs() + TOL_MAG * mag + 1e-6
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance"


def _sample(gen, m, n, rows=64, cols=512):
    """Seeded rows and columns that always include the corners of the first and last tiles."""
    ri = torch.cat([torch.tensor([0, m - 1, min(255, m - 1), min(256, m - 1)]), torch.randperm(m, generator=gen)[:rows]])
    ci = torch.cat([torch.tensor([0, n - 1, min(255, n - 1), min(256, n - 1)]), torch.randperm(n, generator=gen)[:cols]])
    return ri.unique(), ci.unique()


@pytest.fixture(scope="module")
def c3_operands():
    """The Llama-3-8B up/gate shape at 2048 rows, quantized by the (parity-checked) GPU quantizers."""
    gen = torch.Generator().manual_seed(3)
    m, n, k = 2048, 14336, 4096
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    xq, xs = capi.quantize(x, "mxfp4", "hadamard", 128)
    wq, ws = capi.quantize(w, "mxfp4", "hadamard", 128)
    xp, xsp = capi.quantize_packed(x, g=128)          # what FPQuantLinear feeds the kernel
    wp, wsp = capi.pack(wq, ws)
    bias = torch.randn(n, generator=gen).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=gen) * 4).to(torch.bfloat16)
    return dict(m=m, n=n, k=k, x=x, w=w, xq=xq, xs=xs, wq=wq, ws=ws, xp=xp, xsp=xsp, wp=wp, wsp=wsp, bias=bias,
                res=res, gen=gen)


@pytest.mark.parametrize("bias", [False, True])
def test_c3_m2048_packed_gemm_matches_oracle_and_row_major(c3_operands, bias):
    c = c3_operands
    m, n, k = c["m"], c["n"], c["k"]
    assert big_tiles(m, n) >= 100
    b = c["bias"] if bias else None
    y = capi.gemm_packed(c["xp"], c["xsp"], c["wp"], c["wsp"], m, n, k, ALPHA_MX, bias=b)
    assert not torch.isnan(y.float()).any()
    ri, ci = _sample(torch.Generator().manual_seed(17), m, n)
    ref, mag = O.gemm_ref(c["xq"][ri], c["xs"][ri], c["wq"][ci], c["ws"][ci], ALPHA_MX, "mxfp4")
    if bias:
        _assert_close(y[ri][:, ci], (ref.to(torch.bfloat16) + b[ci]).double(), mag, "C3 M=2048 packed + bias", rel=2.0 ** -7)
    else:
        _assert_close(y[ri][:, ci], ref, mag, "C3 M=2048 packed")
    y_rm = capi.gemm(c["xq"], c["xs"], c["wq"], c["ws"], ALPHA_MX, "mxfp4", bias=b)
    assert torch.equal(y.view(torch.int16), y_rm.view(torch.int16))


@pytest.mark.parametrize("bias", [False, True])
def test_c3_m2048_packed_residual_epilogue(c3_operands, bias):
    c = c3_operands
    m, n, k = c["m"], c["n"], c["k"]
    b = c["bias"] if bias else None
    plain = capi.gemm_packed(c["xp"], c["xsp"], c["wp"], c["wsp"], m, n, k, ALPHA_MX, bias=b)
    got = capi.gemm_packed(c["xp"], c["xsp"], c["wp"], c["wsp"], m, n, k, ALPHA_MX, bias=b, residual=c["res"])
    assert torch.equal(got.view(torch.int16), (plain + c["res"]).view(torch.int16))
    got = capi.gemm_packed(c["xp"], c["xsp"], c["wp"], c["wsp"], m, n, k, ALPHA_MX, bias=b, residual=c["res"],
                           in_place=True)
    assert torch.equal(got.view(torch.int16), (plain + c["res"]).view(torch.int16))


@needs_packed
def test_c3_m2048_through_module(c3_operands, monkeypatch):
    """FPQuantLinear.forward on the shape the headline is measured on: packed weights, packed
    activations, big-tile kernel; against the oracle's quantizers + fp64 GEMM and against the module
    with the row-major kernels."""
    import fp_quant
    c = c3_operands
    m, n, k = c["m"], c["n"], c["k"]
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=128)
    lin = fp_quant.FPQuantLinear(k, n, cfg, bias=True, device="cuda", dtype=torch.bfloat16)
    lin.weight.data = c["w"].cuda()
    lin.bias.data = c["bias"].cuda()
    lin.pre_forward()
    assert torch.equal(row_major_weights(lin)[0], c["wq"])
    y = lin(c["x"].cuda()).cpu()
    assert packed_copy(lin) is not None
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    ri, ci = _sample(torch.Generator().manual_seed(18), m, n, rows=32, cols=256)
    norm = float(O.hadamard_matrix(128)[0, 0])
    oxq, oxs, _ = O.quantize_mx(c["x"][ri], O.ROT_HADAMARD, 128, norm)
    owq, ows, _ = O.quantize_mx(c["w"][ci], O.ROT_HADAMARD, 128, norm)
    ref, mag = O.gemm_ref(oxq, oxs, owq, ows, alpha, "mxfp4")
    want = ref.to(torch.bfloat16) + c["bias"][ci]
    _assert_close(y[ri][:, ci], want.double(), mag, "FPQuantLinear C3 M=2048", rel=2.0 ** -7)
    monkeypatch.setenv("FPQ_PACKED_WEIGHTS", "0")
    y_rm = lin(c["x"].cuda()).cpu()
    assert torch.equal(y.view(torch.int16), y_rm.view(torch.int16))


# Ragged shapes with at least 100 big tiles; K of one, two, three and five 256-blocks runs the short
# ring's prologue with fewer units than slots, its drain, and the steady state for one block.
RAGGED = [(2500, 2570, 256), (2500, 2570, 512), (2049, 3330, 768), (2300, 2817, 1280), (2561, 2564, 512)]


@pytest.mark.parametrize("m,n,k", RAGGED)
@pytest.mark.parametrize("bias", [False, True])
def test_ragged_large_mx_packed(m, n, k, bias):
    assert big_tiles(m, n) >= 100
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    b = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    y = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA_MX, bias=b)
    assert not torch.isnan(y.float()).any()
    ref, mag = O.gemm_ref(xq, xs, wq, ws, ALPHA_MX, "mxfp4")
    want = ref.to(torch.bfloat16)
    if bias:
        want = want + b
    _assert_close(y, want.double(), mag, f"mx {m}x{n}x{k}", rel=2.0 ** -7)
    y_rm = capi.gemm(xq, xs, wq, ws, ALPHA_MX, "mxfp4", bias=b)
    assert torch.equal(y.view(torch.int16), y_rm.view(torch.int16))
    if not bias:
        res = (torch.randn(m, n, generator=g) * 20).to(torch.bfloat16)
        got = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA_MX, residual=res)
        assert torch.equal(got.view(torch.int16), (y + res).view(torch.int16))


@pytest.mark.parametrize("m,n,k", [(2500, 2570, 256), (2500, 2570, 512), (2049, 3330, 1024), (2561, 2564, 768)])
@pytest.mark.parametrize("bias", [False, True])
def test_ragged_large_nv_packed(m, n, k, bias):
    """fpq_gemm_nvf4_packed above the tile threshold (256 x 256 tiles, full ring)."""
    assert big_tiles(m, n) >= 100
    g = torch.Generator().manual_seed(m + 2 * n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(1, 0x7f, (m, k // 16), dtype=torch.uint8, generator=g)
    ws = torch.randint(24, 72, (n, k // 16), dtype=torch.uint8, generator=g)
    b = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    alpha = 2.0 ** -6
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    y = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b)
    assert not torch.isnan(y.float()).any()
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "nvfp4")
    want = ref.to(torch.bfloat16)
    if bias:
        want = want + b
    tol = (2.0 if bias else 1.0) * 2.0 ** -7 * torch.maximum(want.double().abs(), ref.abs()) + 1e-5 * mag + 1e-6
    assert ((y.double() - want.double()).abs() <= tol).all()
    assert (y.view(torch.int16) == want.view(torch.int16)).double().mean() > 0.97


def test_nv_packed_large_llama_shape():
    """NVFP4 packed kernel on quantized (not random) operands at 2048 x 14336 x 4096."""
    gen = torch.Generator().manual_seed(9)
    m, n, k = 2048, 14336, 4096
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    xq, xs = capi.quantize(x, "nvfp4", "hadamard", 16, global_scale=10.0)
    wq, ws = capi.quantize(w, "nvfp4", "hadamard", 16, global_scale=10.0)
    xp, xsp = capi.pack_nv(xq, xs)
    wp, wsp = capi.pack_nv(wq, ws)
    alpha = 0.010009765625
    y = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha)
    ri, ci = _sample(gen, m, n, rows=32, cols=256)
    ref, mag = O.gemm_ref(xq[ri], xs[ri], wq[ci], ws[ci], alpha, "nvfp4")
    _assert_close(y[ri][:, ci], ref, mag, "nv packed 2048x14336x4096")


@pytest.mark.parametrize("m", [16, 64, 128])
def test_vocabulary_sized_output(m):
    """A vocabulary-sized N (4008 weight tiles; an `lm_head` if someone quantizes it) on the weight-streaming
    kernel with one and with two weight tiles per workgroup, and on the tile kernel: a sample of columns that
    includes the last ones, against the oracle."""
    n, k = 128256, 512
    g = torch.Generator().manual_seed(m)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = capi.pack(wq, ws)
    y = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA_MX)
    assert not torch.isnan(y.float()).any()
    ci = torch.cat([torch.tensor([0, 31, 32, 63, 64, n - 65, n - 64, n - 33, n - 32, n - 1]),
                    torch.randperm(n, generator=g)[:1024]]).unique()
    ref, mag = O.gemm_ref(xq, xs, wq[ci], ws[ci], ALPHA_MX, "mxfp4")
    _assert_close(y[:, ci], ref, mag, f"N = {n}, M = {m}")
