"""Parity of the W4A4 GEMM kernels against the oracle's fp64 dequantize-then-matmul.

Stated tolerance (the reference states none): every product of two dequantized operands is
exact in fp32, so the kernel differs from the fp64 result only by fp32 accumulation order and
the final bf16 rounding:  |y - ref| <= 2^-8 * |ref| + 1e-5 * alpha * sum_k |dq(x)||dq(w)|.
"""
import pytest
import torch

from oracle import fpq_oracle as O

pytestmark = pytest.mark.gpu

TOL_REL = 2.0 ** -8
TOL_MAG = 1e-5


def _operands(m, n, k, fmt, seed, g=None):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    if fmt == "mxfp4":
        g = g or (128 if k % 128 == 0 else 32)
        xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, g)
        wq, ws, _ = O.quantize_mx(w, O.ROT_HADAMARD, g)
        alpha = 0.111328125  # bf16(1/9)
    else:
        g = g or 16
        xq, xs, _ = O.quantize_nv(x, 10.0, O.ROT_HADAMARD, g)
        wq, ws, _ = O.quantize_nv(w, 10.0, O.ROT_HADAMARD, g)
        alpha = 0.010009765625  # bf16(1/100)
    return xq, xs, wq, ws, alpha


def _assert_close(y, ref, mag, what=""):
    err = (y.double() - ref).abs()
    tol = TOL_REL * ref.abs() + TOL_MAG * mag
    bad = err > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, worst excess {float((err - tol).max())}"


@pytest.mark.parametrize("fmt", ["mxfp4", "nvfp4"])
@pytest.mark.parametrize("m,n,k", [
    (1, 16, 32), (1, 64, 128), (3, 48, 96), (16, 128, 256), (17, 130, 384), (33, 257, 512),
    (64, 64, 4096), (100, 200, 160), (130, 96, 1024), (256, 256, 256),
])
def test_gemm_small_shapes(fmt, m, n, k):
    import capi
    xq, xs, wq, ws, alpha = _operands(m, n, k, fmt, seed=m * 1000 + n + k)
    y = capi.gemm(xq, xs, wq, ws, alpha, fmt)
    assert not torch.isnan(y.float()).any()
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, fmt)
    _assert_close(y, ref, mag, f"{fmt} {m}x{n}x{k}")
    exact = (y == ref.to(torch.bfloat16)).float().mean().item()
    assert exact > 0.98, f"only {exact:.4f} of outputs equal bf16(ref)"


@pytest.mark.parametrize("fmt", ["mxfp4", "nvfp4"])
def test_gemm_scales_are_applied_per_block(fmt):
    """Scale bytes that differ wildly between neighbouring K blocks and rows: a kernel that
    pairs a scale with the wrong 32 (16) values cannot pass."""
    import capi
    m, n, k = 32, 48, 512
    gen = torch.Generator().manual_seed(77)
    group = 32 if fmt == "mxfp4" else 16
    xq = torch.randint(0, 256, (m, k // 2), generator=gen, dtype=torch.uint8)
    wq = torch.randint(0, 256, (n, k // 2), generator=gen, dtype=torch.uint8)
    if fmt == "mxfp4":
        xs = torch.randint(117, 138, (m, k // group), generator=gen, dtype=torch.uint8)
        ws = torch.randint(117, 138, (n, k // group), generator=gen, dtype=torch.uint8)
    else:
        xs = torch.randint(1, 0x60, (m, k // group), generator=gen, dtype=torch.uint8)
        ws = torch.randint(1, 0x60, (n, k // group), generator=gen, dtype=torch.uint8)
    y = capi.gemm(xq, xs, wq, ws, 1.0, fmt)
    ref, mag = O.gemm_ref(xq, xs, wq, ws, 1.0, fmt)
    _assert_close(y, ref, mag, fmt)


@pytest.mark.parametrize("fmt", ["mxfp4", "nvfp4"])
def test_gemm_bias_matches_separate_bf16_add(fmt):
    import capi
    xq, xs, wq, ws, alpha = _operands(40, 136, 256, fmt, seed=5)
    bias = torch.randn(136, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    y0 = capi.gemm(xq, xs, wq, ws, alpha, fmt)
    y1 = capi.gemm(xq, xs, wq, ws, alpha, fmt, bias=bias)
    assert torch.equal(y1, y0 + bias)  # the reference adds the bias to the bf16 GEMM result


def test_gemm_padded_activation_scales():
    """The quantize operator pads activation scales to 128 rows / 4 columns; the GEMM reads
    them with that row stride."""
    import capi
    m, n, k = 5, 64, 96
    xq, xs, wq, ws, alpha = _operands(m, n, k, "mxfp4", seed=8, g=32)
    xs_pad = torch.zeros(128, 4, dtype=torch.uint8)
    xs_pad[:m, : k // 32] = xs
    y = capi.gemm(xq, xs_pad, wq, ws, alpha, "mxfp4")
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "mxfp4")
    _assert_close(y, ref, mag)


def _big_case(fmt, m, n, k, seed, rows=48, cols=384):
    """Operands quantized on the GPU (kernel already parity-checked), GEMM compared with the
    oracle on a seeded sample of output rows and columns."""
    import capi
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    if fmt == "mxfp4":
        xq, xs = capi.quantize(x, fmt, "hadamard", 128)
        wq, ws = capi.quantize(w, fmt, "hadamard", 128)
        alpha = 0.111328125
    else:
        xq, xs = capi.quantize(x, fmt, "hadamard", 16, global_scale=10.0)
        wq, ws = capi.quantize(w, fmt, "hadamard", 16, global_scale=10.0)
        alpha = 0.010009765625
    y = capi.gemm(xq, xs, wq, ws, alpha, fmt)
    assert not torch.isnan(y.float()).any()
    ri = torch.randperm(m, generator=gen)[: min(rows, m)]
    ci = torch.randperm(n, generator=gen)[: min(cols, n)]
    ref, mag = O.gemm_ref(xq[ri], xs[ri], wq[ci], ws[ci], alpha, fmt)
    _assert_close(y[ri][:, ci], ref, mag, f"{fmt} {m}x{n}x{k}")
    # size-independent property: rows of y only depend on their own row of x
    if m > 1:
        y_row = capi.gemm(xq[ri[:1]], xs[ri[:1]], wq, ws, alpha, fmt)
        assert torch.equal(y_row[0], y[ri[0]])


@pytest.mark.parametrize("m", [1, 16, 128, 2048])
def test_config3_mxfp4_llama_mlp_shape(m):
    _big_case("mxfp4", m, 14336, 4096, seed=30 + m)


@pytest.mark.parametrize("n,k", [(6144, 4096), (4096, 4096), (24576, 4096), (4096, 12288)])
@pytest.mark.parametrize("m", [1, 64, 512, 4096])
def test_config4_nvfp4_qwen3_shapes(m, n, k):
    _big_case("nvfp4", m, n, k, seed=40 + m + n // 1024, rows=24, cols=256)


def test_gemm_rejects_bad_arguments():
    import capi
    xq = torch.zeros(4, 24, dtype=torch.uint8)   # K = 48: not a multiple of 32
    wq = torch.zeros(8, 24, dtype=torch.uint8)
    s = torch.zeros(8, 4, dtype=torch.uint8)
    with pytest.raises(ValueError):
        capi.gemm(xq, s, wq, s, 1.0, "mxfp4")
    xq = torch.zeros(4, 64, dtype=torch.uint8)
    wq = torch.zeros(8, 64, dtype=torch.uint8)
    with pytest.raises(ValueError):
        capi.gemm(xq, s[:, :2], wq, s, 1.0, "mxfp4")  # scale stride smaller than K/32
