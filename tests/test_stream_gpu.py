"""The weight-streaming packed MXFP4 GEMM (at most 128 activation rows): K whole, and K split across
workgroups through a workspace (fpq_gemm_mxf4_packed_splitk), against the oracle's fp64
dequantize-then-matmul with the tolerance of tests/test_gemm_gpu.py."""
import pytest
import torch

from oracle import fpq_oracle as O
from fp_quant import _engine
import capi
from test_packed_gpu import pack_by_definition

pytestmark = pytest.mark.gpu

ALPHA = 0.111328125


def _operands(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    return g, xq, xs, wq, ws


def _check(y, xq, xs, wq, ws, bias=None, residual=None):
    ref, mag = O.gemm_ref(xq, xs, wq, ws, ALPHA, "mxfp4")
    assert not torch.isnan(y.float()).any()
    if bias is None and residual is None:
        tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
        assert ((y.double() - ref).abs() <= tol).all()
        assert (y == ref.to(torch.bfloat16)).float().mean() > 0.98
        return
    want = ref.to(torch.bfloat16)
    if bias is not None:
        want = want + bias
    if residual is not None:
        want = want + residual
    # each further bf16 addition is one more rounding of a value that may differ by one ulp
    tol = 2.0 ** -6 * torch.maximum(want.double().abs(), ref.abs()) + 1e-5 * mag + 1e-6
    if residual is not None:
        tol = tol + 2.0 ** -7 * residual.double().abs()
    assert ((y.double() - want.double()).abs() <= tol).all()


def _workspace(m, n, k, cap=None):
    need = _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes(m, n, k)
    size = need if cap is None else min(need, cap)
    return need, torch.zeros(max(size, 256), dtype=torch.uint8, device="cuda")


# one to four activation row tiles (65-96 rows with at most 512 weight tiles, 97-128 rows with at most 256;
# the shapes just beyond run the tile kernels and meet the same oracle), odd tile counts, ragged rows and
# columns, one to 56 blocks of K
SHAPES = [(1, 32, 256), (1, 100, 512), (5, 257, 768), (16, 1024, 1024), (31, 64, 1280), (32, 4096, 4096),
          (33, 130, 2048), (64, 96, 3072), (70, 515, 1024), (96, 2048, 4096), (100, 36, 256), (128, 1000, 2304),
          (127, 4099, 1536), (8, 1024, 14336), (64, 8200, 512), (40, 8290, 768), (33, 16384, 256),
          # 768 weight tiles or more at 33-64 rows: two weight tiles per workgroup (an odd tile count, a ragged N)
          (64, 24600, 512), (45, 28672, 256), (33, 24577, 256),
          # three activation row tiles with more than 256 weight tiles, up to the limit and past it
          (96, 8290, 512), (70, 14336, 256), (96, 16384, 256), (65, 16416, 256), (96, 32768, 256), (128, 8192, 256), (128, 8224, 256)]
# shapes whose K is split when a workspace is given (few weight tiles, K of 8192 or more), one to four
# activation row tiles
SPLIT_SHAPES = [(1, 32, 8192), (5, 257, 12288), (16, 1024, 8192), (31, 64, 16384), (32, 4096, 8192),
                (8, 1024, 14336), (17, 515, 9216), (33, 4096, 8192), (64, 515, 9216), (96, 64, 16384),
                (128, 1024, 8192), (100, 2050, 12288)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_stream_whole_k_matches_oracle(m, n, k):
    g, xq, xs, wq, ws = _operands(m, n, k, m * 7 + n + k)
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    y = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA)
    _check(y, xq, xs, wq, ws)
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    yb = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=b)
    assert torch.equal(yb, y + b)                       # the reference's separate bf16 `y += bias`
    res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
    yr = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=b, residual=res)
    assert torch.equal(yr, yb + res)                    # and a separate bf16 residual add
    yr2 = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=b, residual=res, in_place=True)
    assert torch.equal(yr2, yr)


@pytest.mark.parametrize("m,n,k", SPLIT_SHAPES + [(16, 1024, 1024), (64, 96, 3072)])
def test_stream_split_k_matches_oracle_and_is_deterministic(m, n, k):
    g, xq, xs, wq, ws = _operands(m, n, k, m * 11 + n + k)
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    need, wspace = _workspace(m, n, k)
    assert (need > 16384) == ((m, n, k) in SPLIT_SHAPES)
    y = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, workspace=wspace)
    _check(y, xq, xs, wq, ws)
    assert int(wspace[:16384].max()) == 0               # counters are left at zero
    # the same bits whatever order the parts arrive in, call after call on a used workspace
    again = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, workspace=wspace, calls=5)
    assert torch.equal(again.view(torch.int16), y.view(torch.int16))
    assert int(wspace[:16384].max()) == 0
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
    yr = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=b, residual=res, workspace=wspace)
    assert torch.equal(yr, (y + b) + res)
    if need:
        # a workspace too small for the preferred split means fewer parts, never an error
        _, small = _workspace(m, n, k, cap=16384 + 2 * ((n + 31) // 32) * 4096)
        ys = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, workspace=small)
        _check(ys, xq, xs, wq, ws)
    # without a workspace the entry point is fpq_gemm_mxf4_packed
    y0 = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA)
    assert torch.equal(y0, capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA))


@pytest.mark.parametrize("m,n,k", [(1, 32, 8192), (16, 1024, 8192), (31, 64, 16384), (17, 515, 9216), (16, 1024, 1024)])
def test_nvfp4_split_k_matches_oracle_and_is_deterministic(m, n, k):
    """fpq_gemm_nvf4_packed_splitk: the same split, exchange and fixed summation order on NVFP4 operands."""
    from test_packed_gpu import pack_nv_by_definition
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(0x20, 0x50, (m, k // 16), dtype=torch.uint8, generator=g)
    ws = torch.randint(0x20, 0x50, (n, k // 16), dtype=torch.uint8, generator=g)
    alpha = 2.0 ** -6
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    need, wspace = _workspace(m, n, k)
    y = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, workspace=wspace, nv=True)
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "nvfp4")
    assert not torch.isnan(y.float()).any()
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6).all()
    assert int(wspace[:16384].max()) == 0
    again = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, workspace=wspace, calls=4, nv=True)
    assert torch.equal(again.view(torch.int16), y.view(torch.int16)) and int(wspace[:16384].max()) == 0
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
    yr = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res, workspace=wspace, nv=True)
    assert torch.equal(yr, (y + b) + res)
    y0 = capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, alpha, nv=True)     # no workspace: the plain entry
    assert torch.equal(y0, capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha))


@pytest.mark.parametrize("m,n,k", [(64, 24576, 512), (40, 17000, 768), (33, 20480, 256), (64, 16416, 1280)])
def test_nvfp4_three_weight_tiles_per_workgroup(m, n, k):
    """NVFP4 at 33-64 rows with 513-768 weight tiles (a whole number of groups of three, a ragged N whose last
    group holds one tile, one block of K so that three of the four waves have nothing to multiply): rows sampled
    against the oracle, bias and residual as separate bf16 additions, the same bits on a second call."""
    from test_packed_gpu import pack_nv_by_definition
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(0x20, 0x50, (m, k // 16), dtype=torch.uint8, generator=g)
    ws = torch.randint(0x20, 0x50, (n, k // 16), dtype=torch.uint8, generator=g)
    alpha = 2.0 ** -6
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    y = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha)
    assert not torch.isnan(y.float()).any()
    ci = torch.cat([torch.tensor([0, 31, 32, 95, 96, n - 97, n - 33, n - 1]), torch.randperm(n, generator=g)[:600]]).unique()
    ref, mag = O.gemm_ref(xq, xs, wq[ci], ws[ci], alpha, "nvfp4")
    assert ((y[:, ci].double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6).all()
    assert (y[:, ci] == ref.to(torch.bfloat16)).float().mean() > 0.98
    assert torch.equal(capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha).view(torch.int16), y.view(torch.int16))
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
    assert torch.equal(capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res), (y + b) + res)


def test_split_k_is_taken_for_few_weight_rows_and_long_k():
    need = _engine.lib().fpq_gemm_mxf4_packed_workspace_bytes
    assert need(16, 4096, 14336) == 16384 + 2 * 128 * 4096   # 128 weight tiles, 56 blocks: two parts
    assert need(16, 1024, 14336) == 16384 + 3 * 32 * 4096    # 32 weight tiles: three parts of 4864
    assert need(16, 4096, 4096) == 0                         # a part would be shorter than 4096
    assert need(16, 14336, 4096) == 0                        # 448 weight tiles fill the chip
    assert need(33, 4096, 14336) == 16384 + 2 * 128 * 2 * 4096   # two activation row tiles: partial tiles twice as many
    assert need(128, 4096, 14336) == 16384 + 2 * 128 * 4 * 4096  # four: 4 MB, the most a split ever needs
    assert need(96, 16384, 14336) == 0                       # 512 weight tiles: K stays whole at every row count
    assert need(129, 4096, 14336) == 0                       # tile kernels above 128 rows
    assert need(16, 4096, 256) == 0                          # one block of K: nothing to split


@pytest.mark.parametrize("m", [1, 16, 128])
def test_config3_small_m_on_packed_operands(m):
    """The benchmark linear (weight [14336, 4096], Hadamard 128) at M = 1, 16, 128 on the kernel FPQuantLinear runs for those rows."""
    gen = torch.Generator().manual_seed(50 + m)
    n, k = 14336, 4096
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    xq, xs = capi.quantize(x, "mxfp4", "hadamard", 128)
    wq, ws = capi.quantize(w, "mxfp4", "hadamard", 128)
    xp, xsp = capi.quantize_packed(x, g=128)
    wp, wsp = capi.pack(wq, ws)
    ci = torch.randperm(n, generator=gen)[:512]
    ref, mag = O.gemm_ref(xq, xs, wq[ci], ws[ci], ALPHA, "mxfp4")
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
    _, wspace = _workspace(m, n, k)
    for y in (capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA),
              capi.gemm_packed_splitk(xp, xsp, wp, wsp, m, n, k, ALPHA, workspace=wspace)):
        assert ((y[:, ci].double() - ref).abs() <= tol).all()


def test_split_k_rejects_misaligned_workspace():
    g, xq, xs, wq, ws = _operands(4, 64, 1024, 3)
    xp, xsp = pack_by_definition(xq, xs, 1024)
    wp, wsp = pack_by_definition(wq, ws, 1024)
    wspace = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        capi.gemm_packed_splitk(xp, xsp, wp, wsp, 4, 64, 1024, ALPHA, workspace=wspace[16:])


# rows that take the weight-streaming kernel with one and with two activation row tiles, the
# 128 x 128 tile kernel and the 256 x 128 tile kernel; 2 to 4 layers of 256 to 1024 output features
@pytest.mark.parametrize("m,splits,k", [(1, [512, 256, 256], 512), (16, [1024, 256], 1024), (33, [256, 512], 256),
                                        (64, [4096, 4096, 256], 256), (128, [256, 256, 256, 256], 768),
                                        (300, [512, 256, 256], 512), (2048, [2048, 1024, 256, 768], 256),
                                        (37, [9216], 256), (64, [14336, 14336], 256), (40, [12288, 256, 12288], 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_layers_end_to_end_get_their_own_outputs(m, splits, k, with_bias):
    """fpq_gemm_mxf4_packed_multi: every layer's matrix equals its column range of the one-output GEMM
    on the same operands bit for bit (same kernels, same accumulation order), and that GEMM is checked
    against the oracle."""
    n = sum(splits)
    g, xq, xs, wq, ws = _operands(m, n, k, 4000 + m + n)
    bias = (torch.randn(n, generator=g) * 2).to(torch.bfloat16) if with_bias else None
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    whole = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, ALPHA, bias=bias)
    _check(whole, xq, xs, wq, ws, bias=bias)
    outs = capi.gemm_packed_multi(xp, xsp, wp, wsp, m, splits, k, ALPHA, bias=bias)
    col = 0
    for o, s in zip(outs, splits):
        assert o.shape == (m, s)
        assert torch.equal(o.view(torch.int16), whole[:, col:col + s].contiguous().view(torch.int16))
        col += s
