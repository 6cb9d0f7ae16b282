"""Packed MXFP4 operand layout: the re-tiling kernel, the quantizer that writes it directly and
the GEMM that reads it, each against an index-level restatement of the layout and the oracle."""
import pytest
import torch

from oracle import fpq_oracle as O
from fp_quant import _engine
import capi
from conftest import make_outlier_normal, needs_packed, needs_row_major_parameters, packed_copy

pytestmark = pytest.mark.gpu


def pack_by_definition(codes, scales, k):
    """The layout as include/fpq.h states it, written with reshapes (rows padded with zeros):
    codes  [(rt, ks), (kh, r), 16 bytes] = row 32 rt + r, bytes 32 ks + 16 kh ...
    scales [(rt, kb), (kh, r), q]        = row 32 rt + r, group 8 kb + 2 q + kh"""
    rows = codes.shape[0]
    rt = (rows + 31) // 32
    c = torch.zeros(rt * 32, k // 2, dtype=torch.uint8)
    c[:rows] = codes[:, : k // 2]
    s = torch.zeros(rt * 32, k // 32, dtype=torch.uint8)
    s[:rows] = scales[:rows, : k // 32]
    pc = c.view(rt, 32, k // 64, 2, 16).permute(0, 2, 3, 1, 4).contiguous().view(-1)
    ps = s.view(rt, 32, k // 256, 4, 2).permute(0, 2, 4, 1, 3).contiguous().view(-1)
    return pc, ps


@pytest.mark.parametrize("rows,k", [(32, 256), (64, 512), (33, 256), (100, 1024), (257, 768)])
def test_pack_kernel_matches_definition(rows, k):
    g = torch.Generator().manual_seed(rows + k)
    codes = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, generator=g)
    scales = torch.randint(0, 256, (rows + 3, k // 32 + 4), dtype=torch.uint8, generator=g)  # padded tensor
    pc, ps = capi.pack(codes, scales)
    wc, ws = pack_by_definition(codes, scales, k)
    assert torch.equal(pc, wc)
    assert torch.equal(ps, ws)


def test_pack_rejects():
    codes = torch.zeros(32, 64, dtype=torch.uint8)
    scales = torch.zeros(32, 4, dtype=torch.uint8)
    with pytest.raises(ValueError):
        capi.pack(codes, scales)  # K = 128 is not a multiple of 256


CASES = [("hadamard", 128), ("hadamard", 64), ("hadamard", 32), ("hadamard", 16), ("identity", 32),
         ("gsr", 64), ("gsr", 32), ("gsr", 16)]


@pytest.mark.parametrize("rot,g", CASES)
@pytest.mark.parametrize("policy", [_engine.ZERO_REFERENCE, _engine.ZERO_SIGNED])
@pytest.mark.parametrize("rows", [70, 1, 13, 24, 64, 65])   # up to 64 rows: the generic kernel writes the packed layout
def test_quantize_packed_bit_exact(rot, g, policy, rows):
    cols = 512  # 70 rows: ragged last row tile
    x = make_outlier_normal(rows, cols, 11 * g + len(rot))
    x[3 % rows, 64:96] = 0.0     # a zero group
    x[5 % rows, :32] = -0.0
    if rows > 9:
        x[7] *= 2.0 ** -110      # exponents outside the fast range
        x[9] *= 2.0 ** 105
    okind = {"hadamard": O.ROT_HADAMARD, "identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR}[rot]
    norm = float(O.hadamard_matrix(g)[0, 0])
    wc, ws, _ = O.quantize_mx(x, okind, g, norm, zero_nibble=policy)
    want_c, want_s = pack_by_definition(wc, ws, cols)
    pc, ps = capi.quantize_packed(x, rot=rot, g=g, norm=norm, zero_policy=policy)
    assert torch.equal(pc, want_c)
    assert torch.equal(ps, want_s)


def test_quantize_packed_large_matches_row_major_path():
    """Full-size activation block: the packed quantizer equals re-tiling the row-major one."""
    gen = torch.Generator().manual_seed(5)
    x = (torch.randn(2048, 4096, generator=gen) * 3).to(torch.bfloat16)
    rc, rs = capi.quantize(x, "mxfp4", g=128)
    want_c, want_s = pack_by_definition(rc, rs, 4096)
    pc, ps = capi.quantize_packed(x, g=128)
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)


def test_quantize_packed_rejects():
    x = torch.zeros(32, 384, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        capi.quantize_packed(x, g=128)                       # cols % 256 != 0
    with pytest.raises(ValueError):
        capi.quantize_packed(torch.zeros(32, 512, dtype=torch.bfloat16), rot="gsr", g=128)


# row slabs of the weight-streaming kernel while slabs x weight tiles stay within 256 (a short last slab, one
# with fewer row tiles than the others, eight slabs), else 64x128 tiles (up to 128 tiles of 128x128) or
# 128x128 tiles, both with ragged edges
@pytest.mark.parametrize("m,n,k", [(32, 32, 256), (65, 100, 256), (256, 256, 512), (300, 520, 768),
                                   (256, 512, 2304), (512, 256, 4096), (129, 4096, 512), (260, 100, 256),
                                   (1000, 1000, 256), (300, 2790, 512), (300, 8300, 256), (257, 4100, 256)])
@pytest.mark.parametrize("bias", [False, True])
def test_gemm_packed_matches_oracle_and_row_major_kernel(m, n, k, bias):
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    b = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    alpha = 0.111328125
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    y = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b)
    assert not torch.isnan(y.float()).any()
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "mxfp4")
    want = ref.to(torch.bfloat16)
    if bias:
        want = want + b
    # fp32 accumulation in another order than the oracle's, then one bf16 rounding (two with bias)
    tol = 2.0 ** -7 * want.double().abs() + 1e-5 * mag + 1e-6
    assert ((y.double() - want.double()).abs() <= tol).all()
    y_rm = capi.gemm(xq, xs, wq, ws, alpha, "mxfp4", bias=b)
    if k == 256 or (m > 128 and ((m + 127) // 128) * ((n + 31) // 32) > 256):
        # the tile kernels (and any kernel on one block of K): the same MFMA sequence per output as the
        # row-major kernel, identical bits
        assert torch.equal(y.view(torch.int16), y_rm.view(torch.int16))
    else:
        # the weight-streaming kernel (also in slabs) adds four K parts: another order, the same tolerance
        assert ((y.double() - y_rm.double()).abs() <= 2 * tol).all()


@pytest.mark.parametrize("m,n,k", [(257, 11008, 8192), (700, 5400, 8448)])
def test_long_k_half_tiles_with_a_cu_to_themselves(m, n, k):
    """More than 256 tiles of 128 x 128, at most 256 of 256 x 128 and K >= 8192: the 256 x 128 MXFP4 tiles with a
    ring of eight units.  Bit for bit the row-major kernel's result (the same MFMA sequence per output), and within
    tolerance of the oracle on a sample of the columns."""
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    b = torch.randn(n, generator=g).to(torch.bfloat16)
    alpha = 0.111328125
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    y = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b)
    assert torch.equal(y.view(torch.int16), capi.gemm(xq, xs, wq, ws, alpha, "mxfp4", bias=b).view(torch.int16))
    cols = torch.randperm(n, generator=g)[:300]
    ref, mag = O.gemm_ref(xq, xs, wq[cols], ws[cols], alpha, "mxfp4")
    want = ref.to(torch.bfloat16) + b[cols]
    tol = 2.0 ** -7 * want.double().abs() + 1e-5 * mag + 1e-6
    assert ((y[:, cols].double() - want.double()).abs() <= tol).all()


def test_gemm_packed_rejects():
    z = torch.zeros(4096, dtype=torch.uint8)
    with pytest.raises(ValueError):
        capi.gemm_packed(z, z, z, z, 32, 32, 128, 1.0)       # K % 256 != 0


@needs_packed
def test_linear_uses_packed_path_and_matches_row_major(monkeypatch):
    """FPQuantLinear above the row threshold runs quantize-to-packed + packed GEMM; the result is
    bit-identical to the row-major kernels (FPQ_PACKED_WEIGHTS=0)."""
    import fp_quant
    from fp_quant.module import hip_ops
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.MXFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=128)
    torch.manual_seed(2)
    lin = fp_quant.FPQuantLinear(512, 384, cfg, bias=True, device="cuda", dtype=torch.bfloat16)
    lin.weight.data.normal_(0, 0.02)
    lin.bias.data.normal_()
    lin.pre_forward()
    x = torch.randn(3, 100, 512, device="cuda", dtype=torch.bfloat16)
    assert x.shape[0] * x.shape[1] >= hip_ops.PACKED_LINEAR_MIN_M
    y_packed = lin(x)
    assert packed_copy(lin) is not None
    monkeypatch.setenv("FPQ_PACKED_WEIGHTS", "0")
    y_rm = lin(x)
    assert torch.equal(y_packed, y_rm)


def pack_nv_by_definition(codes, scales, k):
    """NVFP4 packed scales as include/fpq.h states them: [(rt, kb), (kh, r), q, 2 bytes] = row 32 rt + r,
    groups 16 kb + 4 q + 2 kh (+1); codes as for MXFP4."""
    rows = codes.shape[0]
    rt = (rows + 31) // 32
    pc, _ = pack_by_definition(codes, torch.zeros(rows, k // 32, dtype=torch.uint8), k)
    s = torch.zeros(rt * 32, k // 16, dtype=torch.uint8)
    s[:rows] = scales[:rows, : k // 16]
    ps = s.view(rt, 32, k // 256, 4, 2, 2).permute(0, 2, 4, 1, 3, 5).contiguous().view(-1)
    return pc, ps


@pytest.mark.parametrize("rows,k", [(32, 256), (70, 512), (257, 768)])
def test_pack_nv_kernel_matches_definition(rows, k):
    g = torch.Generator().manual_seed(rows * 3 + k)
    codes = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, generator=g)
    scales = torch.randint(0, 127, (rows + 5, k // 16 + 16), dtype=torch.uint8, generator=g)
    pc, ps = capi.pack_nv(codes, scales)
    wc, ws = pack_nv_by_definition(codes, scales, k)
    assert torch.equal(pc, wc)
    assert torch.equal(ps, ws)


# up to 96 rows, and 97-128 rows with at most 512 weight tiles: the weight-streaming kernel (one to four
# activation row tiles, ragged rows and columns, odd tile counts, long K); everything else: the tile kernels
@pytest.mark.parametrize("m,n,k", [(1, 64, 256), (32, 32, 256), (65, 100, 512), (256, 256, 768), (300, 520, 1024),
                                   (512, 256, 4096), (16, 1024, 1024), (48, 515, 768), (64, 14336, 256),
                                   (96, 2048, 4096), (128, 1000, 2304), (5, 257, 12288), (100, 8290, 256),
                                   (96, 40000, 256), (128, 16384, 256), (128, 16400, 256), (97, 14339, 512),
                                   # 129-256 rows at up to 256 weight tiles: two passes of the weight-streaming kernel
                                   (130, 515, 512), (192, 6144, 256), (256, 8192, 256), (255, 8200, 256), (161, 100, 1024),
                                   # more than 128 rows in slabs, and the tile kernels' ragged edges past them
                                   (129, 4096, 512), (260, 100, 256), (1000, 1000, 256), (300, 2790, 512), (300, 8300, 256),
                                   # 33-64 rows at 768 weight tiles or more: two weight tiles per workgroup (odd count, ragged N)
                                   (64, 24600, 256), (45, 28672, 256),
                                   # more than 256 tiles of 128 x 128: 256 x 128 tiles (six scale pieces per block; an odd
                                   # and an even number of 128-row tiles, ragged rows and columns), 256 x 256 tiles where
                                   # they fill whole rounds
                                   (384, 11010, 256), (300, 11100, 512), (512, 8450, 512), (1024, 16384, 256)])
@pytest.mark.parametrize("bias", [False, True])
def test_gemm_nv_packed_matches_oracle(m, n, k, bias):
    g = torch.Generator().manual_seed(m + 2 * n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(1, 0x7f, (m, k // 16), dtype=torch.uint8, generator=g)    # every positive E4M3 value
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
    # one bf16 rounding of a sum accumulated in another order; with bias a second rounding on top
    tol = (2.0 if bias else 1.0) * 2.0 ** -7 * torch.maximum(want.double().abs(), ref.abs()) + 1e-5 * mag + 1e-6
    assert ((y.double() - want.double()).abs() <= tol).all()
    exact = (y.view(torch.int16) == want.view(torch.int16)).double().mean()
    assert exact > 0.97
    # the residual epilogue is the separate bf16 addition, bit for bit, also written in place
    res = (torch.randn(m, n, generator=g) * 4).to(torch.bfloat16)
    yr = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res)
    assert torch.equal(yr, y + res)
    assert torch.equal(capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res, in_place=True), yr)


@pytest.mark.parametrize("m,n,k", [(32, 32, 256), (65, 100, 256), (300, 520, 768), (256, 4096, 512), (2048, 1024, 512),
                                   (300, 2790, 256), (300, 8300, 256), (129, 4096, 256)])
@pytest.mark.parametrize("bias", [False, True])
def test_gemm_packed_residual_equals_gemm_then_add(m, n, k, bias):
    """The residual epilogue is the separate bf16 addition, bit for bit, for every tile shape and at
    ragged edges (N not a multiple of 8 takes the element-wise stores); also when written in place."""
    g = torch.Generator().manual_seed(3 * m + n + k)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(118, 134, (m, k // 32), dtype=torch.uint8, generator=g)
    ws = torch.randint(118, 134, (n, k // 32), dtype=torch.uint8, generator=g)
    b = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    res = (torch.randn(m, n, generator=g) * 20).to(torch.bfloat16)
    xp, xsp = pack_by_definition(xq, xs, k)
    wp, wsp = pack_by_definition(wq, ws, k)
    plain = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, 0.111328125, bias=b)
    want = plain + res                                   # torch's bf16 add: one rounding of the fp32 sum
    got = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, 0.111328125, bias=b, residual=res)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    got2 = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, 0.111328125, bias=b, residual=res, in_place=True)
    assert torch.equal(got2.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("rot,g", [("hadamard", 16), ("hadamard", 32), ("hadamard", 64), ("hadamard", 128),
                                   ("identity", 16), ("gsr", 32)])
@pytest.mark.parametrize("policy", [0, 1])
@pytest.mark.parametrize("rows", [70, 1, 13, 64])
def test_quantize_nv_packed_bit_exact(rot, g, policy, rows):
    cols = 512  # 70 rows: ragged last row tile
    x = make_outlier_normal(rows, cols, 13 * g + len(rot))
    x[3 % rows, 64:96] = 0.0     # zero groups
    x[5 % rows, :32] = -0.0
    if rows > 7:
        x[7] *= 2.0 ** -20       # E4M3 scales that underflow to zero
    okind = {"hadamard": O.ROT_HADAMARD, "identity": O.ROT_IDENTITY, "gsr": O.ROT_GSR}[rot]
    norm = float(O.hadamard_matrix(g)[0, 0])
    for gs in (40.0, 2.0 ** 70):  # the second takes the generic per-element path
        wc, ws, _ = O.quantize_nv(x, gs, okind, g, norm, zero_nibble=policy)
        want_c, want_s = pack_nv_by_definition(wc, ws, cols)
        pc, ps = capi.quantize_nv_packed(x, gs, rot=rot, g=g, norm=norm, zero_policy=policy)
        assert torch.equal(pc, want_c)
        assert torch.equal(ps, want_s)


@pytest.mark.parametrize("fmt,rot,g", [("mxfp4", "hadamard", 128), ("mxfp4", "gsr", 64), ("mxfp4", "identity", 32),
                                       ("nvfp4", "hadamard", 16), ("nvfp4", "hadamard", 128)])
def test_quantize_packed_from_two_to_the_24_elements(fmt, rot, g):
    """From 2^24 elements on a lane of the packed streaming quantizer owns 64 elements instead of 32: equal to
    re-tiling the row-major quantizer's result (itself checked against the oracle at this size), ragged last
    row tile, rows with exponents outside the fast range."""
    rows, cols = 4100, 4096
    gen = torch.Generator().manual_seed(g + len(rot))
    x = (torch.randn(rows, cols, generator=gen) * 3).to(torch.bfloat16)
    x[7] *= 2.0 ** -110
    x[9] *= 2.0 ** 105
    x[11, 64:96] = 0.0
    if fmt == "mxfp4":
        rc, rs = capi.quantize(x, fmt, rot=rot, g=g)
        want_c, want_s = pack_by_definition(rc, rs, cols)
        pc, ps = capi.quantize_packed(x, rot=rot, g=g)
    else:
        rc, rs = capi.quantize(x, fmt, rot=rot, g=g, global_scale=25.0)
        want_c, want_s = pack_nv_by_definition(rc, rs, cols)
        pc, ps = capi.quantize_nv_packed(x, 25.0, rot=rot, g=g)
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)


def test_quantize_nv_packed_large_matches_row_major_path():
    gen = torch.Generator().manual_seed(6)
    x = (torch.randn(1000, 4096, generator=gen) * 3).to(torch.bfloat16)
    rc, rs = capi.quantize(x, "nvfp4", g=16, global_scale=25.0)
    want_c, want_s = pack_nv_by_definition(rc, rs, 4096)
    pc, ps = capi.quantize_nv_packed(x, 25.0, g=16)
    assert torch.equal(pc, want_c) and torch.equal(ps, want_s)
    with pytest.raises(ValueError):
        capi.quantize_nv_packed(torch.zeros(32, 384, dtype=torch.bfloat16), 1.0)   # cols % 256 != 0


@needs_packed
def test_nvfp4_linear_mid_m_runs_packed_and_matches_oracle(monkeypatch):
    import fp_quant
    from fp_quant.module import hip_ops
    cfg = fp_quant.FPQuantConfig(forward_dtype=fp_quant.FPQuantDtype.NVFP4, forward_method="abs_max",
                                 backward_dtype=fp_quant.FPQuantDtype.BF16, hadamard_group_size=16)
    gen = torch.Generator().manual_seed(21)
    k, n, m = 512, 384, 100
    w = (torch.randn(n, k, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    lin = fp_quant.FPQuantLinear(k, n, cfg, bias=False, device="cuda", dtype=torch.bfloat16)
    lin.weight.data = w.cuda()
    lin.pre_forward()
    assert hip_ops.nv_packed_eligible(m, n, k)
    y = lin(x.cuda()).cpu()
    assert packed_copy(lin) is not None
    gs = float(lin.act_global_scale)
    norm = float(O.hadamard_matrix(16)[0, 0])
    wq, ws, _ = O.quantize_nv(w, gs, O.ROT_HADAMARD, 16, norm)
    xq, xs, _ = O.quantize_nv(x, gs, O.ROT_HADAMARD, 16, norm)
    alpha = O.alpha_from_global_scales(lin.weight_global_scale.cpu(), lin.act_global_scale.cpu())
    ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, "nvfp4")
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6).all()
    monkeypatch.setenv("FPQ_PACKED_WEIGHTS", "0")
    y_rm = lin(x.cuda()).cpu()
    assert ((y.double() - y_rm.double()).abs() <= 2.0 ** -7 * ref.abs() + 1e-5 * mag + 1e-6).all()


@pytest.mark.parametrize("rows,k", [(1, 256), (33, 768), (70, 512), (256, 4096), (1000, 1024)])
def test_unpack_is_the_inverse_of_the_layout_definition(rows, k):
    """fpq_unpack_mxf4 on a packed operand written by the layout's definition gives back the row-major codes
    and scales (ragged last row tile; a scale matrix wider than K/32 keeps its other entries)."""
    g = torch.Generator().manual_seed(rows + k)
    codes = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, generator=g)
    scales = torch.randint(0, 256, (rows, k // 32), dtype=torch.uint8, generator=g)
    pc, ps = pack_by_definition(codes, scales, k)
    got_c, got_s = capi.unpack(pc, ps, rows, k)
    assert torch.equal(got_c, codes) and torch.equal(got_s, scales)
    got_c, got_s = capi.unpack(pc, ps, rows, k, scale_pad=4)
    assert torch.equal(got_c, codes) and torch.equal(got_s[:, : k // 32], scales)
    assert (got_s[:, k // 32:] == 0xCD).all()
    # and of fpq_pack_mxf4
    pc2, ps2 = capi.pack(codes, scales)
    assert torch.equal(pc2, pc) and torch.equal(ps2, ps)


@pytest.mark.parametrize("rows,k", [(1, 256), (33, 768), (70, 512), (1000, 1024)])
def test_unpack_nv_is_the_inverse_of_the_layout_definition(rows, k):
    g = torch.Generator().manual_seed(rows + k)
    codes = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, generator=g)
    scales = torch.randint(0, 256, (rows, k // 16), dtype=torch.uint8, generator=g)
    pc, ps = pack_nv_by_definition(codes, scales, k)
    got_c, got_s = capi.unpack(pc, ps, rows, k, nv=True)
    assert torch.equal(got_c, codes) and torch.equal(got_s, scales)
    got_c, got_s = capi.unpack(pc, ps, rows, k, scale_pad=8, nv=True)
    assert torch.equal(got_c, codes) and torch.equal(got_s[:, : k // 16], scales)
    assert (got_s[:, k // 16:] == 0xCD).all()


@pytest.mark.parametrize("m,splits,k", [(1, [512, 256, 256], 512), (48, [1024, 256], 1024), (96, [256, 512], 256),
                                        (128, [256, 256, 256, 256], 768), (300, [512, 256, 256], 512),
                                        (2048, [2048, 1024, 256, 768], 256), (200, [256, 512], 512),
                                        (131, [1024, 256, 256], 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_nv_layers_end_to_end_get_their_own_outputs(m, splits, k, with_bias):
    """fpq_gemm_nvf4_packed_multi: every layer's matrix equals its column range of fpq_gemm_nvf4_packed on the
    same operands bit for bit (weight-streaming kernel in one pass and in two, 128x128 tiles, 256x256 tiles)."""
    n = sum(splits)
    g = torch.Generator().manual_seed(900 + m + n)
    xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
    wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
    xs = torch.randint(24, 72, (m, k // 16), dtype=torch.uint8, generator=g)
    ws = torch.randint(24, 72, (n, k // 16), dtype=torch.uint8, generator=g)
    bias = torch.randn(n, generator=g).to(torch.bfloat16) if with_bias else None
    xp, xsp = pack_nv_by_definition(xq, xs, k)
    wp, wsp = pack_nv_by_definition(wq, ws, k)
    whole = capi.gemm_nv_packed(xp, xsp, wp, wsp, m, n, k, 2.0 ** -6, bias=bias)
    outs = capi.gemm_packed_multi(xp, xsp, wp, wsp, m, splits, k, 2.0 ** -6, bias=bias, nv=True)
    col = 0
    for o, s_ in zip(outs, splits):
        assert o.shape == (m, s_)
        assert torch.equal(o.view(torch.int16), whole[:, col:col + s_].contiguous().view(torch.int16))
        col += s_
