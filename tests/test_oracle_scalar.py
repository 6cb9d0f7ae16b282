"""Pins for the oracle's scalar building blocks: each check is a closed form, an exhaustive
table, a library cast or a brute force written independently of the oracle's own formula."""
import itertools
import math

import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import fpq_oracle as O

GRID = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


# ------------------------------------------------------------------ rotation matrices
@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_sylvester_matches_scipy_and_is_orthogonal(g):
    s = O.sylvester_signs(g)
    assert np.array_equal(s, scipy.linalg.hadamard(g))
    assert np.array_equal(s, s.T)
    assert np.array_equal(s @ s, g * np.eye(g))


def test_bf16_norm_values():
    # entries are +-bf16(g**-0.5): exact for 16/64, rounded for 32/128
    expect = {16: 0.25, 32: 0.1767578125, 64: 0.125, 128: 0.08837890625}
    for g, v in expect.items():
        h = O.hadamard_matrix(g)
        assert h.dtype == torch.bfloat16
        assert set(h.float().abs().flatten().tolist()) == {v}


@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_gsr_is_sequency_order(g):
    # independent construction straight from the matrix with torch ops
    h = torch.tensor(scipy.linalg.hadamard(g) * g ** -0.5, dtype=torch.bfloat16)
    changes = torch.diff(h, dim=0).ne(0).sum(dim=0)
    assert sorted(changes.tolist()) == list(range(g))  # all distinct -> argsort unambiguous
    perm = torch.argsort(changes)
    assert torch.equal(O.gsr_matrix(g), h[:, perm].contiguous())
    assert np.array_equal(O.gsr_permutation(g), perm.numpy())
    # column k of the GSR matrix has exactly k sign changes
    gm = O.gsr_matrix(g).float()
    assert (torch.diff(torch.sign(gm), dim=0).ne(0).sum(0) == torch.arange(g)).all()


@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_classify_rotation(g):
    assert O.classify_rotation(O.hadamard_matrix(g)) == (O.ROT_HADAMARD, float(O.hadamard_matrix(g)[0, 0]))
    assert O.classify_rotation(O.identity_matrix(g))[0] == O.ROT_IDENTITY
    assert O.classify_rotation(O.gsr_matrix(g))[0] == O.ROT_GSR
    h = O.hadamard_matrix(g).clone()
    h[3, 5] = -h[3, 5]
    assert O.classify_rotation(h)[0] == O.ROT_GENERAL


# ------------------------------------------------------------------ FWHT
@pytest.mark.parametrize("g", [2, 4, 16, 32, 64, 128])
def test_fwht_equals_definition_on_small_integers(g):
    # integer inputs: every partial sum is exact in fp32, so any summation order agrees
    gen = torch.Generator().manual_seed(g)
    x = torch.randint(-64, 65, (7, 2 * g), generator=gen).float()
    y = O.fwht_fp32(x, g)
    ref = (x.double().view(-1, g) @ torch.from_numpy(O.sylvester_signs(g))).view(7, 2 * g)
    assert torch.equal(y.double(), ref)


def test_fwht_butterfly_order_brute_force():
    # pure-Python restatement of the summation tree with explicit fp32 rounding per node
    g = 8
    gen = torch.Generator().manual_seed(1)
    x = (torch.randn(5, g, generator=gen) * torch.tensor([1e-3, 1.0, 1e3, 1e-6, 7.0]).view(5, 1)).float()
    y = O.fwht_fp32(x, g)
    for r in range(5):
        v = [np.float32(t) for t in x[r].tolist()]
        s = 1
        while s < g:
            nv = list(v)
            for i in range(g):
                if i & s == 0:
                    nv[i] = np.float32(v[i] + v[i + s])
                    nv[i + s] = np.float32(v[i] - v[i + s])
            v = nv
            s *= 2
        assert [float(t) for t in v] == y[r].tolist()


@pytest.mark.parametrize("g", [16, 32, 64, 128])
def test_rotation_close_to_fp64_matmul(g):
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(64, 4 * g, generator=gen).to(torch.bfloat16)
    h = O.hadamard_matrix(g)
    y = O.rotate(x, O.ROT_HADAMARD, g, float(h[0, 0]))
    ref = O.rotate_matmul_fp64(x, h)
    assert torch.allclose(y.double(), ref, rtol=0, atol=2e-6 * float(ref.abs().max()))
    yg = O.rotate(x, O.ROT_GSR, g, float(h[0, 0]))
    refg = O.rotate_matmul_fp64(x, O.gsr_matrix(g))
    assert torch.allclose(yg.double(), refg, rtol=0, atol=2e-6 * float(ref.abs().max()))
    # a wrong sign / transposed operand would fail this: non-symmetric general matrix
    hm = torch.randn(g, g, generator=gen).to(torch.bfloat16)
    yy = O.rotate(x, O.ROT_GENERAL, g, h=hm)
    assert torch.allclose(yy.double(), O.rotate_matmul_fp64(x, hm), rtol=0, atol=1e-4)
    assert torch.equal(O.rotate(x, O.ROT_IDENTITY, g), x.float())


# ------------------------------------------------------------------ exponent extraction
def test_floor_log2_exact_special_values():
    vals, want = [], []
    for k in range(-126, 128):
        vals += [2.0 ** k, float(np.nextafter(np.float32(2.0 ** k), np.float32(0)))]
        want += [k, k - 1]
    for k in range(-149, -126):  # subnormals
        vals.append(2.0 ** k)
        want.append(k)
    got = O.floor_log2_exact(torch.tensor(vals, dtype=torch.float32)).tolist()
    assert got == want
    gen = torch.Generator().manual_seed(0)
    r = (torch.rand(20000, generator=gen) * 1000 + 1e-3).float()
    assert O.floor_log2_exact(r).tolist() == [math.frexp(v)[1] - 1 for v in r.tolist()]


def test_reference_scale_argument_never_changes_the_exponent():
    # quantizer.py:111,165 feed 6*fl(fl(2a)/12), not a, to floor(log2()).  Exhaustive over the
    # mantissa: the binade never differs while a/6 is a normal number.
    f32 = np.float32
    for base in (0x3F800000, 0x41000000, 0x02000000, 0x7E000000):
        a = (np.arange(1 << 23, dtype=np.uint32) + np.uint32(base)).view(np.float32)
        arg = ((a * f32(2.0)) / f32(12.0)) * f32(6.0)
        assert np.array_equal(np.frexp(a)[1], np.frexp(arg)[1])


# ------------------------------------------------------------------ E2M1
def _nearest_even_code(a):
    """Independent statement: nearest grid point; on a tie the even code wins."""
    best, bestd = None, None
    for code, gv in enumerate(GRID):
        d = abs(a - gv)
        if bestd is None or d < bestd or (d == bestd and code % 2 == 0 and best % 2 == 1):
            best, bestd = code, d
    return best


def test_e2m1_rne_exhaustive_bf16():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    v = bits.view(torch.bfloat16).float()
    v = v[torch.isfinite(v)]
    got = O.e2m1_round_rne(v).tolist()
    for val, c in zip(v.tolist(), got):
        assert c == _nearest_even_code(min(abs(val), 100.0)), val


def test_e2m1_midpoints_and_neighbours():
    mids = {0.25: 0, 0.75: 2, 1.25: 2, 1.75: 4, 2.5: 4, 3.5: 6, 5.0: 6}
    for m, code in mids.items():
        lo = float(np.nextafter(np.float32(m), np.float32(0)))
        hi = float(np.nextafter(np.float32(m), np.float32(10)))
        t = torch.tensor([m, -m, lo, hi], dtype=torch.float32)
        below = GRID.index(max(gv for gv in GRID if gv < m))
        assert O.e2m1_round_rne(t).tolist() == [code, code, below, below + 1]
    assert O.e2m1_round_rne(torch.tensor([6.0, 7.0, 1e30, float("inf")])).tolist() == [7, 7, 7, 7]


def test_code_table_and_zero_nibble_policies():
    v = torch.tensor([0.0, -0.0, 0.1, -0.1, 0.5, -0.5, 6.0, -6.0, 1.5, -3.0])
    assert O.e2m1_codes(v, O.ZERO_NIBBLE_REFERENCE).tolist() == [8, 8, 8, 8, 1, 9, 7, 15, 3, 13]
    assert O.e2m1_codes(v, O.ZERO_NIBBLE_SIGNED).tolist() == [0, 8, 0, 8, 1, 9, 7, 15, 3, 13]
    for code, val in enumerate(O.E2M1_VALUES):
        if code not in (0, 8):
            assert O.e2m1_codes(torch.tensor([val]), O.ZERO_NIBBLE_REFERENCE).item() == code


def test_reference_packer_semantics_via_bucketize():
    # The reference maps value -> code through torch.bucketize on a 16-entry grid with two
    # zeros; bucketize(0.0) lands on index 7 whose tie-break picks the entry with code 8.
    grid = torch.tensor([-6.0, -4.0, -3.0, -2.0, -1.5, -1.0, -0.5, 0.0, 0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    code_of_slot = [15, 14, 13, 12, 11, 10, 9, 8, 0, 1, 2, 3, 4, 5, 6, 7]
    assert torch.bucketize(torch.tensor([0.0, -0.0]), grid).tolist() == [7, 7]
    q = torch.tensor([[0.0, -0.0, 0.5, -0.5, 1.0, -6.0, 6.0, 3.0]])
    ids = torch.bucketize(q, grid)
    slot_codes = torch.tensor(code_of_slot)[ids.clamp(0, 15)]  # exact grid hits land on their slot
    mine = O.e2m1_codes(q, O.ZERO_NIBBLE_REFERENCE)
    assert torch.equal(mine.int(), slot_codes.int())
    packed = O.pack_nibbles(mine)
    assert packed.tolist() == [[0x88, 0x91, 0xF2, 0x57]]
    assert torch.equal(O.unpack_nibbles(packed), mine)


# ------------------------------------------------------------------ fp8 casts (library routines)
def test_e4m3_encode_matches_torch_cast():
    gen = torch.Generator().manual_seed(5)
    pts = [0.0, -0.0, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10, 2.0 ** -6, 448.0, 449.0, 464.0,
           465.0, 480.0, 1e9, -448.0, -464.0, -465.0, 17.0, 18.0, 19.0, 1e-12, float("nan")]
    # every representable value, every midpoint between neighbours and their fp32 neighbours
    allv = sorted(set(abs(v) for v in O.e4m3_decode(torch.arange(256).to(torch.uint8)).tolist() if v == v))
    for lo, hi in zip(allv[:-1], allv[1:]):
        m = (lo + hi) / 2
        pts += [lo, m, float(np.nextafter(np.float32(m), np.float32(0))),
                float(np.nextafter(np.float32(m), np.float32(1e9))), -m]
    t = torch.cat([torch.tensor(pts, dtype=torch.float32),
                   (torch.randn(200000, generator=gen) * 100).float(),
                   torch.randn(100000, generator=gen).float() * 2.0 ** -7])
    want = t.to(torch.float8_e4m3fn).view(torch.uint8)
    got = O.e4m3_encode(t)
    nan = torch.isnan(t) | ((want & 0x7F) == 0x7F)
    assert torch.equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7F) == 0x7F).all()
    back = torch.arange(256).to(torch.uint8)
    ref = back.view(torch.float8_e4m3fn).float()
    mine = O.e4m3_decode(back)
    ok = ~torch.isnan(ref)
    assert torch.equal(mine[ok], ref[ok]) and torch.isnan(mine[~ok]).all()


def test_e8m0_encode_matches_torch_cast():
    vals = [2.0 ** k for k in range(-149, 128)]
    vals += [1.5 * 2.0 ** k for k in range(-140, 127)] + [1.4999 * 2.0 ** k for k in range(-126, 127)]
    vals += [0.0, 3.0e38, (2 ** 24 - 1) * 2.0 ** -149, 8388609 * 2.0 ** -149]
    t = torch.tensor(vals, dtype=torch.float32)
    assert torch.equal(O.e8m0_encode(t), t.to(torch.float8_e8m0fnu).view(torch.uint8))
    b = torch.arange(1, 255).to(torch.uint8)
    assert torch.equal(O.e8m0_decode(b), b.view(torch.float8_e8m0fnu).float())


# ------------------------------------------------------------------ scale derivations
def test_mx_scale_closed_forms():
    f32 = np.float32
    assert f32(f32(1.0) / f32(0.75)) * f32(3.0) == f32(4.0)  # stored scale is exactly 2^e
    a = torch.tensor([1.0, 1.99, 2.0, 0.75, 5.9, 6.0, 100.0, 2.0 ** -40, 0.0, 2.0 ** -126, 1.0e38],
                     dtype=torch.float32)
    s, stored = O.mx_scales_from_absmax(a)
    e = [0, 0, 1, -1, 2, 2, 6, -40, -126, -126, 126]
    c = float(f32(1.0) / f32(0.75))
    for i, ei in enumerate(e):
        if ei - 2 >= -126:
            assert float(s[i]) == c * 2.0 ** (ei - 2)
            assert int(stored[i]) == ei + 127
    # zero group: clamp to 2^-126 -> e = -126 -> s = fl(2^-128 / 0.75) (subnormal), byte 1
    assert float(s[8]) == 2796203 * 2.0 ** -149 and int(stored[8]) == 1
    # abs-max never clips: a / s < 6 for every mantissa in a binade
    am = (np.arange(1 << 23, dtype=np.uint32) + np.uint32(0x40000000)).view(np.float32)
    assert (am / f32(c * 2.0 ** (1 - 2)) < 6.0 + 1e-6).all()


def test_nv_scale_chain():
    gs = 10.0
    a = torch.tensor([6.0, 0.6, 0.0, 1e-9, 448.0 * 6 / 10, 1e6, 3.3], dtype=torch.float32)
    sw, stored = O.nv_scales_from_absmax(a, gs)
    f32 = np.float32
    rg = f32(1.0) / f32(gs)
    # a = 6 -> sc0 = 1 -> 10 -> e4m3(10) = 10 -> sw = 10 * fl(0.1)
    assert float(sw[0]) == float(f32(10.0) * rg) and int(stored[0]) == int(torch.tensor(10.0).to(torch.float8_e4m3fn).view(torch.uint8))
    assert float(sw[2]) == 0.0 and int(stored[2]) == 0      # zero group: byte 0
    assert float(sw[3]) == 0.0 and int(stored[3]) == 0      # e4m3 underflow to zero
    assert int(stored[4]) == 0x7E and int(stored[5]) == 0x7E  # 448 and clamped overflow
    # generic value against torch's own cast chain
    t = (f32(3.3) * f32(2.0) / f32(12.0)) * f32(gs)
    sc = torch.tensor(float(t)).to(torch.float8_e4m3fn)
    assert int(stored[6]) == int(sc.view(torch.uint8)) and float(sw[6]) == float(f32(float(sc.float())) * rg)
    assert O.nv_tracked_global_scale(torch.tensor([[0.5, -4.0]])) == float(f32(2688.0) * (f32(1.0) / f32(4.0)))


# ------------------------------------------------------------------ whole quantizers on tiny inputs
def _brute_quantize_mx_row(xr):
    """Per-element Python loop from the written-out definition, numpy fp32 scalars."""
    f32 = np.float32
    out_codes, out_scales = [], []
    for g0 in range(0, len(xr), 32):
        grp = [f32(v) for v in xr[g0:g0 + 32]]
        a = max(abs(v) for v in grp)
        arg = max(f32(f32(f32(a * f32(2)) / f32(12)) * f32(6)), f32(2.0 ** -126))
        e = math.frexp(float(arg))[1] - 1
        s = f32(f32(2.0 ** (e - 2)) / f32(0.75))
        out_scales.append(e + 127)
        for v in grp:
            q = f32(v / s)
            c = _nearest_even_code(min(abs(float(q)), 100.0))
            out_codes.append(c | (8 if (q < 0 or c == 0) else 0))
    return out_codes, out_scales


def test_quantize_mx_against_python_loop():
    gen = torch.Generator().manual_seed(11)
    x = (torch.randn(6, 128, generator=gen) * torch.tensor([1, 30, 1e-3, 1e4, 0.2, 5]).view(6, 1)).to(torch.bfloat16)
    x[0, :32] = 0
    packed, scales, xr = O.quantize_mx(x, O.ROT_HADAMARD, 32)
    codes = O.unpack_nibbles(packed)
    for r in range(6):
        c, s = _brute_quantize_mx_row(xr[r].tolist())
        if r == 0:
            s[0] = 1
        assert codes[r].tolist() == c and scales[r].tolist() == s


def _e4m3_grid():
    """Every finite non-negative float8_e4m3fn value by its byte, from the format's definition."""
    vals = []
    for byte in range(127):                     # 0x7f is NaN
        e, m = byte >> 3, byte & 7
        vals.append((m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
    return vals


def _e4m3_nearest_byte(t, grid=_e4m3_grid()):
    """Nearest E4M3 value of t >= 0 (already clamped to 448), ties to the even byte."""
    best = min(range(127), key=lambda b: (abs(grid[b] - t), b % 2))
    return best


def _brute_quantize_nv_row(xr, gs):
    """Per-element Python loop of the NVFP4 chain as quantizer.py:107-112,143-168 and rtn.py:187-188
    write it, in numpy fp32 scalars, with the E4M3 cast as a nearest-value search."""
    f32 = np.float32
    grid = _e4m3_grid()
    gs = f32(gs)
    rg = f32(1.0) / gs
    out_codes, out_scales = [], []
    for g0 in range(0, len(xr), 16):
        grp = [f32(v) for v in xr[g0:g0 + 16]]
        a = max(abs(v) for v in grp)
        sc0 = f32(f32(f32(2) * a) / f32(12))
        t = min(f32(sc0 * gs), f32(448))
        sc = f32(grid[_e4m3_nearest_byte(float(t))])
        sw = f32(sc * rg)
        if sw == 0:                                   # the documented deviation: byte 0, zero codes
            out_scales.append(0)
            out_codes += [8] * 16
            continue
        stored = _e4m3_nearest_byte(float(min(f32(sw * gs), f32(448))))
        out_scales.append(stored)
        for v in grp:
            q = f32(v / sw)
            c = _nearest_even_code(min(abs(float(q)), 100.0))
            out_codes.append(c | (8 if (q < 0 or c == 0) else 0))
    return out_codes, out_scales


@pytest.mark.parametrize("gs", [3.0, 10.0, 0.0897435918450355, 1234.5])
def test_quantize_nv_against_python_loop(gs):
    gen = torch.Generator().manual_seed(21)
    x = (torch.randn(6, 128, generator=gen) * torch.tensor([1, 30, 1e-3, 1e3, 0.2, 5]).view(6, 1)).to(torch.bfloat16)
    x[0, :16] = 0
    x[4, 16:32] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 2)
    packed, scales, xr = O.quantize_nv(x, gs, O.ROT_HADAMARD, 16)
    codes = O.unpack_nibbles(packed)
    for r in range(6):
        c, s = _brute_quantize_nv_row(xr[r].tolist(), gs)
        assert codes[r].tolist() == c and scales[r].tolist() == s


def test_quantize_roundtrip_error_bound():
    # dequant(code, stored)/3 reproduces the rotated input to within half an E2M1 step
    gen = torch.Generator().manual_seed(12)
    x = torch.randn(32, 256, generator=gen).to(torch.bfloat16)
    packed, scales, xr = O.quantize_mx(x, O.ROT_HADAMARD, 128)
    dq = O.dequantize(packed, scales, "mxfp4") / 3.0
    step = O.e8m0_decode(scales).double().repeat_interleave(32, dim=1) / 3.0  # value of 1.0 code unit
    assert ((dq - xr.double()).abs() <= 1.0 * step + 1e-12).all()
    gs = O.nv_tracked_global_scale(O.rotate(x, O.ROT_HADAMARD, 16, 0.25))
    p2, s2, xr2 = O.quantize_nv(x, gs, O.ROT_HADAMARD, 16)
    dq2 = O.dequantize(p2, s2, "nvfp4") / gs
    unit = O.e4m3_decode(s2).double().repeat_interleave(16, dim=1) / gs
    assert ((dq2 - xr2.double()).abs() <= 1.0 * unit + 1e-9).all()
    assert (O.e4m3_decode(s2) <= 448).all()


def test_gemm_ref_brute_force():
    gen = torch.Generator().manual_seed(13)
    x = torch.randn(3, 64, generator=gen).to(torch.bfloat16)
    w = (torch.randn(5, 64, generator=gen) * 0.02).to(torch.bfloat16)
    xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, 32)
    wq, ws, _ = O.quantize_mx(w, O.ROT_HADAMARD, 32)
    y, mag = O.gemm_ref(xq, xs, wq, ws, 1.0 / 9.0, "mxfp4")
    xc, wc = O.unpack_nibbles(xq), O.unpack_nibbles(wq)
    for m, n in itertools.product(range(3), range(5)):
        acc = 0.0
        for k in range(64):
            acc += (O.E2M1_VALUES[xc[m, k]] * 2.0 ** (int(xs[m, k // 32]) - 127)
                    * O.E2M1_VALUES[wc[n, k]] * 2.0 ** (int(ws[n, k // 32]) - 127))
        assert abs(acc / 9.0 - float(y[m, n])) <= 1e-12 * max(1.0, abs(acc))
    # quantized linear approximates the bf16 linear (rotation is orthogonal up to bf16 norm rounding)
    ref = x.double() @ w.double().T
    assert (y - ref).abs().max() < 0.2 * ref.abs().max()
    assert O.alpha_from_global_scales(torch.tensor([3.0], dtype=torch.bfloat16),
                                      torch.tensor([3.0], dtype=torch.bfloat16)) == 0.111328125
