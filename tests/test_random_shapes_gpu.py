"""Seeded random shapes through the C ABI: the packed and row-major GEMMs (MXFP4, NVFP4, several layers in one
launch, bias and residual epilogues) within the GEMM tolerance of the oracle's fp64 product, and every
quantizer (row-major, packed, fused with RMSNorm / SiLU*up, a few rows in one launch) bit for bit.  The row
counts sit around the borders between kernels (32, 64, 128, 256 rows; 100 and 256 tiles)."""
import random

import pytest
import torch

from oracle import fpq_oracle as O
import capi
from test_packed_gpu import pack_by_definition, pack_nv_by_definition

pytestmark = pytest.mark.gpu

ALPHA = 0.111328125


def _close(y, ref, mag):
    tol = 2.0 ** -8 * ref.abs() + 1e-5 * mag + 1e-6
    return (not torch.isnan(y.float()).any() and bool(((y.double() - ref).abs() <= tol).all())
            and (y == ref.to(torch.bfloat16)).float().mean().item() > 0.97)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_gemms_on_random_shapes(seed):
    rnd = random.Random(seed)
    done = 0
    while done < 120:
        m = max(1, rnd.choice([1, 2, 16, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 200, 255, 256, 257, 384, 511, 512, 640])
                + rnd.choice([0, 0, 0, -1, 1, 3]))
        n = max(1, rnd.choice([32, 64, 100, 128, 255, 256, 257, 512, 512, 1000, 1024, 1024, 2048, 2048, 3000, 4096,
                               6144, 8192]) + rnd.choice([0, 0, 0, 0, 0, -1, 1, 31, 33]))
        k = 256 * rnd.choice([1, 1, 2, 3, 4, 5, 8, 9, 16])
        if m * n * k > 2.5e9:
            continue
        done += 1
        fmt = rnd.choice(["mxfp4", "mxfp4", "nvfp4"])
        what = f"{fmt} m={m} n={n} k={k}"
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        group = 32 if fmt == "mxfp4" else 16
        xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
        wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
        lo, hi = (118, 134) if fmt == "mxfp4" else (0x08, 0x7f)     # E8M0 around 1; positive finite E4M3
        xs = torch.randint(lo, hi, (m, k // group), dtype=torch.uint8, generator=g)
        ws = torch.randint(lo, hi, (n, k // group), dtype=torch.uint8, generator=g)
        alpha = ALPHA if fmt == "mxfp4" else ALPHA / 4096
        ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, fmt)
        nv = fmt == "nvfp4"
        xp, xsp = (pack_nv_by_definition if nv else pack_by_definition)(xq, xs, k)
        wp, wsp = (pack_nv_by_definition if nv else pack_by_definition)(wq, ws, k)
        y = (capi.gemm_nv_packed if nv else capi.gemm_packed)(xp, xsp, wp, wsp, m, n, k, alpha)
        assert _close(y, ref, mag), what + " packed"
        assert _close(capi.gemm(xq, xs, wq, ws, alpha, fmt), ref, mag), what + " row-major"
        if not nv and rnd.random() < 0.5:
            b = torch.randn(n, generator=g).to(torch.bfloat16)
            res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
            yr = capi.gemm_packed(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res)
            assert torch.equal(yr, (y + b) + res), what + " bias and residual"
        if n >= 512 and n % 256 == 0:
            cut = rnd.randrange(1, n // 256) * 256
            outs = capi.gemm_packed_multi(xp, xsp, wp, wsp, m, [cut, n - cut], k, alpha, nv=nv)
            assert torch.equal(outs[0], y[:, :cut]) and torch.equal(outs[1], y[:, cut:]), what + f" two layers at {cut}"


@pytest.mark.parametrize("seed", [21, 22])
def test_gemms_beyond_one_round_of_small_tiles(seed):
    """More than 256 tiles of 128 x 128: the 256 x 128 and 256 x 256 tiles of both formats (an odd or even number of
    128-row tiles, ragged rows and columns), alone, with bias and residual, and as several layers in one launch."""
    rnd = random.Random(seed)
    for _ in range(10):
        m = rnd.choice([257, 300, 384, 512, 640, 700, 1024]) + rnd.choice([0, 0, -1, 1])
        n = rnd.choice([8192, 12288, 16384]) + rnd.choice([0, 0, 0, 31, 100, -1])
        k = 256 * rnd.choice([1, 1, 2])
        if ((m + 127) // 128) * ((n + 127) // 128) <= 256:
            n += 4096
        fmt = rnd.choice(["mxfp4", "nvfp4", "nvfp4"])
        nv = fmt == "nvfp4"
        what = f"{fmt} m={m} n={n} k={k}"
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        group = 16 if nv else 32
        xq = torch.randint(0, 256, (m, k // 2), dtype=torch.uint8, generator=g)
        wq = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=g)
        lo, hi = (0x08, 0x7f) if nv else (118, 134)
        xs = torch.randint(lo, hi, (m, k // group), dtype=torch.uint8, generator=g)
        ws = torch.randint(lo, hi, (n, k // group), dtype=torch.uint8, generator=g)
        alpha = ALPHA / 4096 if nv else ALPHA
        ref, mag = O.gemm_ref(xq, xs, wq, ws, alpha, fmt)
        xp, xsp = (pack_nv_by_definition if nv else pack_by_definition)(xq, xs, k)
        wp, wsp = (pack_nv_by_definition if nv else pack_by_definition)(wq, ws, k)
        gemm = capi.gemm_nv_packed if nv else capi.gemm_packed
        y = gemm(xp, xsp, wp, wsp, m, n, k, alpha)
        assert _close(y, ref, mag), what + " packed"
        b = torch.randn(n, generator=g).to(torch.bfloat16)
        res = (torch.randn(m, n, generator=g) * 8).to(torch.bfloat16)
        assert torch.equal(gemm(xp, xsp, wp, wsp, m, n, k, alpha, bias=b, residual=res), (y + b) + res), what + " bias and residual"
        if n % 256 == 0:
            cut = rnd.randrange(1, n // 256) * 256
            outs = capi.gemm_packed_multi(xp, xsp, wp, wsp, m, [cut, n - cut], k, alpha, nv=nv)
            assert torch.equal(outs[0], y[:, :cut]) and torch.equal(outs[1], y[:, cut:]), what + f" two layers at {cut}"


def _data(rnd, rows, cols, gen):
    x = torch.randn(rows, cols, generator=gen)
    kind = rnd.randrange(5)
    if kind == 0:
        x = x * torch.exp2(torch.randint(-30, 30, (rows, 1), generator=gen).float())
    elif kind == 1:
        x[torch.rand(rows, cols, generator=gen) < 0.01] *= 40.0
    elif kind == 2:
        x = torch.round(x * 2) / 2          # many exact ties on the grid
    elif kind == 3:
        x[:, : cols // 2] = 0.0
    x = x.to(torch.bfloat16)
    if rows > 2:
        x[rnd.randrange(rows)] = 0.0
    return x


@pytest.mark.parametrize("seed", [21, 22, 23, 24])
def test_quantizers_on_random_shapes(seed):
    rnd = random.Random(seed)
    done = 0
    while done < 120:
        fmt = rnd.choice(["mxfp4", "nvfp4"])
        rot = rnd.choice(["hadamard", "hadamard", "identity"])
        g = rnd.choice([16, 32, 64, 128]) if rot == "hadamard" else (32 if fmt == "mxfp4" else 16)
        rows = max(1, rnd.choice([1, 3, 31, 32, 33, 64, 65, 100, 129, 300, 513, 1100]) + rnd.choice([0, 0, 1, -1]))
        mult = rnd.choice([max(g, 32), 64, 256, 256])
        cols = mult * rnd.randrange(1, max(2, 8192 // mult // rnd.choice([1, 2, 8])))
        if cols % max(g, 32) or rows * cols > 3e6:
            continue
        done += 1
        gen = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        x = _data(rnd, rows, cols, gen)
        gs = rnd.choice([1.0, 3.0, 10.0, 777.0, 0.01])
        okind = O.ROT_HADAMARD if rot == "hadamard" else O.ROT_IDENTITY
        norm = float(O.hadamard_matrix(g)[0, 0])
        what = f"{fmt} {rot}{g} rows={rows} cols={cols}"
        nv = fmt == "nvfp4"

        def oracle_q(v):
            if nv:
                c, s, _ = O.quantize_nv(v, gs, okind, g, norm)
            else:
                c, s, _ = O.quantize_mx(v, okind, g, norm)
            return c, s

        def oracle_packed(v):
            c, s = oracle_q(v)
            return (pack_nv_by_definition if nv else pack_by_definition)(c, s, cols)

        wc, ws = oracle_q(x)
        c, s = capi.quantize(x, fmt, rot=rot, g=g, global_scale=gs)
        assert torch.equal(c, wc) and torch.equal(s, ws), what + " row-major"
        if cols % 256:
            continue
        want = oracle_packed(x)
        got = capi.quantize_nv_packed(x, gs, rot=rot, g=g) if nv else capi.quantize_packed(x, rot=rot, g=g)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), what + " packed"
        nv_gs = dict(global_scale=gs) if nv else {}
        w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
        v = O.rmsnorm(x, w, 1e-5)
        want = oracle_packed(v)
        pc, ps, out = capi.fused_quantize_packed("rmsnorm", x, w, g=g, rot=rot, **nv_gs)
        assert torch.equal(pc, want[0]) and torch.equal(ps, want[1]), what + " rmsnorm"
        assert torch.equal(out.view(torch.int16), v.view(torch.int16)), what + " rmsnorm by-product"
        if rows <= 64:
            pc, ps, out, inv = capi.rmsnorm_rows_quantize_packed(x, w, g=g, rot=rot, **nv_gs)
            assert torch.equal(pc, want[0]) and torch.equal(ps, want[1]), what + " rmsnorm, one launch"
            assert torch.equal(out.view(torch.int16), v.view(torch.int16)) and torch.equal(inv, O.row_inv_rms(x, 1e-5))
        up = _data(rnd, rows, cols, gen)
        v = O.silu_mul(x, up)
        want = oracle_packed(v)
        pc, ps, out = capi.fused_quantize_packed("silu_mul", x, up, g=g, rot=rot, **nv_gs)
        assert torch.equal(pc, want[0]) and torch.equal(ps, want[1]), what + " silu*up"
        assert torch.equal(out.view(torch.int16), v.view(torch.int16)), what + " silu*up by-product"
