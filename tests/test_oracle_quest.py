"""Pins for the oracle's "quest" MXFP4 quantizer: the scale rule against float64 statistics and
closed forms, the clip mask and the saturation against the dequantized values."""
import math

import numpy as np
import torch

from oracle import fpq_oracle as O

G = 2.92247856 / 6.0


def test_quest_scale_closed_forms():
    # constant group: std = 0 -> sc = 1e-8 -> floor(log2) = -27 -> byte 100
    x = torch.full((1, 32), 3.25, dtype=torch.float32)
    s, b = O.quest_scales(x.view(1, 1, 32))
    assert int(b) == 100 and float(s) == 2.0 ** -27
    # +a, -a alternating: mean 0, std = a exactly
    for a in (1.0, 0.37, 5.0, 1000.0, 2.0 ** -20):
        x = torch.tensor([a, -a] * 16, dtype=torch.float32).view(1, 1, 32)
        s, b = O.quest_scales(x)
        sc = float(np.float32(np.float32(a) * np.float32(G)) + np.float32(1e-8))
        e = math.frexp(sc)[1] - 1
        assert float(s) == 2.0 ** e and int(b) == e + 127
    # a shift does not change std (up to rounding): mean is removed
    x = torch.tensor([1.0, -1.0] * 16, dtype=torch.float32).view(1, 1, 32)
    s0, _ = O.quest_scales(x)
    s1, _ = O.quest_scales(x + 0.5)
    assert float(s0) == float(s1)


def test_quest_scale_matches_float64_statistics():
    gen = torch.Generator().manual_seed(3)
    x = (torch.randn(4000, 32, generator=gen) * torch.exp(torch.randn(4000, 1, generator=gen) * 3)).float()
    s, b = O.quest_scales(x.view(4000, 1, 32))
    x64 = x.double().numpy()
    sc64 = G * x64.std(axis=1) + 1e-8        # population std, as sqrt(E[x^2] - E[x]^2)
    e64 = np.floor(np.log2(sc64)).astype(np.int64)
    e = b.view(-1).numpy().astype(np.int64) - 127
    # fp32 rounding of the statistics can only move the exponent where sc sits on a power of two
    frac = np.abs(np.log2(sc64) - np.round(np.log2(sc64)))
    bad = e != e64
    assert bad.sum() <= 4 and (frac[bad] < 1e-4).all()
    assert (s.view(-1).numpy() == np.exp2(e.astype(np.float64))).all()


def test_quest_against_a_python_loop_and_mask_semantics():
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(6, 128, generator=gen)
    x[0, 5] = 40.0      # an outlier that must clip
    x[2, 70] = -55.0
    xb = x.to(torch.bfloat16)
    codes, scales, mask, xr = O.quantize_mx_quest(xb, O.ROT_IDENTITY, 32)
    vals = torch.tensor(O.E2M1_VALUES, dtype=torch.float64)
    dq = vals[O.unpack_nibbles(codes).long()] * torch.exp2(scales.double() - 127).repeat_interleave(32, dim=1)
    clipped = 0
    for r in range(6):
        for grp in range(4):
            seg = [np.float32(v) for v in xr[r, grp * 32:(grp + 1) * 32].tolist()]
            octs, octq = [], []
            for o in range(4):
                a, q = seg[o * 8], np.float32(seg[o * 8] * seg[o * 8])
                for i in range(1, 8):
                    a = np.float32(a + seg[o * 8 + i])
                    q = np.float32(q + np.float32(seg[o * 8 + i] * seg[o * 8 + i]))
                octs.append(a); octq.append(q)
            tot = np.float32(np.float32(octs[0] + octs[1]) + np.float32(octs[2] + octs[3]))
            totq = np.float32(np.float32(octq[0] + octq[1]) + np.float32(octq[2] + octq[3]))
            mean, msq = np.float32(tot / 32), np.float32(totq / 32)
            var = max(np.float32(msq - np.float32(mean * mean)), np.float32(0))
            sc = np.float32(np.float32(np.sqrt(var)) * np.float32(G)) + np.float32(1e-8)
            e = math.frexp(float(sc))[1] - 1
            assert int(scales[r, grp]) == e + 127
            for i in range(32):
                c = grp * 32 + i
                q = float(seg[i]) / 2.0 ** e
                inside = abs(q) < 6.0
                assert ((int(mask[r, c // 8]) >> (c % 8)) & 1) == int(inside)
                if not inside:
                    clipped += 1
                    assert abs(float(dq[r, c])) == 6.0 * 2.0 ** e and (dq[r, c] < 0) == (q < 0)
                else:
                    # nearest grid point of the E2M1 grid (spacing at most 2 below 6)
                    assert abs(float(dq[r, c]) / 2.0 ** e - q) <= 1.0
    assert clipped >= 2


def test_quest_zero_policies_differ_only_in_zero_nibbles():
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(4, 64, generator=gen).to(torch.bfloat16)
    x[1, :32] = 0
    c0, s0, m0, _ = O.quantize_mx_quest(x, O.ROT_IDENTITY, 32, zero_nibble=O.ZERO_NIBBLE_REFERENCE)
    c1, s1, m1, _ = O.quantize_mx_quest(x, O.ROT_IDENTITY, 32, zero_nibble=O.ZERO_NIBBLE_SIGNED)
    assert torch.equal(s0, s1) and torch.equal(m0, m1)
    n0, n1 = O.unpack_nibbles(c0), O.unpack_nibbles(c1)
    diff = n0 != n1
    assert ((n0[diff] & 7) == 0).all() and ((n1[diff] & 7) == 0).all()
