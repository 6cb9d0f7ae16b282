"""Frozen vectors (tests/golden/quantize_golden.npz, written by make_quantize_golden.py from the
CPU oracle: the reference itself ships no fixtures for this path).  The CPU test guards the
oracle against drift; the GPU tests check the kernels against the same frozen bytes."""
import os

import numpy as np
import pytest
import torch

from oracle import fpq_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "quantize_golden.npz"))


def _bf16(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


CASES = ([("mxfp4", f"mx_g{g}_z{z}", dict(rot="hadamard", g=g, zero=z)) for g in (32, 128) for z in (0, 1)]
         + [("mxfp4", "mx_identity", dict(rot="identity", g=32, zero=0))]
         + [("nvfp4", f"nv_g{g}_gs{gs}", dict(rot="hadamard", g=g, zero=0, gs=float(gs)))
            for g, gs in ((16, 3), (16, 10), (64, 3))])


@pytest.mark.parametrize("fmt,key,kw", CASES)
def test_oracle_reproduces_frozen_vectors(fmt, key, kw):
    x = _bf16(G["x_bits"])
    kind = O.ROT_HADAMARD if kw["rot"] == "hadamard" else O.ROT_IDENTITY
    if fmt == "mxfp4":
        c, s, _ = O.quantize_mx(x, kind, kw["g"], zero_nibble=kw["zero"])
    else:
        c, s, _ = O.quantize_nv(x, kw["gs"], kind, kw["g"], zero_nibble=kw["zero"])
    assert np.array_equal(c.numpy(), G[key + "_codes"]) and np.array_equal(s.numpy(), G[key + "_scales"])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,key,kw", CASES)
def test_kernels_reproduce_frozen_vectors(fmt, key, kw):
    import capi
    x = _bf16(G["x_bits"])
    c, s = capi.quantize(x, fmt, kw["rot"], kw["g"], global_scale=kw.get("gs"), zero_policy=kw["zero"])
    assert np.array_equal(c.numpy(), G[key + "_codes"]) and np.array_equal(s.numpy(), G[key + "_scales"])


@pytest.mark.gpu
def test_gemm_reproduces_frozen_linear():
    import capi
    xq, xs = G["mx_g128_z0_codes"], G["mx_g128_z0_scales"]
    w = _bf16(G["w_bits"])
    wq, ws = capi.quantize(w, "mxfp4", "hadamard", 128)
    y = capi.gemm(torch.from_numpy(xq), torch.from_numpy(xs), wq, ws, 0.111328125, "mxfp4")
    ref = torch.from_numpy(G["mx_linear_y"])
    assert ((y.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-6).all()
