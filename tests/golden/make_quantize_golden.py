"""Writes tests/golden/quantize_golden.npz: small frozen input/output vectors of the rotate+quantize
path.  The reference ships no fixtures for this path, so these vectors are produced by this
repository's CPU oracle (itself pinned by tests/test_oracle_scalar.py); they freeze the expected
bytes so that neither the oracle nor the kernels can drift unnoticed.

Run from the repository root:  python tests/golden/make_quantize_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import fpq_oracle as O  # noqa: E402


def inputs():
    gen = torch.Generator().manual_seed(2024)
    x = torch.randn(24, 256, generator=gen)
    mask = torch.rand(24, 256, generator=gen) < 0.01
    x = torch.where(mask, x * 25.0, x)
    x[3] = 0.0                       # all-zero row
    x[4, :64] = 0.0                  # zero groups inside a row
    x[5] *= 1e-20
    x[6] *= 1e4
    x[7] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 32)
    x[8] = 2.0
    return x.to(torch.bfloat16)


def main():
    x = inputs()
    out = {"x_bits": x.view(torch.int16).numpy().view(np.uint16)}
    for g in (32, 128):
        for zero in (0, 1):
            c, s, _ = O.quantize_mx(x, O.ROT_HADAMARD, g, zero_nibble=zero)
            out[f"mx_g{g}_z{zero}_codes"] = c.numpy()
            out[f"mx_g{g}_z{zero}_scales"] = s.numpy()
    c, s, _ = O.quantize_mx(x, O.ROT_IDENTITY, 32)
    out["mx_identity_codes"], out["mx_identity_scales"] = c.numpy(), s.numpy()
    for g, gs in ((16, 3.0), (16, 10.0), (64, 3.0)):
        c, s, _ = O.quantize_nv(x, gs, O.ROT_HADAMARD, g)
        out[f"nv_g{g}_gs{int(gs)}_codes"] = c.numpy()
        out[f"nv_g{g}_gs{int(gs)}_scales"] = s.numpy()
    # one small linear: operands and the fp64 result, for the GEMM tests
    gen = torch.Generator().manual_seed(7)
    w = (torch.randn(48, 256, generator=gen) * 0.02).to(torch.bfloat16)
    out["w_bits"] = w.view(torch.int16).numpy().view(np.uint16)
    xq, xs, _ = O.quantize_mx(x, O.ROT_HADAMARD, 128)
    wq, ws, _ = O.quantize_mx(w, O.ROT_HADAMARD, 128)
    y, _ = O.gemm_ref(xq, xs, wq, ws, 0.111328125, "mxfp4")
    out["mx_linear_y"] = y.numpy()
    path = os.path.join(ROOT, "tests", "golden", "quantize_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
