"""Pins of the oracle's producer functions (the elementwise operators whose output the quantizer
consumes): the fixed-sequence exp against float64, silu_mul and rmsnorm against float64 evaluations
with explicit roundings and against torch's / transformers' own operators, the summation order of
the row statistic against a per-row Python loop."""
import math

import numpy as np
import pytest
import torch

from oracle import fpq_oracle as O


def _bf16_ulp(t):
    """Spacing of bf16 numbers at |t| (float64): 2^(exponent - 7)."""
    return torch.exp2(torch.floor(torch.log2(t.double().abs().clamp_min(2.0 ** -126))) - 7)


def test_exp_det_accuracy_and_edges():
    t = torch.linspace(-104, 88.7, 400001)
    got = O.exp_det(t).double()
    ref = torch.exp(t.double())
    normal = ref > 2.0 ** -126
    assert float(((got - ref).abs() / ref)[normal].max()) < 1.2e-7          # ~1 ulp
    assert torch.equal(O.exp_det(torch.tensor([0.0, 1000.0, -1000.0, 89.0, -110.0])),
                       torch.tensor([1.0, float("inf"), 0.0, float("inf"), 0.0]))
    # gradual underflow below 2^-126 and the last finite binade
    assert 0.0 < float(O.exp_det(torch.tensor([-100.0]))) < 2.0 ** -126
    assert math.isfinite(float(O.exp_det(torch.tensor([88.5]))))
    # arguments next to multiples of ln 2 (where n = rint(t * log2e) switches binade)
    for n in (-20, -1, 1, 7, 60):
        x = torch.tensor([n * math.log(2.0)])
        assert abs(float(O.exp_det(x)) / math.exp(float(x)) - 1.0) < 1.2e-7


def test_exp_det_is_the_stated_sequence():
    """One value by hand with numpy float32 scalars, operation by operation."""
    f = np.float32
    t = f(-3.337)
    n = f(np.rint(t * f(1.44269504088896341)))
    r = (t - n * f(0.693359375)) - n * f(-2.12194440e-4)
    p = f(1.9875691500e-4)
    for c in (1.3981999507e-3, 8.3334519073e-3, 4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1):
        p = f(p * r) + f(c)
    y = f(f(f(p * f(r * r)) + r) + f(1.0))
    want = np.ldexp(y, int(n))
    assert float(O.exp_det(torch.tensor([float(t)]))) == float(want)
    assert n == -5.0 and abs(float(want) - math.exp(-3.337)) < 1e-8


def test_silu_mul_against_float64_and_torch():
    gen = torch.Generator().manual_seed(0)
    g = (torch.randn(257, 384, generator=gen) * 4).to(torch.bfloat16)
    u = torch.randn(257, 384, generator=gen).to(torch.bfloat16)
    got = O.silu_mul(g, u)
    assert got.dtype == torch.bfloat16
    gd = g.double()
    s64 = (gd / (1 + torch.exp(-gd)))
    # away from bf16 rounding boundaries of silu the fp32 sequence and the float64 value round alike
    s_bf = s64.to(torch.float32).to(torch.bfloat16)
    safe = (s64 - s_bf.double()).abs() < 0.49 * _bf16_ulp(s_bf)
    want = (s_bf.float() * u.float()).to(torch.bfloat16)
    assert float(safe.float().mean()) > 0.95 and torch.equal(got[safe], want[safe])
    # torch's own operators (silu then mul, one bf16 rounding each) give the same tensor
    assert int((got != torch.nn.functional.silu(g) * u).sum()) <= 2
    # extremes: silu(-inf side) -> -0, silu(+large) -> x, zeros stay zeros
    e = torch.tensor([[-300.0, 300.0, 0.0, -0.0, -88.5, 1e-30]]).to(torch.bfloat16)
    out = O.silu_mul(e, torch.ones_like(e)).float()
    assert out[0, 0] == 0.0 and out[0, 1] == 300.0 and out[0, 2] == 0.0 and out[0, 3] == 0.0
    assert -1e-35 < float(out[0, 4]) < 0.0 and float(out[0, 5]) == float(torch.tensor(0.5e-30).to(torch.bfloat16))


@pytest.mark.parametrize("cols", [8, 64, 520, 4096])
def test_row_inv_rms_order_and_value(cols):
    gen = torch.Generator().manual_seed(cols)
    x = (torch.randn(5, cols, generator=gen) * 3).to(torch.bfloat16)
    eps = 1e-5
    got = O.row_inv_rms(x, eps)
    ref = 1.0 / torch.sqrt((x.double() ** 2).mean(-1) + eps)
    assert float(((got.double() - ref).abs() / ref).max()) < 3e-7
    # the stated order, one row in a Python loop over numpy float32 scalars
    f = np.float32
    row = x[3].float().numpy()
    acc = [f(0.0)] * 64
    for k in range(cols // 8):
        s = f(row[8 * k] * row[8 * k])
        for i in range(1, 8):
            s = f(s + f(row[8 * k + i] * row[8 * k + i]))
        acc[k % 64] = f(acc[k % 64] + s)
    for m in (1, 2, 4, 8, 16, 32):
        acc = [f(acc[i] + acc[i ^ m]) for i in range(64)]
    want = f(1.0) / np.sqrt(f(f(acc[0] / f(cols)) + f(eps)))
    assert float(got[3]) == float(want)


def test_rmsnorm_against_float64_and_transformers():
    gen = torch.Generator().manual_seed(2)
    x = (torch.randn(33, 1024, generator=gen) * 2).to(torch.bfloat16)
    w = (1 + 0.2 * torch.randn(1024, generator=gen)).to(torch.bfloat16)
    got = O.rmsnorm(x, w, 1e-6)
    assert got.dtype == torch.bfloat16
    r64 = 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    n64 = x.double() * r64
    n_bf = n64.float().to(torch.bfloat16)
    safe = (n64 - n_bf.double()).abs() < 0.49 * _bf16_ulp(n_bf)
    want = (n_bf.float() * w.float()).to(torch.bfloat16)
    assert float(safe.float().mean()) > 0.95 and torch.equal(got[safe], want[safe])
    from transformers.models.llama.modeling_llama import LlamaRMSNorm
    hf = LlamaRMSNorm(1024, 1e-6).to(torch.bfloat16)
    hf.weight.data = w
    assert int((got != hf(x)).sum()) <= 2
    # a zero row normalises to zeros (inv_rms = 1/sqrt(eps) stays finite)
    z = torch.zeros(1, 1024, dtype=torch.bfloat16)
    assert float(O.rmsnorm(z, w, 1e-6).abs().max()) == 0.0
