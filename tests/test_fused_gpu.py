"""Quantizers fused with the producer of their input (RMSNorm, SiLU*up): codes, scales and the
optional bf16 by-product must be bit-identical to the oracle's producer followed by its quantizer."""
import pytest
import torch

from oracle import fpq_oracle as O
from tests import capi
from tests.conftest import make_outlier_normal, make_student_t

pytestmark = pytest.mark.gpu


def _oracle_quantize(v_bf16, fmt, rot, g, gs):
    kind = O.ROT_HADAMARD if rot == "hadamard" else O.ROT_IDENTITY
    norm = float(O.hadamard_matrix(g)[0, 0])
    if fmt == "mxfp4":
        q, s, _ = O.quantize_mx(v_bf16, kind, g, norm)
    else:
        q, s, _ = O.quantize_nv(v_bf16, gs, kind, g, norm)
    return q, s


@pytest.mark.parametrize("rows,cols,ld", [(1, 128, None), (37, 384, 512), (300, 4096, None)])
def test_row_inv_rms_bit_exact(rows, cols, ld):
    x = make_student_t(rows, cols, seed=rows)
    x[0, :8] = 0
    got = capi.row_inv_rms(x, 1e-5, ld)
    assert torch.equal(got, O.row_inv_rms(x, 1e-5))
    z = torch.zeros(3, cols, dtype=torch.bfloat16)
    assert torch.equal(capi.row_inv_rms(z, 1e-6), O.row_inv_rms(z, 1e-6))


CASES = [("mxfp4", "hadamard", 32), ("mxfp4", "hadamard", 128), ("mxfp4", "identity", 32),
         ("nvfp4", "hadamard", 16), ("nvfp4", "hadamard", 64), ("nvfp4", "identity", 16)]


@pytest.mark.parametrize("fmt,rot,g", CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (45, 384), (260, 1024)])
def test_rmsnorm_quantize_bit_exact(fmt, rot, g, rows, cols):
    x = make_outlier_normal(rows, cols, seed=rows + g) * 1.7
    gen = torch.Generator().manual_seed(cols)
    w = (1 + 0.3 * torch.randn(cols, generator=gen)).to(torch.bfloat16)
    eps = 1e-5
    want_v = O.rmsnorm(x, w, eps)
    gs = 1234.5 if fmt == "nvfp4" else None
    wq, ws = _oracle_quantize(want_v, fmt, rot, g, gs)
    codes, scales, out = capi.fused_quantize("rmsnorm", fmt, x, w, g=g, rot=rot, global_scale=gs, eps=eps,
                                             ld_a=cols + 64 if rows == 45 else None)
    assert torch.equal(out, want_v)
    assert torch.equal(codes, wq) and torch.equal(scales, ws)
    # without the by-product
    codes2, scales2, none = capi.fused_quantize("rmsnorm", fmt, x, w, g=g, rot=rot, global_scale=gs, eps=eps,
                                                want_out=False)
    assert none is None and torch.equal(codes2, wq) and torch.equal(scales2, ws)


@pytest.mark.parametrize("fmt,rot,g", CASES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (45, 384), (260, 1024)])
def test_silu_mul_quantize_bit_exact(fmt, rot, g, rows, cols):
    gate = make_student_t(rows, cols, seed=rows + g) * 2
    up = make_outlier_normal(rows, cols, seed=cols + g)
    # extremes of the activation: saturated both ways, zeros, the last finite binade of exp
    gate[0, :8] = torch.tensor([-300.0, 300.0, 0.0, -0.0, -88.5, 88.5, -20.0, 20.0]).to(torch.bfloat16)
    want_v = O.silu_mul(gate, up)
    gs = 777.0 if fmt == "nvfp4" else None
    wq, ws = _oracle_quantize(want_v, fmt, rot, g, gs)
    # gate and up as the two halves of one [rows, 2 * cols] tensor (a fused gate/up projection)
    both = torch.cat((gate, up), dim=1).cuda()
    if rows == 45:
        lib_args = dict(ld_a=2 * cols, ld_b=cols + 8)
    else:
        lib_args = {}
    codes, scales, out = capi.fused_quantize("silu_mul", fmt, gate, up, g=g, rot=rot, global_scale=gs, **lib_args)
    assert torch.equal(out.view(torch.int16), want_v.view(torch.int16))   # bit pattern: keeps -0 apart from +0
    assert torch.equal(codes, wq) and torch.equal(scales, ws)
    del both


def test_fused_quantize_argument_checks():
    from fp_quant import _engine
    lib = _engine.lib()
    x = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda")
    w = torch.ones(128, dtype=torch.bfloat16, device="cuda")
    inv = torch.ones(4, dtype=torch.float32, device="cuda")
    c = torch.zeros(4, 64, dtype=torch.uint8, device="cuda")
    s = torch.zeros(4, 4, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    ok = lib.fpq_rmsnorm_quantize_mx(x.data_ptr(), 128, inv.data_ptr(), w.data_ptr(), 4, 128, 0, 32, 0.177, None,
                                     c.data_ptr(), s.data_ptr(), 4, 4, 0, st)
    assert ok == 0
    # sequency-ordered and general rotations are not fused
    assert lib.fpq_rmsnorm_quantize_mx(x.data_ptr(), 128, inv.data_ptr(), w.data_ptr(), 4, 128, _engine.ROT_GSR, 32,
                                       0.177, None, c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == _engine.E_UNSUPPORTED
    # row stride smaller than the row, or not a multiple of 8
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 64, x.data_ptr(), 128, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -2
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 128, x.data_ptr(), 132, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -2
    assert lib.fpq_silu_mul_quantize_mx(x.data_ptr(), 128, None, 128, 4, 128, 0, 32, 0.177, None,
                                        c.data_ptr(), s.data_ptr(), 4, 4, 0, st) == -1
    assert lib.fpq_row_inv_rms(x.data_ptr(), 128, 4, 100, 1e-5, inv.data_ptr(), st) == -2
    torch.cuda.synchronize()
