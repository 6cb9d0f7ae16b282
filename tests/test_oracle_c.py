"""The plain-C restatement (oracle/fpq_oracle.c) and the torch restatement (oracle/fpq_oracle.py)
were written independently; they must agree byte for byte on random, adversarial and tiny inputs."""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from conftest import make_outlier_normal, make_student_t
from oracle import fpq_oracle as O

ORACLE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")


@pytest.fixture(scope="module")
def clib():
    path = os.path.join(ORACLE_DIR, "libfpq_oracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR])
    lib = ctypes.CDLL(path)
    lib.fpq_oracle_quantize.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_long, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p]
    return lib


def _c_quantize(lib, x, fmt, rot, g, gs, zero):
    rows, cols = x.shape
    group = 32 if fmt == 0 else 16
    xb = x.contiguous().view(torch.int16).numpy()
    codes = np.zeros((rows, cols // 2), dtype=np.uint8)
    scales = np.zeros((rows, cols // group), dtype=np.uint8)
    norm = float(O.hadamard_matrix(g)[0, 0])
    st = lib.fpq_oracle_quantize(xb.ctypes.data, rows, cols, fmt, rot, g, norm, gs, zero,
                                 codes.ctypes.data, scales.ctypes.data)
    assert st == 0
    return codes, scales


def _adversarial():
    gen = torch.Generator().manual_seed(4)
    base = torch.randn(256, generator=gen)
    rows = [torch.zeros(256), base, base * 1e-30, base * 1e-38, base * 1e30, base * 3e37,
            torch.full((256,), 2.0), torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 32),
            -torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 32) * 8]
    r = base.clone(); r[:96] = 0; rows.append(r)
    r = torch.zeros(256); r[::2] = -0.0; r[7] = 1.0; rows.append(r)
    return torch.stack(rows).to(torch.bfloat16)


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("zero", [0, 1])
def test_mx_c_equals_torch(clib, g, zero):
    for x in (make_outlier_normal(64, 512, seed=g), _adversarial()):
        c, s, _ = O.quantize_mx(x, O.ROT_HADAMARD, g, zero_nibble=zero)
        cc, cs = _c_quantize(clib, x, 0, 0, g, 0.0, zero)
        assert np.array_equal(c.numpy(), cc) and np.array_equal(s.numpy(), cs)
    x = _adversarial()
    c, s, _ = O.quantize_mx(x, O.ROT_IDENTITY, 32, zero_nibble=zero)
    cc, cs = _c_quantize(clib, x, 0, 1, 32, 0.0, zero)
    assert np.array_equal(c.numpy(), cc) and np.array_equal(s.numpy(), cs)


@pytest.mark.parametrize("g", [16, 32, 128])
@pytest.mark.parametrize("gs", [3.0, 10.0, 2688.0 / 13.0, 1e-3, 1e-25])
def test_nv_c_equals_torch(clib, g, gs):
    for zero in (0, 1):
        for x in (make_student_t(64, 512, seed=g), _adversarial()):
            c, s, _ = O.quantize_nv(x, gs, O.ROT_HADAMARD, g, zero_nibble=zero)
            cc, cs = _c_quantize(clib, x, 1, 0, g, gs, zero)
            assert np.array_equal(c.numpy(), cc) and np.array_equal(s.numpy(), cs)
