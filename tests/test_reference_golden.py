"""Vectors produced by the reference's own PyTorch quantizer (tests/golden/reference_golden.npz, written
in the build container by tests/golden/make_reference_golden.py from src/quantization/{quant_args,
quant_ops,quantizer}.py and src/helpers.py of the reference).  The CPU tests pin the oracle to them, the
GPU tests the kernels (identity rotation: the rotation is not part of those modules).

The one documented exception: an NVFP4 group whose E4M3 scale rounds to zero.  The reference then
divides by 1 and stores the byte of e4m3(1 * global_scale) (src/quantization/quantizer.py:168,
src/quantization/rtn.py:188); the oracle and the kernels store byte 0.  Such a group holds only
zero codes on both sides, so the dequantized values agree."""
import os

import numpy as np
import pytest
import torch

from oracle import fpq_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_golden.npz"))
NV_CASES = ("tracked", "gs3", "gs10")


def _bf16(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _check_nv(codes, scales, tag):
    want_c, want_s = G[f"nv_{tag}_codes"], G[f"nv_{tag}_scales"]
    gs = float(G[f"nv_{tag}_global_scale"][0])
    assert np.array_equal(codes, want_c)
    differ = scales != want_s
    gs_byte = int(torch.tensor(gs).to(torch.float8_e4m3fn).view(torch.uint8))
    assert (scales[differ] == 0).all() and (want_s[differ] == gs_byte).all()
    assert (want_c.reshape(64, 16, 8)[differ] == 0x88).all()          # nothing but zero nibbles there
    assert ((scales == 0) == differ).all()                             # and every zero scale is such a group
    assert 0 < differ.sum() < 128 and (~differ).sum() > 900            # most groups are compared byte for byte


def test_oracle_mx_equals_reference_quantizer():
    c, s, _ = O.quantize_mx(_bf16(G["mx_x_bits"]), O.ROT_IDENTITY, 32)
    assert np.array_equal(c.numpy(), G["mx_codes"]) and np.array_equal(s.numpy(), G["mx_scales"])
    assert (G["mx_scales"] == 1).sum() >= 12                           # zero groups are in the vectors: byte 1


@pytest.mark.parametrize("tag", NV_CASES)
def test_oracle_nv_equals_reference_quantizer(tag):
    gs = float(G[f"nv_{tag}_global_scale"][0])
    c, s, _ = O.quantize_nv(_bf16(G["nv_x_bits"]), gs, O.ROT_IDENTITY, 16)
    _check_nv(c.numpy(), s.numpy(), tag)


def test_oracle_tracked_global_scale_equals_reference():
    # quantizer.py:145-150: 448 * 6 * (1 / max|x|), minimum over calls (one call here)
    assert np.float32(O.nv_tracked_global_scale(_bf16(G["nv_x_bits"]).float())) == G["nv_tracked_global_scale"][0]


def test_oracle_packing_equals_reference_pack_fp4_to_uint8():
    v = torch.from_numpy(G["pack_values"])
    assert np.array_equal(O.pack_nibbles(O.e2m1_codes(v, O.ZERO_NIBBLE_REFERENCE)).numpy(), G["pack_bytes"])


def test_oracle_rounding_equals_reference_cast_to_fp4():
    v = torch.from_numpy(G["fp4_in"])
    grid = torch.tensor(O.E2M1_VALUES[:8], dtype=torch.float32)
    got = grid[O.e2m1_round_rne(v).long()] * torch.sign(v)
    assert np.array_equal(got.numpy(), G["fp4_out"])


@pytest.mark.gpu
def test_kernel_mx_equals_reference_quantizer():
    import capi
    c, s = capi.quantize(_bf16(G["mx_x_bits"]), "mxfp4", "identity", 32)
    assert np.array_equal(c.numpy(), G["mx_codes"]) and np.array_equal(s.numpy(), G["mx_scales"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag", NV_CASES)
def test_kernel_nv_equals_reference_quantizer(tag):
    import capi
    gs = float(G[f"nv_{tag}_global_scale"][0])
    c, s = capi.quantize(_bf16(G["nv_x_bits"]), "nvfp4", "identity", 16, global_scale=gs)
    _check_nv(c.numpy(), s.numpy(), tag)


@pytest.mark.gpu
def test_streaming_kernels_equal_reference_quantizer():
    """The same vectors tiled to 8192 rows, which takes the streaming kernels (row-major and packed)."""
    import capi
    reps = 128
    x = _bf16(G["mx_x_bits"]).repeat(reps, 1)
    c, s = capi.quantize(x, "mxfp4", "identity", 32)
    assert np.array_equal(c.numpy(), np.tile(G["mx_codes"], (reps, 1)))
    assert np.array_equal(s.numpy(), np.tile(G["mx_scales"], (reps, 1)))
    pc, ps = capi.quantize_packed(x, rot="identity", g=32)
    wc, ws = capi.pack(torch.from_numpy(np.tile(G["mx_codes"], (reps, 1))), torch.from_numpy(np.tile(G["mx_scales"], (reps, 1))))
    assert torch.equal(pc, wc) and torch.equal(ps, ws)
    x = _bf16(G["nv_x_bits"]).repeat(reps, 1)
    gs = float(G["nv_gs10_global_scale"][0])
    c, s = capi.quantize(x, "nvfp4", "identity", 16, global_scale=gs)
    want_s = np.tile(G["nv_gs10_scales"], (reps, 1))
    assert np.array_equal(c.numpy(), np.tile(G["nv_gs10_codes"], (reps, 1)))
    assert np.array_equal(s.numpy()[s.numpy() != 0], want_s[s.numpy() != 0])
