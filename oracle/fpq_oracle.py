"""CPU oracle for the FP-Quant inference hot path (TEST INFRASTRUCTURE, NOT PRODUCT).

This module restates, on the CPU and in IEEE fp32, the arithmetic of the reference's
rotate -> group-scale -> E2M1 round -> pack path and of its W4A4 linear.  It exists only
so that tests, the smoke check and the benchmark's CPU-baseline leg can check the HIP
kernels; nothing in the shipped package may import it.

What it follows (all paths relative to the reference checkout):

* rotation matrix ............ inference_lib/src/fp_quant/module/linear.py:24-41
* group reshape .............. src/helpers.py:14-18, src/quantization/quantizer.py:71-85
* abs-max scale .............. src/quantization/quantizer.py:107-112
* E8M0 (MXFP4) scale ......... src/quantization/quantizer.py:162-165,
                               src/quantization/quant_ops.py:82-94
* E4M3 (NVFP4) scale ......... src/quantization/quantizer.py:143-160,168
* E2M1 round to nearest even . src/quantization/quant_ops.py:57-68
* nibble packing ............. src/quantization/quant_ops.py:15-16,31-40
* stored scale bytes ......... src/quantization/rtn.py:187-188,
                               src/quantization/quant_ops.py:111-118
* quest scale + clip mask .... inference_lib/src/fp_quant/module/triton/mxfp4.py:51-59,105-110,
                               inference_lib/src/fp_quant/module/pseudoquant_linear_fns.py:20-22,
                               inference_lib/src/fp_quant/module/linear_fns.py:67-76
* producers of x ............. src/utils/llama_utils.py:60-71 (act_fn(gate) * up before down_proj;
                               RMSNorm before the q/k/v and gate/up quantizers)
* linear ..................... inference_lib/src/fp_quant/module/linear_fns.py:496-514,
                               inference_lib/src/fp_quant/module/qutlass_ops.py:111-168

Canonical choices where the reference's own statements of the math disagree with each
other (fp32 everywhere, bf16 only at the input and at the rotation matrix entries):

* rotation = sum of exact products x[i]*H[i,j] accumulated by radix-2 butterflies with
  strides 1, 2, 4, ..., g/2 (fp32 add/sub, one rounding per butterfly output);
* floor(log2(.)) is taken from the exponent field, never from a libm log2;
* E2M1 rounding is round-to-nearest-even (the PyTorch statement), not the Triton ladder;
* a zero E4M3 scale stores byte 0 with all-zero codes (the reference would store
  e4m3(1*global_scale)); this is a deliberate, documented deviation;
* the zero nibble is a named policy: ZERO_NIBBLE_REFERENCE packs every zero as 0x8 (what
  pack_fp4_to_uint8 does because torch.bucketize(0.0, grid) == 7), ZERO_NIBBLE_SIGNED
  keeps the sign bit of the scaled value (what a hardware cvt does).

Pin status (each function below is checked in tests/test_oracle_*.py against closed
forms, exhaustive tables, library casts or brute force): rotation, E8M0 exponent, E2M1 RNE, packing, E4M3 cast, E8M0 cast, GEMM, the quest
scale (against numpy float64 statistics and a per-group Python loop) and clip mask; the two
producers (silu_mul, rmsnorm) against float64 evaluations and torch's own operators.
tests/test_reference_golden.py additionally pins quantize_mx, quantize_nv, nv_tracked_global_scale,
e2m1_round_rne, e2m1_codes and pack_nibbles to bytes written by the reference's own modules
(src/quantization/{quant_args,quant_ops,quantizer}.py, src/helpers.py, loaded by file path in the
build container by tests/golden/make_reference_golden.py); the only difference is the documented
zero-scale deviation above.
The third-party kernels the reference calls for this path (QuTLASS, un-vendored, version
unpinned) have no fixtures in the reference: bit parity against QuTLASS itself is unpinned.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

# ----------------------------------------------------------------------------- constants
FP4_E2M1_MAX = 6.0
FP8_E4M3_MAX = 448.0
NVFP_GROUPSIZE = 16
MXFP_GROUPSIZE = 32
FP32_MIN_NORMAL = 2.0 ** -126
FP4_SCALE = 0.75  # quant_ops.py:17

# code -> value (quant_ops.py:15-16: grid value g has code perm[g])
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
               -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)

ZERO_NIBBLE_REFERENCE = 0  # every zero packs as 0x8
ZERO_NIBBLE_SIGNED = 1     # sign bit of the scaled value is kept (+0 -> 0x0, -0 -> 0x8)

ROT_HADAMARD = 0
ROT_IDENTITY = 1
ROT_GSR = 2
ROT_GENERAL = 3


# ----------------------------------------------------------------------------- rotation
def sylvester_signs(g: int) -> np.ndarray:
    """+-1 Sylvester-Hadamard matrix, H[i, j] = (-1)^popcount(i & j)."""
    idx = np.arange(g)
    anded = idx[:, None] & idx[None, :]
    pop = np.zeros_like(anded)
    for b in range(max(1, g.bit_length())):
        pop += (anded >> b) & 1
    return (1 - 2 * (pop & 1)).astype(np.float64)


def hadamard_matrix(g: int, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """linear.py:24-30: hadamard(g) * g**-0.5 cast to the weight dtype."""
    return torch.tensor(sylvester_signs(g) * g ** -0.5, dtype=dtype)


def identity_matrix(g: int, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """linear.py:33-34."""
    return torch.eye(g, dtype=dtype)


def gsr_permutation(g: int) -> np.ndarray:
    """Column order of the GSR matrix: argsort of the number of sign changes per column
    (linear.py:37-41).  All counts are distinct (0..g-1), so the order is unambiguous."""
    signs = sylvester_signs(g)
    changes = (np.diff(signs, axis=0) != 0).sum(axis=0)
    return np.argsort(changes, kind="stable")


def gsr_matrix(g: int, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    h = hadamard_matrix(g, dtype)
    return h[:, torch.from_numpy(gsr_permutation(g))].contiguous()


def classify_rotation(h: torch.Tensor) -> Tuple[int, float]:
    """Recognise a [g, g] rotation matrix as +-norm Sylvester (ROT_HADAMARD), its
    sequency-ordered column permutation (ROT_GSR), the identity, or none of them."""
    g = h.shape[0]
    hf = h.detach().to(torch.float32).cpu()
    if torch.equal(hf, torch.eye(g)):
        return ROT_IDENTITY, 1.0
    norm = float(hf[0, 0])
    signs = torch.from_numpy(sylvester_signs(g)).to(torch.float32)
    if norm != 0.0 and torch.equal(hf, signs * norm):
        return ROT_HADAMARD, norm
    if norm != 0.0 and torch.equal(hf, (signs * norm)[:, torch.from_numpy(gsr_permutation(g))]):
        return ROT_GSR, norm
    return ROT_GENERAL, 0.0


def fwht_fp32(p: torch.Tensor, g: int) -> torch.Tensor:
    """In-place-order Sylvester FWHT over contiguous g-chunks of the last dim, fp32,
    butterfly strides 1, 2, ..., g/2; pair (i, i+s) with (i & s) == 0 -> (a+b, a-b)."""
    assert p.dtype == torch.float32
    shape = p.shape
    v = p.reshape(-1, g)
    s = 1
    while s < g:
        w = v.view(-1, g // (2 * s), 2, s)
        a = w[:, :, 0, :]
        b = w[:, :, 1, :]
        v = torch.stack((a + b, a - b), dim=2).reshape(-1, g)
        s *= 2
    return v.reshape(shape)


def rotate(x: torch.Tensor, kind: int, g: int, norm: float = 0.0,
           h: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (bf16-representable) times block-diag(H), fp32 result, not re-rounded to bf16.

    HADAMARD / GSR: p = fp32(x) * norm (exact for bf16 x and bf16 norm), butterflies,
    GSR then permutes the outputs of every g-chunk.  GENERAL: y[j] = sum_i x[i] * H[i, j]
    accumulated sequentially over i = 0..g-1 with fp32 fused multiply-adds."""
    xf = x.detach().to(torch.float32).cpu().contiguous()
    assert xf.shape[-1] % g == 0
    if kind == ROT_IDENTITY:
        return xf.clone()
    if kind in (ROT_HADAMARD, ROT_GSR):
        y = fwht_fp32(xf * torch.tensor(norm, dtype=torch.float32), g)
        if kind == ROT_GSR:
            perm = torch.from_numpy(gsr_permutation(g))
            y = y.reshape(-1, g)[:, perm].reshape(xf.shape)
        return y.contiguous()
    if kind == ROT_GENERAL:
        assert h is not None
        hf = h.detach().to(torch.float32).cpu().numpy().astype(np.float64)
        v = xf.reshape(-1, g).numpy().astype(np.float64)
        acc = np.zeros_like(v, dtype=np.float32)
        for i in range(g):
            # fp32 fma: the product of two bf16-representable numbers is exact in fp64,
            # and fp64 add of an fp32 and that product followed by one rounding to fp32
            # is a correctly rounded fma (no double rounding: 53 >= 2*24 + 2).
            acc = (acc.astype(np.float64) + v[:, i:i + 1] * hf[i:i + 1, :]).astype(np.float32)
        return torch.from_numpy(acc).reshape(xf.shape)
    raise ValueError(f"unknown rotation kind {kind}")


def rotate_matmul_fp64(x: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    """Order-free cross-check of the rotation: x.view(-1, g) @ H in fp64."""
    g = h.shape[0]
    xf = x.detach().to(torch.float64).cpu()
    return (xf.reshape(-1, g) @ h.detach().to(torch.float64).cpu()).reshape(xf.shape)


# ----------------------------------------------------------------------------- scalar casts
def floor_log2_exact(a: torch.Tensor) -> torch.Tensor:
    """floor(log2(a)) for positive finite fp32 a, from the exponent field (subnormals via frexp)."""
    assert a.dtype == torch.float32
    _, ex = torch.frexp(a)  # a = m * 2**ex, 0.5 <= m < 1
    return (ex - 1).to(torch.int32)


def e2m1_round_rne(v: torch.Tensor) -> torch.Tensor:
    """Magnitude index 0..7 of round-to-nearest-even on the E2M1 grid (quant_ops.py:57-68),
    saturating above 5."""
    a = v.abs()
    idx = torch.zeros(a.shape, dtype=torch.int32)
    idx[(a > 0.25) & (a < 0.75)] = 1
    idx[(a >= 0.75) & (a <= 1.25)] = 2
    idx[(a > 1.25) & (a < 1.75)] = 3
    idx[(a >= 1.75) & (a <= 2.5)] = 4
    idx[(a > 2.5) & (a < 3.5)] = 5
    idx[(a >= 3.5) & (a <= 5.0)] = 6
    idx[a > 5.0] = 7
    return idx


def e2m1_codes(v: torch.Tensor, zero_nibble: int = ZERO_NIBBLE_REFERENCE) -> torch.Tensor:
    """4-bit codes (uint8 in 0..15) of the scaled values v; sign is bit 3."""
    mag = e2m1_round_rne(v)
    if zero_nibble == ZERO_NIBBLE_REFERENCE:
        neg = (v < 0) | (mag == 0)
    elif zero_nibble == ZERO_NIBBLE_SIGNED:
        neg = torch.signbit(v)
    else:
        raise ValueError("bad zero nibble policy")
    return (mag | (neg.to(torch.int32) << 3)).to(torch.uint8)


def pack_nibbles(codes: torch.Tensor) -> torch.Tensor:
    """Two codes per byte, even element in the low nibble (quant_ops.py:40)."""
    return (codes[..., 1::2] << 4 | codes[..., 0::2]).to(torch.uint8)


def unpack_nibbles(packed: torch.Tensor) -> torch.Tensor:
    lo = packed & 0xF
    hi = packed >> 4
    return torch.stack((lo, hi), dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def e4m3_encode(t: torch.Tensor) -> torch.Tensor:
    """fp32 -> float8_e4m3fn byte: RNE, subnormals down to 2^-9, |t| in (448, 464] -> 448,
    above -> NaN byte 0x7f, written out by hand (checked against torch's cast in the tests)."""
    assert t.dtype == torch.float32
    a = t.abs().to(torch.float64)
    sign = torch.signbit(t).to(torch.int32) << 7
    out = torch.zeros(t.shape, dtype=torch.int32)
    # spacing: subnormal region [0, 2^-6): 2^-9 ; normal binade [2^e, 2^(e+1)): 2^(e-3)
    _, ex = torch.frexp(a)
    e = (ex - 1).clamp(min=-6)
    step = torch.ldexp(torch.ones_like(a), (e - 3).to(torch.int32))
    k = a / step                         # exact: division by a power of two
    kr = torch.round(k)                  # torch.round is round-half-to-even
    val = kr * step
    # re-derive exponent/mantissa of the rounded value
    _, ex2 = torch.frexp(val)
    e2 = ex2 - 1
    normal = val >= 2.0 ** -6
    mant_n = (val / torch.ldexp(torch.ones_like(a), (e2 - 3).to(torch.int32))).to(torch.int32) - 8
    byte_n = ((e2 + 7).to(torch.int32) << 3) | mant_n
    byte_s = (val / 2.0 ** -9).to(torch.int32)
    out = torch.where(normal, byte_n, byte_s)
    out = torch.where(val > 448.0, torch.full_like(out, 0x7F), out)
    out = torch.where(torch.isnan(t), torch.full_like(out, 0x7F), out)
    return (out | sign).to(torch.uint8)


def e4m3_decode(b: torch.Tensor) -> torch.Tensor:
    bi = b.to(torch.int32)
    sign = 1.0 - 2.0 * ((bi >> 7) & 1).to(torch.float32)
    ex = (bi >> 3) & 0xF
    man = (bi & 7).to(torch.float32)
    normal = torch.ldexp(1.0 + man / 8.0, ex - 7)
    sub = man * 2.0 ** -9
    v = torch.where(ex == 0, sub, normal)
    v = torch.where((bi & 0x7F) == 0x7F, torch.full_like(v, float("nan")), v)
    return (sign * v).to(torch.float32)


def e8m0_encode(t: torch.Tensor) -> torch.Tensor:
    """fp32 (>= 0) -> float8_e8m0fnu byte: nearest power of two in the mantissa, halves
    round up; results below 2^-127 give byte 0; NaN/overflow give 255 (as torch's cast)."""
    assert t.dtype == torch.float32
    bits = t.contiguous().view(torch.int32)
    ex = (bits >> 23) & 0xFF
    man = bits & 0x7FFFFF
    up = (man >= 0x400000).to(torch.int32)
    byte = ex + up
    # subnormal inputs: value = man * 2^-149; >= 2^-127 (man >= 2^22) rounds to 2^-127 or 2^-126
    sub = ex == 0
    byte_sub = torch.where(man >= 0x600000, torch.ones_like(byte), torch.zeros_like(byte))
    byte = torch.where(sub, byte_sub, byte)
    byte = byte.clamp(max=255)
    byte = torch.where(torch.isnan(t), torch.full_like(byte, 255), byte)
    return byte.to(torch.uint8)


def e8m0_decode(b: torch.Tensor) -> torch.Tensor:
    return torch.ldexp(torch.ones(b.shape, dtype=torch.float32), b.to(torch.int32) - 127)


# ----------------------------------------------------------------------------- quantizers
def mx_scales_from_absmax(a: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Working scale s (fp32) and stored E8M0 byte for group abs-max a (fp32).

    quantizer.py:111 -> 2*a/12 ; :165 -> cast_to_eBm0(6*that, ebits=8, emax=2) / 0.75 ;
    quant_ops.py:94 -> 2 ** (floor(log2(clamp(., min=2^-126))).clamp(-127, 127) - 2) ;
    rtn.py:188 -> stored = e8m0(s * 3.0) (global scale 3.0, quantizer.py:64-65)."""
    f32 = torch.float32
    sc = (a * torch.tensor(2.0, dtype=f32)) / torch.tensor(12.0, dtype=f32)
    arg = (sc * torch.tensor(FP4_E2M1_MAX, dtype=f32)).clamp(min=FP32_MIN_NORMAL)
    e = floor_log2_exact(arg).clamp(-127, 127)
    pow2 = torch.ldexp(torch.ones_like(arg), e - 2)
    s = pow2 / torch.tensor(FP4_SCALE, dtype=f32)
    s = torch.where(s == 0, torch.ones_like(s), s)
    stored = e8m0_encode(s * torch.tensor(3.0, dtype=f32))
    return s, stored


def quantize_mx(x: torch.Tensor, kind: int = ROT_HADAMARD, g: int = 128,
                norm: Optional[float] = None, h: Optional[torch.Tensor] = None,
                zero_nibble: int = ZERO_NIBBLE_REFERENCE):
    """MXFP4 abs-max rotate+quantize of a [R, C] bf16 tensor.

    Returns (packed codes uint8 [R, C/2], E8M0 bytes uint8 [R, C/32], rotated fp32 [R, C])."""
    if norm is None:
        norm = float(hadamard_matrix(g)[0, 0])
    xr = rotate(x, kind, g, norm, h)
    r, c = xr.shape
    xg = xr.view(r, c // MXFP_GROUPSIZE, MXFP_GROUPSIZE)
    a = torch.maximum(-xg.amin(dim=-1), xg.amax(dim=-1))
    s, stored = mx_scales_from_absmax(a)
    v = xg / s.unsqueeze(-1)
    codes = e2m1_codes(v, zero_nibble).view(r, c)
    return pack_nibbles(codes), stored, xr


QUEST_GAUSSIAN_SCALE = 2.92247856 / 6.0  # pseudoquant_linear_fns.py:20-22


def quest_scales(xg: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Working scale s = 2^floor(log2(fl32(2.92247856/6)*std + 1e-8)) and its E8M0 byte for
    groups xg [..., 32] of rotated fp32 values (module/triton/mxfp4.py:51-59).

    Triton leaves the order of its reductions open; the canonical order here (the one the HIP
    kernel uses): per octet of consecutive elements the sums of x and of fl(x*x) run left to
    right, the four octet sums combine as (o0 + o1) + (o2 + o3); mean = sum/32,
    var = max(mean_sq - fl(mean*mean), 0) (the clamp keeps a constant group from producing
    sqrt of a negative rounding residue; the reference would return NaN there)."""
    f32 = torch.float32
    assert xg.dtype == f32 and xg.shape[-1] == 32
    oct_ = xg.reshape(*xg.shape[:-1], 4, 8)
    sq8 = oct_ * oct_
    s_sum, s_sq = oct_[..., 0].clone(), sq8[..., 0].clone()
    for i in range(1, 8):
        s_sum = s_sum + oct_[..., i]
        s_sq = s_sq + sq8[..., i]
    tot = (s_sum[..., 0] + s_sum[..., 1]) + (s_sum[..., 2] + s_sum[..., 3])
    tot_sq = (s_sq[..., 0] + s_sq[..., 1]) + (s_sq[..., 2] + s_sq[..., 3])
    mean = tot * torch.tensor(0.03125, dtype=f32)
    msq = tot_sq * torch.tensor(0.03125, dtype=f32)
    var = (msq - mean * mean).clamp_min(0.0)
    # numpy's sqrt is the correctly rounded one on every machine (torch's vectorised CPU sqrt is not)
    std = torch.from_numpy(np.sqrt(var.contiguous().numpy()))
    sc = std * torch.tensor(QUEST_GAUSSIAN_SCALE, dtype=f32) + torch.tensor(1e-8, dtype=f32)
    e = floor_log2_exact(sc)
    s = torch.ldexp(torch.ones_like(sc), e)
    return s, (e + 127).to(torch.uint8)


def quantize_mx_quest(x: torch.Tensor, kind: int = ROT_HADAMARD, g: int = 128,
                      norm: Optional[float] = None, h: Optional[torch.Tensor] = None,
                      zero_nibble: int = ZERO_NIBBLE_REFERENCE):
    """MXFP4 "quest" rotate+quantize of a [R, C] bf16 tensor (mxfp4.py:51-59,105-110).

    Returns (packed codes uint8 [R, C/2], E8M0 bytes uint8 [R, C/32], clip mask uint8 [R, C/8]
    with bit (c % 8) of byte [r, c/8] set where |x/s| < 6 (linear_fns.py:67-76), rotated fp32)."""
    if norm is None:
        norm = float(hadamard_matrix(g)[0, 0])
    xr = rotate(x, kind, g, norm, h)
    r, c = xr.shape
    xg = xr.view(r, c // MXFP_GROUPSIZE, MXFP_GROUPSIZE)
    s, stored = quest_scales(xg)
    v = xg / s.unsqueeze(-1)
    codes = e2m1_codes(v, zero_nibble).view(r, c)  # magnitudes above 5 saturate at 6: the clip
    inside = (v.abs() < 6.0).view(r, c // 8, 8).to(torch.int32)
    mask = (inside << torch.arange(8, dtype=torch.int32)).sum(dim=-1).to(torch.uint8)
    return pack_nibbles(codes), stored, mask, xr


def nv_scales_from_absmax(a: torch.Tensor, global_scale: float):
    """Working scale sw (fp32, zero where the E4M3 scale is zero) and stored E4M3 byte.

    quantizer.py:111 -> sc0 = 2*a/12 ; :153-157 -> e4m3(clamp(sc0*gs, +-448)) back to
    fp32, times fl(1/gs) ; rtn.py:188 -> stored = e4m3(sw * gs)."""
    f32 = torch.float32
    gs = torch.tensor(global_scale, dtype=f32)
    rg = torch.where(gs == 0, torch.zeros_like(gs), torch.tensor(1.0, dtype=f32) / gs)
    sc0 = (a * torch.tensor(2.0, dtype=f32)) / torch.tensor(12.0, dtype=f32)
    t = (sc0 * gs).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX)
    sc = e4m3_decode(e4m3_encode(t))
    sw = sc * rg
    stored = e4m3_encode(sw * gs)
    stored = torch.where(sw == 0, torch.zeros_like(stored), stored)
    return sw, stored


def quantize_nv(x: torch.Tensor, global_scale: float, kind: int = ROT_HADAMARD, g: int = 16,
                norm: Optional[float] = None, h: Optional[torch.Tensor] = None,
                zero_nibble: int = ZERO_NIBBLE_REFERENCE):
    """NVFP4 rotate+quantize with a given fp32 per-tensor global scale.

    Returns (packed codes uint8 [R, C/2], E4M3 bytes uint8 [R, C/16], rotated fp32 [R, C])."""
    if norm is None:
        norm = float(hadamard_matrix(g)[0, 0])
    xr = rotate(x, kind, g, norm, h)
    r, c = xr.shape
    xg = xr.view(r, c // NVFP_GROUPSIZE, NVFP_GROUPSIZE)
    a = torch.maximum(-xg.amin(dim=-1), xg.amax(dim=-1))
    sw, stored = nv_scales_from_absmax(a, global_scale)
    zero_group = sw == 0
    sw_div = torch.where(zero_group, torch.ones_like(sw), sw)
    v = xg / sw_div.unsqueeze(-1)
    v = torch.where(zero_group.unsqueeze(-1), torch.zeros_like(v), v)
    codes = e2m1_codes(v, zero_nibble).view(r, c)
    return pack_nibbles(codes), stored, xr


def nv_tracked_global_scale(xr: torch.Tensor) -> float:
    """quantizer.py:145-150 with the tracker starting at +inf: 448*6 * fl(1/absmax)."""
    f32 = torch.float32
    amax = xr.abs().max().to(f32)
    rec = torch.where(amax == 0, torch.zeros_like(amax), torch.tensor(1.0, dtype=f32) / amax)
    return float(torch.tensor(FP8_E4M3_MAX * FP4_E2M1_MAX, dtype=f32) * rec)


# ----------------------------------------------------------------------------- producers of x
# The two elementwise producers whose output the quantizer consumes in a Llama block
# (src/utils/llama_utils.py:60-71: act_fn(gate) * up feeds down_proj's quantizer; the block's
# RMSNorm output feeds the q/k/v and gate/up quantizers), stated so that fusing them into the
# quantize kernel is checkable bit for bit: bf16 in, bf16 out, every intermediate an IEEE fp32
# operation in a fixed order (no fused multiply-add, no library exp).
EXP_LOG2E = np.float32(1.44269504088896341)
EXP_LN2_HI = np.float32(0.693359375)           # 9 significant bits: n * hi is exact
EXP_LN2_LO = np.float32(-2.12194440e-4)
EXP_POLY = tuple(np.float32(c) for c in (1.9875691500e-4, 1.3981999507e-3, 8.3334519073e-3,
                                         4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1))


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    """fp32 -> nearest-even bf16 -> fp32."""
    return t.to(torch.float32).to(torch.bfloat16).to(torch.float32)


def exp_det(t: torch.Tensor) -> torch.Tensor:
    """exp(t) in fp32 by a fixed operation sequence: clamp to +-200, n = rint(t * log2e),
    r = (t - n*ln2_hi) - n*ln2_lo, degree-5 polynomial in Horner form with separate multiply and
    add, y = (p*r*r + r) + 1, result = ldexp(y, n) (overflows to inf, underflows gradually)."""
    a = t.to(torch.float32).clamp(-200.0, 200.0).numpy()
    n = np.rint(a * EXP_LOG2E).astype(np.float32)
    r = (a - n * EXP_LN2_HI) - n * EXP_LN2_LO
    p = np.full_like(r, EXP_POLY[0])
    for c in EXP_POLY[1:]:
        p = p * r + c
    y = (p * (r * r) + r) + np.float32(1.0)
    with np.errstate(over="ignore", under="ignore"):
        out = np.ldexp(y, n.astype(np.int32)).astype(np.float32)
    return torch.from_numpy(out)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """bf16(bf16(silu(gate)) * up) with silu(g) = g / (1 + exp_det(-g)) in fp32: the bf16 tensor
    `act_fn(gate) * up` of a Llama MLP (one rounding per PyTorch operator)."""
    g = gate.to(torch.float32)
    with np.errstate(over="ignore"):
        d = torch.from_numpy(np.float32(1.0) + exp_det(-g).numpy())
    s = bf16_round(g / d)
    return (s * up.to(torch.float32)).to(torch.bfloat16)


def row_inv_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """1 / sqrt(mean(x^2) + eps) per row in fp32.  Summation order: squares of 8 consecutive elements
    left to right; those octet sums are dealt to 64 accumulators (octet c to accumulator c % 64, in
    increasing c); the accumulators combine by the butterfly a[i] += a[i ^ m], m = 1, 2, ..., 32."""
    xf = x.to(torch.float32)
    rows, cols = xf.shape
    sq = (xf * xf).view(rows, cols // 8, 8)
    octet = sq[..., 0].clone()
    for i in range(1, 8):
        octet = octet + sq[..., i]
    n_oct = cols // 8
    pad = (-n_oct) % 64
    if pad:
        octet = torch.cat((octet, torch.zeros(rows, pad)), dim=1)
    acc = torch.zeros(rows, 64)
    for it in range(octet.shape[1] // 64):
        acc = acc + octet[:, 64 * it: 64 * it + 64]
    idx = torch.arange(64)
    for m in (1, 2, 4, 8, 16, 32):
        acc = acc + acc[:, idx ^ m]
    # numpy for the correctly rounded division and square root (torch's CPU sqrt is vectorised
    # differently from machine to machine and is not always the correctly rounded one)
    total = acc[:, 0].contiguous().numpy()
    mean = total / np.float32(cols)
    inv = np.float32(1.0) / np.sqrt(mean + np.float32(eps))
    return torch.from_numpy(inv.astype(np.float32))


def rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """bf16(gamma * bf16(x * inv_rms)): RMSNorm as a Llama block applies it to bf16 activations
    (normalised value rounded to bf16, then the bf16 product with the weight)."""
    r = row_inv_rms(x, eps)
    n1 = bf16_round(x.to(torch.float32) * r.unsqueeze(-1))
    return (n1 * gamma.to(torch.float32)).to(torch.bfloat16)


# ----------------------------------------------------------------------------- dequantize / linear
def dequantize(packed: torch.Tensor, scale_bytes: torch.Tensor, fmt: str) -> torch.Tensor:
    """fp64 values code * scale for packed [R, C/2] codes and [R, C/group] scale bytes
    (extra padded rows/cols of the scale tensor are ignored)."""
    lut = torch.tensor(E2M1_VALUES, dtype=torch.float64)
    codes = unpack_nibbles(packed.cpu())
    r, c = codes.shape
    group = MXFP_GROUPSIZE if fmt == "mxfp4" else NVFP_GROUPSIZE
    sb = scale_bytes.cpu().view(torch.uint8)[:r, : c // group]
    sc = (e8m0_decode(sb) if fmt == "mxfp4" else e4m3_decode(sb)).to(torch.float64)
    vals = lut[codes.long()].view(r, c // group, group) * sc.unsqueeze(-1)
    return vals.view(r, c)


def gemm_ref(xq, xs, wq, ws, alpha: float, fmt: str, bias: Optional[torch.Tensor] = None):
    """(y fp64, mag fp64): y = alpha * dq(x) @ dq(w).T (+ bias), mag = alpha * |dq(x)| @ |dq(w)|.T
    (the magnitude sum the stated GEMM tolerance is relative to)."""
    dx = dequantize(xq, xs, fmt)
    dw = dequantize(wq, ws, fmt)
    y = alpha * (dx @ dw.T)
    mag = abs(alpha) * (dx.abs() @ dw.abs().T)
    if bias is not None:
        y = y + bias.detach().to(torch.float64).cpu()
    return y, mag


def alpha_from_global_scales(wgs: torch.Tensor, ags: torch.Tensor) -> float:
    """linear_fns.py:508: 1.0 / (wgs * ags) evaluated in the buffers' dtype, then .float()."""
    return float((1.0 / (wgs * ags)).float())
