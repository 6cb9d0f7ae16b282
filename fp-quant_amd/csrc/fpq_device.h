// Device-side scalar building blocks shared by the quantize and GEMM kernels (gfx950 only).
//
// All arithmetic here is IEEE fp32 with round-to-nearest-even and denormals kept; the
// translation units are built with -ffp-contract=off so every fused multiply-add in this
// file is written explicitly.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fpq {

constexpr int kZeroReference = 0;  // every zero packs as 0x8 (src/quantization/quant_ops.py:31-40)
constexpr int kZeroSigned = 1;     // the sign bit of the scaled value is kept

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Magnitude index 0..7 of |v| rounded to nearest-even on the E2M1 grid {0,.5,1,1.5,2,3,4,6}
// (src/quantization/quant_ops.py:57-68: ties 0.25->0, 0.75->1, 1.25->1, 1.75->2, 2.5->2,
// 3.5->4, 5->4; above 5 saturates to 6).
__device__ __forceinline__ uint32_t e2m1_mag(float a) {
  return (uint32_t)(a > 0.25f) + (uint32_t)(a >= 0.75f) + (uint32_t)(a > 1.25f) +
         (uint32_t)(a >= 1.75f) + (uint32_t)(a > 2.5f) + (uint32_t)(a >= 3.5f) +
         (uint32_t)(a > 5.0f);
}

template <int ZERO>
__device__ __forceinline__ uint32_t e2m1_code(float v) {
  const uint32_t mag = e2m1_mag(__builtin_fabsf(v));
  uint32_t neg;
  if (ZERO == kZeroReference) {
    neg = (uint32_t)((v < 0.0f) | (mag == 0u));
  } else {
    neg = __float_as_uint(v) >> 31;
  }
  return mag | (neg << 3);
}

// fp32 -> float8_e4m3fn byte, round-to-nearest-even, subnormals down to 2^-9,
// (448, 464] -> 448, above 464 and NaN -> 0x7f (what torch's cast does;
// src/quantization/quant_ops.py:113-114).
__device__ __forceinline__ uint32_t e4m3_encode(float t) {
  const uint32_t sign = (__float_as_uint(t) >> 24) & 0x80u;
  const float a = __builtin_fabsf(t);
  uint32_t byte;
  if (!(a <= 464.0f)) {
    byte = 0x7fu;
  } else if (a < 0.015625f) {
    byte = (uint32_t)__builtin_rintf(a * 512.0f);  // multiples of 2^-9; 8 is the first normal
  } else {
    uint32_t b = __float_as_uint(a);
    b += 0x7ffffu + ((b >> 20) & 1u);
    byte = (b >> 20) - ((127u - 7u) << 3);
  }
  return byte | sign;
}

__device__ __forceinline__ float e4m3_decode(uint32_t byte) {
  const uint32_t mag = byte & 0x7fu;
  float v;
  if (mag < 8u) {
    v = (float)mag * 0.001953125f;
  } else {
    v = __uint_as_float((mag << 20) + ((127u - 7u) << 23));
  }
  return (byte & 0x80u) ? -v : v;
}

// fp32 (>= 0) -> float8_e8m0fnu byte as torch's cast does it: nearest power of two with
// halves rounding up, below 2^-127 -> 0 (src/quantization/quant_ops.py:115-117).
__device__ __forceinline__ uint32_t e8m0_encode(float t) {
  const uint32_t b = __float_as_uint(t);
  const uint32_t ex = (b >> 23) & 0xffu;
  const uint32_t man = b & 0x7fffffu;
  uint32_t byte;
  if (ex == 0u) {
    byte = man >= 0x600000u ? 1u : 0u;
  } else {
    byte = ex + (man >= 0x400000u ? 1u : 0u);
    byte = byte > 255u ? 255u : byte;
  }
  return byte;
}

// ---------------------------------------------------------------------------------------------
// Per-group scale parameters.  The element step is  v = fma(x, k1, x * k2)  on the fast path,
// which yields the same E2M1 code as the correctly rounded quotient x / s for every x (proved
// by exhaustion over all divisor mantissas on the host: tests/div_equivalence.c), or the IEEE quotient x / s itself on
// the slow path taken for extreme exponents.
struct GroupScale {
  float k1;      // fast: RN(1/s)            slow: s
  float k2;      // fast: RN((1 - s*k1)/s)   slow: unused
  uint32_t byte; // stored scale byte
  bool slow;     // use the IEEE quotient
  bool zero;     // NVFP4 only: E4M3 scale is zero -> all codes zero
};

// MXFP4 abs-max (src/quantization/quantizer.py:107-112,162-165; quant_ops.py:82-94):
//   s = 2^(floor(log2(max(6*fl(fl(2a)/12), 2^-126))) - 2) / 0.75,  stored byte = e8m0(s * 3).
// For 2^-98 <= a < 2^101 the binade of 6*fl(fl(2a)/12) equals that of a (checked for every
// mantissa), s = 2^(e-2) * fl(4/3), 1/s rounds to 0.75 * 2^(2-e) and s*3 = 2^e exactly.
__device__ __forceinline__ GroupScale mx_group_scale(float a) {
  GroupScale g;
  g.zero = false;
  const int e = (int)((__float_as_uint(a) >> 23) & 0xffu) - 127;
  g.slow = !(e >= -98 && e <= 100);
  if (!g.slow) {
    g.k1 = __uint_as_float(((uint32_t)(128 - e) << 23) | 0x400000u);                // 0.75 * 2^(2-e)
    g.k2 = __uint_as_float(0x80000000u | ((uint32_t)(103 - e) << 23) | 0x400000u);  // -1.5*2^-26 * 2^(2-e)
    g.byte = (uint32_t)(e + 127);
  } else {
    const float sc = (a * 2.0f) / 12.0f;
    float arg = sc * 6.0f;
    arg = arg >= 1.17549435e-38f ? arg : 1.17549435e-38f;
    int el = (int)((__float_as_uint(arg) >> 23) & 0xffu) - 127;
    el = el > 127 ? 127 : el;
    const float s = __builtin_ldexpf(1.0f, el - 2) / 0.75f;
    g.k1 = s;
    g.k2 = 0.0f;
    g.byte = e8m0_encode(s * 3.0f);
  }
  return g;
}

// NVFP4 (src/quantization/quantizer.py:107-112,143-160,168; rtn.py:188):
//   sc = e4m3(clamp(fl(fl(2a)/12) * gs, +-448)),  s = fp32(sc) * fl(1/gs),  byte = e4m3(s * gs);
// a zero s stores byte 0 with all-zero codes.
__device__ __forceinline__ GroupScale nv_group_scale(float a, float gs, float rg) {
  GroupScale g;
  const float sc0 = (a * 2.0f) / 12.0f;
  float t = sc0 * gs;
  t = t > 448.0f ? 448.0f : t;
  t = t < -448.0f ? -448.0f : t;
  const float sc = e4m3_decode(e4m3_encode(t));
  const float s = sc * rg;
  g.zero = (s == 0.0f);
  g.byte = g.zero ? 0u : e4m3_encode(s * gs);
  const float as = __builtin_fabsf(s);
  g.slow = !(as >= 7.8886090522101181e-31f && as <= 1.2676506002282294e30f);  // 2^-100 .. 2^100
  if (!g.slow) {
    const float y = 1.0f / s;
    const float ey = __builtin_fmaf(-s, y, 1.0f);
    g.k1 = y;
    g.k2 = ey / s;
  } else {
    g.k1 = g.zero ? 1.0f : s;
    g.k2 = 0.0f;
  }
  return g;
}

__device__ __forceinline__ float scale_element(float x, const GroupScale& g) {
  return g.slow ? x / g.k1 : __builtin_fmaf(x, g.k1, x * g.k2);
}

// ---------------------------------------------------------------------------------------------
// Direct global -> LDS loads: 16 (4) bytes per lane land at lds_base + lane * 16 (4).  Written as
// inline assembly so that the compiler does not serialise every later LDS read behind them;
// completion is awaited explicitly with wait_vmem().  Nothing else in these kernels uses M0.
__device__ __forceinline__ void lds_dma16(const uint8_t* gbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(voff), "s"(gbase) : "memory");
}
// Same, marked non-temporal: for data that is read exactly once (streaming kernels).
__device__ __forceinline__ void lds_dma16_nt(const uint8_t* gbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :: "s"(lds_base), "v"(voff), "s"(gbase) : "memory");
}
__device__ __forceinline__ void lds_dma4(const uint8_t* gbase, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_base), "v"(voff), "s"(gbase) : "memory");
}
__device__ __forceinline__ void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// a / 6 correctly rounded (the reference writes fl(fl(2a)/12), the same number): Markstein's
// correction with RN(1/6), exact for every mantissa (checked exhaustively on the host).
__device__ __forceinline__ float div6_rn(float a) {
  const float c6 = 0.16666667163372039794921875f;
  const float q = a * c6;
  const float r = __builtin_fmaf(-q, 6.0f, a);
  return __builtin_fmaf(r, c6, q);
}

}  // namespace fpq
