// Pieces shared by the LDS-tiled GEMM kernels (gfx950 only): vector typedefs and the epilogue that
// stages a wave's part of the output tile through LDS so that global stores are whole 256-byte rows.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fpq {

// Raises a kernel's dynamic-LDS limit once per device (the attribute is per device; one
// function-local static instance per kernel lives in the launcher).  Safe from any host thread: a
// race only repeats the idempotent call.
struct LdsLimitOnce {
  std::atomic<uint64_t> done{0};  // bit d: set for device d (devices >= 64 set it on every call)
  int ensure(const void* kernel, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return 0;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return (int)e;
    if (bit) done.fetch_or(bit, std::memory_order_release);
    return 0;
  }
};

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void global_void;

typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// NVFP4 operands for the fp16 MFMA.  e4m3 byte (>= 0) -> the same value * 2^-8 as fp16, in both
// halves of a dword (bits above the byte are ignored) ...
__device__ __forceinline__ v2h e4m3_pair_f16(uint32_t byte) {
  const uint32_t h = (byte << 7) & 0x3f80u;
  return __builtin_bit_cast(v2h, h | (h << 16));
}
// ... and 8 E2M1 codes (one dword) times that scale -> 8 exact fp16 values (code * 2^8 * scale * 2^-8)
__device__ __forceinline__ v8h dequant8_f16_s(uint32_t codes, v2h s2) {
  const v2h p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 0) * s2;
  const v2h p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 1) * s2;
  const v2h p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 2) * s2;
  const v2h p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 3) * s2;
  return v8h{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// Epilogue of the LDS-tiled kernels.  A wave owns TN x TM accumulator tiles of 32 x 32; register
// v of tile (i, j) is y[m][n] with m = j*32 + r32 and n = i*32 + 8*(v/4) + 4*kh + v%4 relative to
// the wave's origin (m0, n0).  The wave's part goes through its share of the (now idle) LDS as
// bf16 [m][n] so that global stores are whole contiguous rows of TN*64 bytes.
template <int TN, int TM, int LDS_BYTES, int NWAVES>
__device__ __forceinline__ void wave_tile_store(const v16f (&acc)[TN][TM], uint8_t* smem,
                                                uint16_t* __restrict__ y,
                                                const uint16_t* __restrict__ bias,
                                                const float* __restrict__ alpha_p, int n0, int m0,
                                                int wave, int lane, int M, int N,
                                                const uint16_t* __restrict__ residual = nullptr) {
  const int r32 = lane & 31, kh = lane >> 5;
  const float alpha = *alpha_p;
  constexpr int WT_N = TN * 32, WT_M = TM * 32;      // this wave's part of the workgroup tile
  constexpr int kRowBytes = WT_N * 2;
  constexpr int kStride = kRowBytes + 16;            // bytes per staged row (+16: spread banks)
  static_assert(NWAVES * WT_M * kStride <= LDS_BYTES, "epilogue staging does not fit in LDS");
  __syncthreads();                                   // every wave is done reading operands
  uint8_t* stg = smem + wave * (WT_M * kStride);
#pragma unroll
  for (int i = 0; i < TN; ++i) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int nl = i * 32 + 8 * g + 4 * kh;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (n0 + nl + u < N) bv[u] = __uint_as_float((uint32_t)bias[n0 + nl + u] << 16);
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        uint32_t lo = pack_bf16x2(acc[i][j][4 * g + 0] * alpha, acc[i][j][4 * g + 1] * alpha);
        uint32_t hi = pack_bf16x2(acc[i][j][4 * g + 2] * alpha, acc[i][j][4 * g + 3] * alpha);
        if (bias) {
          lo = pack_bf16x2(__uint_as_float(lo << 16) + bv[0], __uint_as_float(lo & 0xffff0000u) + bv[1]);
          hi = pack_bf16x2(__uint_as_float(hi << 16) + bv[2], __uint_as_float(hi & 0xffff0000u) + bv[3]);
        }
        *(uint2*)(stg + (j * 32 + r32) * kStride + nl * 2) = make_uint2(lo, hi);
      }
    }
  }
  // read back: kLpr lanes x 16 B cover one row, 64 / kLpr rows per wave instruction
  constexpr int kLpr = kRowBytes / 16 <= 16 ? 16 : 32;
  constexpr int kRpi = 64 / kLpr;
  static_assert(kRowBytes / 16 <= 32 && WT_M % kRpi == 0, "unsupported wave tile shape");
  const int rr = lane / kLpr, cc = lane % kLpr;
  const bool vec_ok = (N & 7) == 0;
#pragma unroll 4
  for (int p = 0; p < WT_M / kRpi; ++p) {
    const int ml = p * kRpi + rr;
    if (cc * 16 >= kRowBytes) continue;
    uint4 v = *(const uint4*)(stg + ml * kStride + cc * 16);
    const int m = m0 + ml, n = n0 + cc * 8;
    if (m >= M || n >= N) continue;
    uint16_t* dst = y + (size_t)m * N + n;
    if (vec_ok && n + 7 < N) {
      if (residual) {  // a separate bf16 add after the GEMM: one more rounding
        const uint4 rv = *(const uint4*)(residual + (size_t)m * N + n);
        const uint32_t a[4] = {v.x, v.y, v.z, v.w}, b[4] = {rv.x, rv.y, rv.z, rv.w};
        uint32_t o[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          o[u] = pack_bf16x2(__uint_as_float(a[u] << 16) + __uint_as_float(b[u] << 16),
                             __uint_as_float(a[u] & 0xffff0000u) + __uint_as_float(b[u] & 0xffff0000u));
        v = make_uint4(o[0], o[1], o[2], o[3]);
      }
      *(uint4*)dst = v;
    } else {
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (n + u < N) {
          uint32_t h = (w[u >> 1] >> (16 * (u & 1))) & 0xffffu;
          if (residual) {
            const float sum = __uint_as_float(h << 16) + __uint_as_float((uint32_t)residual[(size_t)m * N + n + u] << 16);
            h = pack_bf16x2(sum, 0.0f) & 0xffffu;
          }
          dst[u] = (uint16_t)h;
        }
      }
    }
  }
}

// The 2 x WM wave arrangement of the row-major kernels: wave (wn, wm) owns the BN/2 x BM/WM part.
template <int BN, int BM, int LDS_BYTES, int WM = 2>
__device__ __forceinline__ void wave_quadrant_store(const v16f (&acc)[BN / 64][BM / (32 * WM)], uint8_t* smem,
                                                    uint16_t* __restrict__ y,
                                                    const uint16_t* __restrict__ bias,
                                                    const float* __restrict__ alpha_p, int n_blk, int m_blk,
                                                    int wn, int wm, int wave, int lane, int M, int N) {
  wave_tile_store<BN / 64, BM / (32 * WM), LDS_BYTES, 2 * WM>(acc, smem, y, bias, alpha_p, n_blk + wn * (BN / 2),
                                                              m_blk + wm * (BM / WM), wave, lane, M, N);
}

}  // namespace fpq
