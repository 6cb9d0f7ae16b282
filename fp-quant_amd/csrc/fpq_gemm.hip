// W4A4 GEMMs for gfx950:  y[m, n] = bf16(alpha * sum_k dq(x)[m, k] * dq(w)[n, k]) (+ bias[n]).
//
// MXFP4: CDNA4 block-scaled MFMA v_mfma_scale_f32_16x16x128_f8f6f4 with both operands in FP4
// (cbsz = blgp = 4).  A lane supplies 32 consecutive K codes (16 bytes) of one row and the one
// E8M0 byte that scales exactly those 32 values, so the MX group (32) is the hardware block and
// scales are consumed row-major, without any re-tiling.
//
// NVFP4: E4M3 scales per 16 values have a mantissa the block-scaled MFMA cannot apply, so codes
// are dequantized in registers to fp16 (code * 2^8 by v_cvt_scalef32_pk_f16_fp4, then a packed
// fp16 multiply by the E4M3 scale re-biased into fp16) and fed to v_mfma_f32_16x16x32_f16.
// Every product code * scale has at most 6 significant bits and magnitude in [2^-10, 2688], so
// the fp16 operands are exact and the only rounding is fp32 accumulation and the bf16 store.
//
// The MFMA "A" operand holds the weight rows and "B" the activation rows, so a lane's four
// accumulator values are four consecutive n of one m and store as one 8-byte write.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fpq.h"
#include "fpq_device.h"

namespace fpq {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint16_t bf16_bits_rne(float f) {
  uint32_t b = __float_as_uint(f);
  if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40u);  // quiet NaN
  b += 0x7fffu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}

// bf16(alpha * acc), then the reference's separate bf16 `y += bias`
// (inference_lib/src/fp_quant/module/linear_fns.py:512-514) folded into the store.
__device__ __forceinline__ uint16_t epilogue(float acc, float alpha, bool has_bias, float bias) {
  uint16_t o = bf16_bits_rne(acc * alpha);
  if (has_bias) o = bf16_bits_rne(__uint_as_float((uint32_t)o << 16) + bias);
  return o;
}

template <int TN, int TM>
__device__ __forceinline__ void store_tile(const v4f (&acc)[TN][TM], uint16_t* __restrict__ y,
                                           const uint16_t* __restrict__ bias, float alpha, int n0,
                                           int m0, int M, int N, int r, int kb) {
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = n0 + i * 16 + 4 * kb;
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (n + q < N) bv[q] = __uint_as_float((uint32_t)bias[n + q] << 16);
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + j * 16 + r;
      if (m >= M) continue;
      uint16_t o[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) o[q] = epilogue(acc[i][j][q], alpha, bias != nullptr, bv[q]);
      uint16_t* dst = y + (size_t)m * N + n;
      if (n + 3 < N && ((N & 3) == 0)) {
        *(uint2*)dst = make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16),
                                  (uint32_t)o[2] | ((uint32_t)o[3] << 16));
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (n + q < N) dst[q] = o[q];
      }
    }
  }
}

// -------------------------------------------------------------------------------------------
// Direct-from-global kernels: every wave loads its own operand fragments in MFMA layout.
// Wave tile = (TN*16 n) x (TM*16 m); a block has WN x WM waves (WN*WM == 4).
template <int TN, int TM, int WN, int WM>
__global__ __launch_bounds__(256) void gemm_mxf4_direct_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = (blockIdx.x * WN + (wave % WN)) * TN * 16;
  const int m0 = (blockIdx.y * WM + (wave / WN)) * TM * 16;
  const int kbytes = K >> 1;

  const uint8_t* wp[TN];
  const uint8_t* wsp[TN];
  const uint8_t* xp[TM];
  const uint8_t* xsp[TM];
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = min(n0 + i * 16 + r, N - 1);
    wp[i] = wq + (size_t)n * kbytes + kb * 16;
    wsp[i] = ws + (size_t)n * ws_stride + kb;
  }
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = min(m0 + j * 16 + r, M - 1);
    xp[j] = xq + (size_t)m * kbytes + kb * 16;
    xsp[j] = xs + (size_t)m * xs_stride + kb;
  }

  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < K; k0 += 128) {
    const bool kvalid = k0 + kb * 32 < K;
    v8i a[TN], b[TM];
    int sa[TN], sb[TM];
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      sa[i] = 127;
      if (kvalid) {
        v = *(const uint4*)(wp[i] + (k0 >> 1));
        sa[i] = wsp[i][k0 >> 5];
      }
      a[i] = v8i{(int)v.x, (int)v.y, (int)v.z, (int)v.w, 0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      sb[j] = 127;
      if (kvalid) {
        v = *(const uint4*)(xp[j] + (k0 >> 1));
        sb[j] = xsp[j][k0 >> 5];
      }
      b[j] = v8i{(int)v.x, (int)v.y, (int)v.z, (int)v.w, 0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i], b[j], acc[i][j], 4, 4, 0,
                                                                     sa[i], 0, sb[j]);
  }
  store_tile<TN, TM>(acc, y, bias, *alpha_p, n0, m0, M, N, r, kb);
}

// 8 E2M1 codes (one dword) times one E4M3 scale -> 8 exact fp16 values.
__device__ __forceinline__ v8h dequant8_f16(uint32_t codes, uint32_t scale_byte) {
  const uint32_t h = ((scale_byte & 0x7fu) << 7) | ((scale_byte & 0x80u) << 8);
  const v2h s2 = __builtin_bit_cast(v2h, h | (h << 16));  // e4m3 re-biased: value * 2^-8
  const v2h p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 0) * s2;
  const v2h p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 1) * s2;
  const v2h p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 2) * s2;
  const v2h p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 3) * s2;
  return v8h{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// A lane loads 32 consecutive K codes (16 bytes) and their two E4M3 scales per 128-wide K step
// and spends them over four 16x16x32 MFMAs, dword s of the load in MFMA s.  Both operands use
// the same K assignment, so the sum over K is complete and only its order is permuted.
template <int TN, int TM, int WN, int WM>
__global__ __launch_bounds__(256) void gemm_nvf4_direct_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = (blockIdx.x * WN + (wave % WN)) * TN * 16;
  const int m0 = (blockIdx.y * WM + (wave / WN)) * TM * 16;
  const int kbytes = K >> 1;

  const uint8_t* wp[TN];
  const uint8_t* wsp[TN];
  const uint8_t* xp[TM];
  const uint8_t* xsp[TM];
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = min(n0 + i * 16 + r, N - 1);
    wp[i] = wq + (size_t)n * kbytes + kb * 16;
    wsp[i] = ws + (size_t)n * ws_stride + kb * 2;
  }
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = min(m0 + j * 16 + r, M - 1);
    xp[j] = xq + (size_t)m * kbytes + kb * 16;
    xsp[j] = xs + (size_t)m * xs_stride + kb * 2;
  }

  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < K; k0 += 128) {
    // K % 16 == 0: the lane's 32 values may be fully, half or not at all inside K
    const int kl = k0 + kb * 32;
    uint4 a[TN], b[TM];
    uint32_t sa[TN][2], sb[TM][2];
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      a[i] = make_uint4(0u, 0u, 0u, 0u);
      sa[i][0] = sa[i][1] = 0u;
      if (kl + 32 <= K) {
        a[i] = *(const uint4*)(wp[i] + (k0 >> 1));
        sa[i][0] = wsp[i][k0 >> 4];
        sa[i][1] = wsp[i][(k0 >> 4) + 1];
      } else if (kl + 16 <= K) {
        const uint2 v = *(const uint2*)(wp[i] + (k0 >> 1));
        a[i].x = v.x;
        a[i].y = v.y;
        sa[i][0] = wsp[i][k0 >> 4];
      }
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      b[j] = make_uint4(0u, 0u, 0u, 0u);
      sb[j][0] = sb[j][1] = 0u;
      if (kl + 32 <= K) {
        b[j] = *(const uint4*)(xp[j] + (k0 >> 1));
        sb[j][0] = xsp[j][k0 >> 4];
        sb[j][1] = xsp[j][(k0 >> 4) + 1];
      } else if (kl + 16 <= K) {
        const uint2 v = *(const uint2*)(xp[j] + (k0 >> 1));
        b[j].x = v.x;
        b[j].y = v.y;
        sb[j][0] = xsp[j][k0 >> 4];
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      v8h ah[TN], bh[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const uint32_t c = s == 0 ? a[i].x : s == 1 ? a[i].y : s == 2 ? a[i].z : a[i].w;
        ah[i] = dequant8_f16(c, sa[i][s >> 1]);
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const uint32_t c = s == 0 ? b[j].x : s == 1 ? b[j].y : s == 2 ? b[j].z : b[j].w;
        bh[j] = dequant8_f16(c, sb[j][s >> 1]);
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah[i], bh[j], acc[i][j], 0, 0, 0);
    }
  }
  store_tile<TN, TM>(acc, y, bias, *alpha_p, n0, m0, M, N, r, kb);
}

template <int FMT>
static int gemm_dispatch(const void* xq, const void* xs, int64_t xs_stride, const void* wq,
                         const void* ws, int64_t ws_stride, const float* alpha, const void* bias,
                         void* y, int64_t M, int64_t N, int64_t K, void* stream_) {
  constexpr int GROUP = FMT == 0 ? 32 : 16;
  hipStream_t stream = (hipStream_t)stream_;
  if (M < 0 || N < 0 || K < 0) return FPQ_E_SHAPE;
  if (M == 0 || N == 0) return FPQ_OK;
  if (!xq || !xs || !wq || !ws || !alpha || !y) return FPQ_E_NULL;
  if (K == 0 || K % GROUP != 0 || K % 32 != 0) return FPQ_E_SHAPE;
  if (xs_stride < K / GROUP || ws_stride < K / GROUP) return FPQ_E_SHAPE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return FPQ_E_SHAPE;
  if (((uintptr_t)xq & 15u) || ((uintptr_t)wq & 15u) || ((uintptr_t)y & 7u)) return FPQ_E_ALIGN;

#define FPQ_GEMM(TN, TM, WN, WM)                                                                   \
  do {                                                                                             \
    const dim3 grid((unsigned)((N + WN * TN * 16 - 1) / (WN * TN * 16)),                           \
                    (unsigned)((M + WM * TM * 16 - 1) / (WM * TM * 16)));                          \
    if (FMT == 0) {                                                                                \
      hipLaunchKernelGGL((gemm_mxf4_direct_kernel<TN, TM, WN, WM>), grid, dim3(256), 0, stream,    \
                         (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride,                   \
                         (const uint8_t*)wq, (const uint8_t*)ws, (int)ws_stride, alpha,            \
                         (const uint16_t*)bias, (uint16_t*)y, (int)M, (int)N, (int)K);             \
    } else {                                                                                       \
      hipLaunchKernelGGL((gemm_nvf4_direct_kernel<TN, TM, WN, WM>), grid, dim3(256), 0, stream,    \
                         (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride,                   \
                         (const uint8_t*)wq, (const uint8_t*)ws, (int)ws_stride, alpha,            \
                         (const uint16_t*)bias, (uint16_t*)y, (int)M, (int)N, (int)K);             \
    }                                                                                              \
  } while (0)

  if (M <= 16) {
    FPQ_GEMM(1, 1, 4, 1);
  } else if (M <= 32) {
    FPQ_GEMM(2, 2, 4, 1);
  } else if (M <= 64) {
    FPQ_GEMM(2, 4, 4, 1);
  } else {
    FPQ_GEMM(4, 4, 2, 2);
  }
#undef FPQ_GEMM
  return (int)hipGetLastError();
}

}  // namespace fpq

extern "C" int fpq_gemm_mxf4(const void* xq, const void* xs, int64_t xs_stride, const void* wq,
                             const void* ws, int64_t ws_stride, const float* alpha,
                             const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                             void* stream) {
  return fpq::gemm_dispatch<0>(xq, xs, xs_stride, wq, ws, ws_stride, alpha, bias, y, M, N, K, stream);
}

extern "C" int fpq_gemm_nvf4(const void* xq, const void* xs, int64_t xs_stride, const void* wq,
                             const void* ws, int64_t ws_stride, const float* alpha,
                             const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                             void* stream) {
  return fpq::gemm_dispatch<1>(xq, xs, xs_stride, wq, ws, ws_stride, alpha, bias, y, M, N, K, stream);
}
