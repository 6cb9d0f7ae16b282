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
#include "fpq_gemm_epilogue.h"

namespace fpq {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

#ifndef FPQ_GEMM_WM
#define FPQ_GEMM_WM 2  // waves along m in the LDS-tiled MXFP4 kernel (2: 4 waves, 4: 8 waves)
#endif
#ifndef FPQ_SPLITK_MAX_M
#define FPQ_SPLITK_MAX_M 64  // largest M served by the weight-streaming split-K kernel
#endif

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

// -------------------------------------------------------------------------------------------
// Weight-streaming kernel for small M (the reference's disabled small-M entry, linear_fns.py:55).
// The time is the 31 MB weight read, so the job is to keep many loads in flight: a workgroup owns
// 16 weight rows, its four waves each take a quarter of K and issue all of their loads before the
// first MFMA; the four partial 16 x (16 TM) tiles are then summed through LDS by wave 0.
template <int TN, int TM>
__global__ __launch_bounds__(256) void gemm_mxf4_splitk_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K) {
  __shared__ v4f part[3][TN][TM][64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * TN * 16, m0 = blockIdx.y * TM * 16;
  const int kbytes = K >> 1;
  const int kq = K >> 2;                       // K range of this wave: [wave * kq, wave * kq + kq)
  const int steps = kq >> 7;                   // 128 per MFMA

  const uint8_t* wp[TN];
  const uint8_t* wsp[TN];
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = min(n0 + i * 16 + r, N - 1);
    wp[i] = wq + (size_t)n * kbytes + ((wave * kq) >> 1) + kb * 16;
    wsp[i] = ws + (size_t)n * ws_stride + ((wave * kq) >> 5);
  }
  const uint8_t* xp[TM];
  const uint8_t* xsp[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = min(m0 + j * 16 + r, M - 1);
    xp[j] = xq + (size_t)m * kbytes + ((wave * kq) >> 1) + kb * 16;
    xsp[j] = xs + (size_t)m * xs_stride + ((wave * kq) >> 5);
  }
  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // Loads are issued in batches of 4 * Q K steps: per row tile and group of 4 steps four 16-byte
  // code loads and ONE 16-byte scale load (the row's 16 scale bytes of those steps; byte 4 u + kb
  // is this lane's scale in step u), all before the first MFMA of the batch.
  constexpr int Q = (TN + TM <= 4) ? 2 : 1;
  for (int s0 = 0; s0 < steps; s0 += 4 * Q) {
    uint4 a[Q][4][TN], b[Q][4][TM], sa4[Q][TN], sb4[Q][TM];
#pragma unroll
    for (int h = 0; h < Q; ++h) {
      const bool on = s0 + 4 * h < steps;  // steps is a multiple of 4
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        sa4[h][i] = make_uint4(0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu);
        if (on) sa4[h][i] = *(const uint4*)(wsp[i] + (s0 + 4 * h) * 4);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          a[h][u][i] = make_uint4(0u, 0u, 0u, 0u);
          if (on) {
            const v4u ld = __builtin_nontemporal_load((const v4u*)(wp[i] + (s0 + 4 * h + u) * 64));
            a[h][u][i] = make_uint4(ld.x, ld.y, ld.z, ld.w);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        sb4[h][j] = make_uint4(0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu);
        if (on) sb4[h][j] = *(const uint4*)(xsp[j] + (s0 + 4 * h) * 4);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          b[h][u][j] = make_uint4(0u, 0u, 0u, 0u);
          if (on) b[h][u][j] = *(const uint4*)(xp[j] + (s0 + 4 * h + u) * 64);
        }
      }
    }
#pragma unroll
    for (int h = 0; h < Q; ++h) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const uint4 s4 = sb4[h][j];
          const uint32_t sbw = u == 0 ? s4.x : u == 1 ? s4.y : u == 2 ? s4.z : s4.w;
          const int sb = (int)((sbw >> (8 * kb)) & 0xffu);
          const uint4 bq = b[h][u][j];
          const v8i bv = v8i{(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w, 0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < TN; ++i) {
            const uint4 t4 = sa4[h][i];
            const uint32_t saw = u == 0 ? t4.x : u == 1 ? t4.y : u == 2 ? t4.z : t4.w;
            const int sa = (int)((saw >> (8 * kb)) & 0xffu);
            const uint4 aq = a[h][u][i];
            const v8i av = v8i{(int)aq.x, (int)aq.y, (int)aq.z, (int)aq.w, 0, 0, 0, 0};
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[i][j], 4, 4, 0, sa, 0, sb);
          }
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j) part[wave - 1][i][j][lane] = acc[i][j];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j)
        acc[i][j] = ((acc[i][j] + part[0][i][j][lane]) + part[1][i][j][lane]) + part[2][i][j][lane];
    store_tile<TN, TM>(acc, y, bias, *alpha_p, n0, m0, M, N, r, kb);
  }
}

// The same weight-streaming scheme for NVFP4: a lane's 16 bytes of codes (32 K values) carry two
// E4M3 scales; per batch of four 128-K steps a row's 32 scale bytes arrive as two 16-byte loads.
// Dword s of every code load feeds fp16 MFMA s of the step on both operands (K order permuted
// consistently), after exact in-register dequantization to fp16.
template <int TN, int TM>
__global__ __launch_bounds__(256) void gemm_nvf4_splitk_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K) {
  __shared__ v4f part[3][TN][TM][64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int r = lane & 15, kb = lane >> 4;
  const int n0 = blockIdx.x * TN * 16, m0 = blockIdx.y * TM * 16;
  const int kbytes = K >> 1;
  const int kq = K >> 2;                       // K range of this wave: [wave * kq, wave * kq + kq)
  const int steps = kq >> 7;                   // 128 K per step (four fp16 MFMAs)

  const uint8_t* wp[TN];
  const uint8_t* wsp[TN];
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    const int n = min(n0 + i * 16 + r, N - 1);
    wp[i] = wq + (size_t)n * kbytes + ((wave * kq) >> 1) + kb * 16;
    wsp[i] = ws + (size_t)n * ws_stride + ((wave * kq) >> 4);
  }
  const uint8_t* xp[TM];
  const uint8_t* xsp[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = min(m0 + j * 16 + r, M - 1);
    xp[j] = xq + (size_t)m * kbytes + ((wave * kq) >> 1) + kb * 16;
    xsp[j] = xs + (size_t)m * xs_stride + ((wave * kq) >> 4);
  }
  v4f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  for (int s0 = 0; s0 < steps; s0 += 4) {  // steps is a multiple of 4
    uint4 a[4][TN], b[4][TM], sa8[2][TN], sb8[2][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      sa8[0][i] = *(const uint4*)(wsp[i] + s0 * 8);
      sa8[1][i] = *(const uint4*)(wsp[i] + s0 * 8 + 16);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const v4u ld = __builtin_nontemporal_load((const v4u*)(wp[i] + (s0 + u) * 64));
        a[u][i] = make_uint4(ld.x, ld.y, ld.z, ld.w);
      }
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      sb8[0][j] = *(const uint4*)(xsp[j] + s0 * 8);
      sb8[1][j] = *(const uint4*)(xsp[j] + s0 * 8 + 16);
#pragma unroll
      for (int u = 0; u < 4; ++u) b[u][j] = *(const uint4*)(xp[j] + (s0 + u) * 64);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      // step u: scale bytes 8 (u % 2) + 2 kb and + 1 of 16-byte load u / 2
      v8h bh[TM][4];
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const uint4 s4 = sb8[u >> 1][j];
        const uint32_t lo = (u & 1) ? s4.z : s4.x, hi = (u & 1) ? s4.w : s4.y;
        const uint32_t two = ((kb & 2) ? hi : lo) >> (16 * (kb & 1));
        const uint4 c = b[u][j];
        bh[j][0] = dequant8_f16_s(c.x, e4m3_pair_f16(two));
        bh[j][1] = dequant8_f16_s(c.y, e4m3_pair_f16(two));
        bh[j][2] = dequant8_f16_s(c.z, e4m3_pair_f16(two >> 8));
        bh[j][3] = dequant8_f16_s(c.w, e4m3_pair_f16(two >> 8));
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const uint4 s4 = sa8[u >> 1][i];
        const uint32_t lo = (u & 1) ? s4.z : s4.x, hi = (u & 1) ? s4.w : s4.y;
        const uint32_t two = ((kb & 2) ? hi : lo) >> (16 * (kb & 1));
        const uint4 c = a[u][i];
        const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const v8h ah = dequant8_f16_s(cw[s], e4m3_pair_f16(two >> (8 * (s >> 1))));
#pragma unroll
          for (int j = 0; j < TM; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bh[j][s], acc[i][j], 0, 0, 0);
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j) part[wave - 1][i][j][lane] = acc[i][j];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j)
        acc[i][j] = ((acc[i][j] + part[0][i][j][lane]) + part[1][i][j][lane]) + part[2][i][j][lane];
    store_tile<TN, TM>(acc, y, bias, *alpha_p, n0, m0, M, N, r, kb);
  }
}

// -------------------------------------------------------------------------------------------
// LDS-tiled MXFP4 kernel for large M.  A block of 4 waves (2 x 2) owns a BN x BM output tile and
// walks K in steps of 256 (one 128-byte line of codes per row).  Packed codes and scale bytes go
// global -> LDS with direct 16-byte / 4-byte loads into a double buffer; the 16-byte chunks of a
// row are XOR-swizzled by (row & 7) through the choice of the global chunk each lane fetches, so
// that the 16-row x 64-byte MFMA operand reads are bank-conflict free.
constexpr int kKS = 256;                    // K per stage
constexpr int kRowBytes = kKS / 2;          // 128 bytes of codes per row per stage
constexpr int kScaleBytes = kKS / 32;       // 8 scale bytes per row per stage

template <int BN, int BM>
struct MxLdsLayout {
  static constexpr int kCodesW = 0;
  static constexpr int kCodesX = BN * kRowBytes;
  static constexpr int kScalesW = (BN + BM) * kRowBytes;
  static constexpr int kScalesX = kScalesW + BN * kScaleBytes;
  static constexpr int kStage = kScalesX + BM * kScaleBytes;
};

template <int BN, int BM, int WM>
__global__ __launch_bounds__(128 * WM) void gemm_mxf4_lds_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K, int tiles_m) {
  using L = MxLdsLayout<BN, BM>;
  constexpr int NW = 2 * WM;                          // waves: 2 along n x WM along m
  constexpr int TN = BN / 64, TM = BM / (32 * WM);    // 32x32 MFMA tiles per wave along n and m
  extern __shared__ __attribute__((aligned(128))) uint8_t smem[];
  const uint32_t smem_base = (uint32_t)(uintptr_t)smem;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  // Consecutive workgroup ids land on different XCDs (8 of them, each with its own L2), so
  // give every XCD a contiguous run of the tile list: its tiles then share weight row-panels.
  int tile_m, tile_n;
  banded_tile<BM>(tiles_m, tile_m, tile_n);
  const int n_blk = tile_n * BN, m_blk = tile_m * BM;
  const int wn = wave & 1, wm = wave >> 1;
  const int kbytes = K >> 1;

  // ---- global -> LDS assignment.  Codes: one wave instruction moves 8 rows x 128 B.
  constexpr int kInstrW = BN / 8 / NW, kInstrX = BM / 8 / NW;  // per wave
  const int lrow = lane >> 3;                                // row within the 8-row slab
  // LDS holds chunk c of tile row r at 16-byte slot c ^ (r & 7) ^ ((r >> 3) & 1) of the row: with
  // that swizzle the 32-row x 32-byte operand reads of the 32x32 MFMA layout hit every bank group
  // exactly once per pass (checked with the bank-conflict counter); a lane of load instruction
  // `idx` (8 rows) therefore fetches chunk (lane & 7) ^ lrow ^ (idx & 1)
  uint32_t w_off[kInstrW], x_off[kInstrX];
#pragma unroll
  for (int j = 0; j < kInstrW; ++j) {
    const int idx = wave * kInstrW + j;
    const int row = min(n_blk + idx * 8 + lrow, N - 1);
    w_off[j] = (uint32_t)row * (uint32_t)kbytes + (((lane & 7) ^ lrow ^ (idx & 1)) * 16);
  }
#pragma unroll
  for (int j = 0; j < kInstrX; ++j) {
    const int idx = wave * kInstrX + j;
    const int row = min(m_blk + idx * 8 + lrow, M - 1);
    x_off[j] = (uint32_t)row * (uint32_t)kbytes + (((lane & 7) ^ lrow ^ (idx & 1)) * 16);
  }
  // Scales: one wave instruction moves 32 rows x 8 B (two dwords per row); wave w takes
  // instructions j with j % NW == w.
  constexpr int kSInstrW = BN / 32, kSInstrX = BM / 32;
  constexpr int kSW = (kSInstrW + NW - 1) / NW, kSX = (kSInstrX + NW - 1) / NW;
  uint32_t ws_off[kSW], xs_off[kSX];
#pragma unroll
  for (int j = 0; j < kSW; ++j) {
    const int row = min(n_blk + (j * NW + wave) * 32 + (lane >> 1), N - 1);
    ws_off[j] = (uint32_t)row * (uint32_t)ws_stride + (lane & 1) * 4;
  }
#pragma unroll
  for (int j = 0; j < kSX; ++j) {
    const int row = min(m_blk + (j * NW + wave) * 32 + (lane >> 1), M - 1);
    xs_off[j] = (uint32_t)row * (uint32_t)xs_stride + (lane & 1) * 4;
  }

  auto issue_loads = [&](int stage, int k0) {
    const uint32_t base = smem_base + stage * L::kStage;
    const uint8_t* wk = wq + (k0 >> 1);
    const uint8_t* xk = xq + (k0 >> 1);
    const uint8_t* wsk = ws + (k0 >> 5);
    const uint8_t* xsk = xs + (k0 >> 5);
#pragma unroll
    for (int j = 0; j < kInstrW; ++j)
      lds_dma16(wk, w_off[j], base + L::kCodesW + (wave * kInstrW + j) * 1024);
#pragma unroll
    for (int j = 0; j < kInstrX; ++j)
      lds_dma16(xk, x_off[j], base + L::kCodesX + (wave * kInstrX + j) * 1024);
#pragma unroll
    for (int j = 0; j < kSW; ++j)
      if (j * NW + wave < kSInstrW) lds_dma4(wsk, ws_off[j], base + L::kScalesW + (j * NW + wave) * 256);
#pragma unroll
    for (int j = 0; j < kSX; ++j)
      if (j * NW + wave < kSInstrX) lds_dma4(xsk, xs_off[j], base + L::kScalesX + (j * NW + wave) * 256);
  };


  // 32x32x64 MFMA: lane = (row r32 = lane % 32, K half kh = lane / 32); one stage holds four
  // K steps q of 64, the lane's 16-byte chunk in step q is c = 2q + kh, its scale byte is c too.
  v16f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int r32 = lane & 31, kh = lane >> 5;
  const int rw = wn * (BN / 2) + r32, rx = wm * (BM / WM) + r32;
  int slot[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) slot[q] = ((2 * q + kh) ^ (r32 & 7) ^ ((r32 >> 3) & 1)) * 16;
  const int cw0 = L::kCodesW + rw * kRowBytes, cx0 = L::kCodesX + rx * kRowBytes;
  const int sw0 = L::kScalesW + rw * kScaleBytes, sx0 = L::kScalesX + rx * kScaleBytes;
  // bytes kh, 2+kh, 4+kh, 6+kh of a row's 8 scale bytes -> one dword; op_sel q picks K step q
  const uint32_t perm_sel = kh ? 0x07050301u : 0x06040200u;

  const int nk = K / kKS;
  // Operand stream of a stage: 4 K steps x TN weight tiles (16 "steps"), each tile used by TM
  // MFMAs.  Weight tiles are read from LDS three steps ahead (ring of 4), the activation tiles
  // of the next K step during the first steps of the current one.  The one barrier of an
  // iteration sits after step kSync: by then every wave has issued and completed all its reads
  // of the current stage and its share of the next stage's loads has landed, so the steps after
  // it already read the first tiles of the next stage (no bubble at the top of an iteration) and
  // the current buffer is handed to the loads of the stage after next.
  static_assert(TN == 4, "the step schedule below is written for four weight tiles per wave");
  constexpr int kSteps = 4 * TN, kSync = kSteps - 4;
  uint4 bq[2][TM], aq[4];
  uint2 raw_sa[TN], raw_sb[TM];
  auto read_w = [&](const uint8_t* b, int step) {
    return *(const uint4*)(b + cw0 + slot[step / TN] + (step % TN) * 32 * kRowBytes);
  };
  auto read_x = [&](const uint8_t* b, int q, int j) {
    return *(const uint4*)(b + cx0 + slot[q] + j * 32 * kRowBytes);
  };

  issue_loads(0, 0);
  if (nk > 1) issue_loads(1, kKS);
  wait_vmem();
  __syncthreads();
#pragma unroll
  for (int j = 0; j < TM; ++j) bq[0][j] = read_x(smem, 0, j);
#pragma unroll
  for (int u = 0; u < 3; ++u) aq[u] = read_w(smem, u);
#pragma unroll
  for (int j = 0; j < TM; ++j) raw_sb[j] = *(const uint2*)(smem + sx0 + j * 32 * kScaleBytes);
#pragma unroll
  for (int i = 0; i < TN; ++i) raw_sa[i] = *(const uint2*)(smem + sw0 + i * 32 * kScaleBytes);

  for (int it = 0; it < nk; ++it) {
    const uint8_t* base = smem + (it & 1) * L::kStage;
    const uint8_t* next = smem + ((it + 1) & 1) * L::kStage;  // stale bytes after the last stage: read, never used
    int sa[TN], sb[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) sb[j] = (int)__builtin_amdgcn_perm(raw_sb[j].y, raw_sb[j].x, perm_sel);
#pragma unroll
    for (int i = 0; i < TN; ++i) sa[i] = (int)__builtin_amdgcn_perm(raw_sa[i].y, raw_sa[i].x, perm_sel);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < kSteps; ++t) {
      const int q = t / TN, i = t % TN;
      aq[(t + 3) % 4] = t + 3 < kSteps ? read_w(base, t + 3) : read_w(next, t + 3 - kSteps);
      if (i < (TM + 1) / 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int j = i * 2 + u;
          if (j < TM && q < 3) bq[(q + 1) & 1][j] = read_x(base, q + 1, j);
        }
      }
      if (t > kSync && i - 1 < (TM + 1) / 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int j = (i - 1) * 2 + u;
          if (j < TM) bq[0][j] = read_x(next, 0, j);
        }
      }
      if (t == kSteps - 1) {
#pragma unroll
        for (int j = 0; j < TM; ++j) raw_sb[j] = *(const uint2*)(next + sx0 + j * 32 * kScaleBytes);
#pragma unroll
        for (int i2 = 0; i2 < TN; ++i2) raw_sa[i2] = *(const uint2*)(next + sw0 + i2 * 32 * kScaleBytes);
      }
      __builtin_amdgcn_sched_barrier(0);
      const uint4 av = aq[t % 4];
      const v8i a = v8i{(int)av.x, (int)av.y, (int)av.z, (int)av.w, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const uint4 bv = bq[q & 1][j];
        const v8i b = v8i{(int)bv.x, (int)bv.y, (int)bv.z, (int)bv.w, 0, 0, 0, 0};
        if (q == 0) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i][j], 4, 4, 0, sa[i], 0, sb[j]);
        if (q == 1) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i][j], 4, 4, 1, sa[i], 1, sb[j]);
        if (q == 2) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i][j], 4, 4, 2, sa[i], 2, sb[j]);
        if (q == 3) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i][j], 4, 4, 3, sa[i], 3, sb[j]);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t == kSync) {
        wait_vmem();      // this wave's loads for the next stage have landed
        __syncthreads();  // ... and everyone's; nobody reads the current stage any more
        if (it + 2 < nk) issue_loads(it & 1, (it + 2) * kKS);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  wave_quadrant_store<BN, BM, 2 * L::kStage, WM>(acc, smem, y, bias, alpha_p, n_blk, m_blk, wn, wm, wave, lane, M, N);
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

// -------------------------------------------------------------------------------------------
// LDS-tiled NVFP4 kernel for large M: the staging, swizzle, tile order and epilogue of the MXFP4
// kernel, with the operands dequantized to exact fp16 in registers right before
// v_mfma_f32_32x32x16_f16.  A lane's 16-byte chunk (32 codes, two E4M3 groups) feeds four MFMAs,
// dword s of the chunk in MFMA s; both operands use that same K assignment.  Per K step of 64 a
// wave dequantizes 8 tiles x 4 dwords (8 VALU ops each) for 64 MFMAs of 32 cycles, so the
// conversion hides behind the matrix pipe.
template <int BN, int BM>
struct NvLdsLayout {
  static constexpr int kScaleBytes = kKS / 16;  // 16 E4M3 bytes per row per stage
  static constexpr int kCodesW = 0;
  static constexpr int kCodesX = BN * kRowBytes;
  static constexpr int kScalesW = (BN + BM) * kRowBytes;
  static constexpr int kScalesX = kScalesW + BN * kScaleBytes;
  static constexpr int kStage = kScalesX + BM * kScaleBytes;
};

template <int BN, int BM>
__global__ __launch_bounds__(256) void gemm_nvf4_lds_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, int xs_stride,
    const uint8_t* __restrict__ wq, const uint8_t* __restrict__ ws, int ws_stride,
    const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
    int M, int N, int K, int tiles_m) {
  using L = NvLdsLayout<BN, BM>;
  constexpr int TN = BN / 64, TM = BM / 64;
  static_assert(BN == 256 && BM == 256, "scale DMA split assumes 64 rows per wave per operand");
  extern __shared__ __attribute__((aligned(128))) uint8_t smem[];
  const uint32_t smem_base = (uint32_t)(uintptr_t)smem;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  int tile_m, tile_n;
  banded_tile<BM>(tiles_m, tile_m, tile_n);
  const int n_blk = tile_n * BN, m_blk = tile_m * BM;
  const int wn = wave & 1, wm = wave >> 1;
  const int kbytes = K >> 1;

  constexpr int kInstrW = BN / 8 / 4, kInstrX = BM / 8 / 4;  // per wave: 8 rows x 128 B each
  const int lrow = lane >> 3;
  uint32_t w_off[kInstrW], x_off[kInstrX];  // same chunk swizzle as the MXFP4 kernel
#pragma unroll
  for (int j = 0; j < kInstrW; ++j) {
    const int idx = wave * kInstrW + j;
    const int row = min(n_blk + idx * 8 + lrow, N - 1);
    w_off[j] = (uint32_t)row * (uint32_t)kbytes + (((lane & 7) ^ lrow ^ (idx & 1)) * 16);
  }
#pragma unroll
  for (int j = 0; j < kInstrX; ++j) {
    const int idx = wave * kInstrX + j;
    const int row = min(m_blk + idx * 8 + lrow, M - 1);
    x_off[j] = (uint32_t)row * (uint32_t)kbytes + (((lane & 7) ^ lrow ^ (idx & 1)) * 16);
  }
  // scales: one 16-byte load per row per stage; wave w moves rows [64 w, 64 w + 64) of both operands
  const uint32_t ws_off = (uint32_t)min(n_blk + wave * 64 + lane, N - 1) * (uint32_t)ws_stride;
  const uint32_t xs_off = (uint32_t)min(m_blk + wave * 64 + lane, M - 1) * (uint32_t)xs_stride;

  auto issue_loads = [&](int stage, int k0) {
    const uint32_t base = smem_base + stage * L::kStage;
    const uint8_t* wk = wq + (k0 >> 1);
    const uint8_t* xk = xq + (k0 >> 1);
#pragma unroll
    for (int j = 0; j < kInstrW; ++j)
      lds_dma16(wk, w_off[j], base + L::kCodesW + (wave * kInstrW + j) * 1024);
#pragma unroll
    for (int j = 0; j < kInstrX; ++j)
      lds_dma16(xk, x_off[j], base + L::kCodesX + (wave * kInstrX + j) * 1024);
    lds_dma16(ws + (k0 >> 4), ws_off, base + L::kScalesW + wave * 1024);
    lds_dma16(xs + (k0 >> 4), xs_off, base + L::kScalesX + wave * 1024);
  };

  v16f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int r32 = lane & 31, kh = lane >> 5;
  const int rw = wn * (BN / 2) + r32, rx = wm * (BM / 2) + r32;
  int slot[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) slot[q] = ((2 * q + kh) ^ (r32 & 7) ^ ((r32 >> 3) & 1)) * 16;
  const int cw0 = L::kCodesW + rw * kRowBytes, cx0 = L::kCodesX + rx * kRowBytes;
  // the lane's chunk in K step q covers E4M3 groups 4q + 2kh and 4q + 2kh + 1 of the stage
  const int sw0 = L::kScalesW + rw * L::kScaleBytes + 2 * kh, sx0 = L::kScalesX + rx * L::kScaleBytes + 2 * kh;

  // Raw codes and scales are read from LDS one K step ahead, and dequantized operands run one MFMA
  // group ahead: while the four MFMAs of weight tile i (K sub-step `sub`) execute, the wave
  // converts weight tile i + 1 and activation tile i of the following sub-step, and the
  // instruction order is pinned to one MFMA followed by four or five conversion instructions, which
  // is what fits under the 32 cycles of a 32x32x16 MFMA.  (Issue is in order: conversions written
  // in a block ahead of the MFMAs leave the matrix pipe idle; pinned this way the pipe's duty rose
  // from 52 % to 64 %.  Carrying the pipeline across the stage barrier as well measured no faster.)
  const int nk = K / kKS;
  uint4 aq[2][TN], bq[2][TM];
  uint32_t sa[2][TN], sb[2][TM];
  auto read_raw = [&](const uint8_t* base, int q, int set) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      bq[set][j] = *(const uint4*)(base + cx0 + slot[q] + j * 32 * kRowBytes);
      sb[set][j] = *(const uint16_t*)(base + sx0 + 4 * q + j * 32 * L::kScaleBytes);
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      aq[set][i] = *(const uint4*)(base + cw0 + slot[q] + i * 32 * kRowBytes);
      sa[set][i] = *(const uint16_t*)(base + sw0 + 4 * q + i * 32 * L::kScaleBytes);
    }
  };
  auto a_half = [&](int set, int sub, int i) {
    const uint4 c = aq[set][i];
    const uint32_t cd = sub == 0 ? c.x : sub == 1 ? c.y : sub == 2 ? c.z : c.w;
    return dequant8_f16_h(cd, e4m3_byte_f16(sa[set][i], sub >> 1));
  };
  auto b_half = [&](int set, int sub, int j) {
    const uint4 c = bq[set][j];
    const uint32_t cd = sub == 0 ? c.x : sub == 1 ? c.y : sub == 2 ? c.z : c.w;
    return dequant8_f16_h(cd, e4m3_byte_f16(sb[set][j], sub >> 1));
  };

  issue_loads(0, 0);
  for (int it = 0; it < nk; ++it) {
    const uint8_t* base = smem + (it & 1) * L::kStage;
    wait_vmem();
    __syncthreads();
    if (it + 1 < nk) issue_loads((it + 1) & 1, (it + 1) * kKS);
    read_raw(base, 0, 0);
    v8h ah_cur, ah_next, bh_cur[TM], bh_next[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) bh_cur[j] = bh_next[j] = b_half(0, 0, j);
    ah_cur = ah_next = a_half(0, 0, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (q < 3) read_raw(base, q + 1, (q + 1) & 1);  // the next K step, read while this one computes
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int sub = 0; sub < 4; ++sub) {
        // the sub-step after this one; after the last one of the stage the conversions run on stale
        // registers and nothing consumes them
        const int nset = sub == 3 ? (q + 1) & 1 : q & 1, nsub = sub == 3 ? 0 : sub + 1;
#pragma unroll
        for (int i = 0; i < TN; ++i) {
          ah_next = i + 1 < TN ? a_half(q & 1, sub, i + 1) : a_half(nset, nsub, 0);
          bh_next[i] = b_half(nset, nsub, i);
#pragma unroll
          for (int j = 0; j < TM; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah_cur, bh_cur[j], acc[i][j], 0, 0, 0);
          static_assert(TM == 4, "the instruction pattern below is written for four MFMAs per weight tile");
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA ...
          __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);  // ... conversions behind it
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
          ah_cur = ah_next;
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) bh_cur[j] = bh_next[j];
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  wave_quadrant_store<BN, BM, 2 * L::kStage>(acc, smem, y, bias, alpha_p, n_blk, m_blk, wn, wm, wave, lane, M, N);
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
  if (((uintptr_t)xq & 15u) || ((uintptr_t)wq & 15u) || ((uintptr_t)y & 15u)) return FPQ_E_ALIGN;

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

  if (FMT == 1 && M > 64 && K % kKS == 0 && xs_stride % 16 == 0 && ws_stride % 16 == 0 &&
      !((uintptr_t)xs & 15u) && !((uintptr_t)ws & 15u) && N * (K / 2) < ((int64_t)1 << 32) &&
      M * (K / 2) < ((int64_t)1 << 32)) {
    constexpr int BN = 256, BM = 256;
    using L = NvLdsLayout<BN, BM>;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    static LdsLimitOnce nv_lds_limit;
    if (const int st = nv_lds_limit.ensure((const void*)gemm_nvf4_lds_kernel<BN, BM>, 2 * L::kStage)) return st;
    hipLaunchKernelGGL((gemm_nvf4_lds_kernel<BN, BM>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256),
                       2 * L::kStage, stream, (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride,
                       (const uint8_t*)wq, (const uint8_t*)ws, (int)ws_stride, alpha,
                       (const uint16_t*)bias, (uint16_t*)y, (int)M, (int)N, (int)K, tiles_m);
    return (int)hipGetLastError();
  }
  if (FMT == 0 && M > 64 && K % kKS == 0 && xs_stride % 4 == 0 && ws_stride % 4 == 0 &&
      !((uintptr_t)xs & 3u) && !((uintptr_t)ws & 3u) && N * (K / 2) < ((int64_t)1 << 32) &&
      M * (K / 2) < ((int64_t)1 << 32)) {
    constexpr int BN = 256, BM = 256;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    using L = MxLdsLayout<BN, BM>;
    static LdsLimitOnce mx_lds_limit;
    if (const int st = mx_lds_limit.ensure((const void*)gemm_mxf4_lds_kernel<BN, BM, FPQ_GEMM_WM>, 2 * L::kStage)) return st;
    hipLaunchKernelGGL((gemm_mxf4_lds_kernel<BN, BM, FPQ_GEMM_WM>), dim3((unsigned)(tiles_m * tiles_n)),
                       dim3(128 * FPQ_GEMM_WM),
                       2 * L::kStage, stream, (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride,
                       (const uint8_t*)wq, (const uint8_t*)ws, (int)ws_stride, alpha,
                       (const uint16_t*)bias, (uint16_t*)y, (int)M, (int)N, (int)K, tiles_m);
    return (int)hipGetLastError();
  }
#define FPQ_SPLITK(TNN, TMM)                                                                       \
  do {                                                                                             \
    const dim3 grid((unsigned)((N + TNN * 16 - 1) / (TNN * 16)),                                   \
                    (unsigned)((M + TMM * 16 - 1) / (TMM * 16)));                                  \
    hipLaunchKernelGGL((gemm_mxf4_splitk_kernel<TNN, TMM>), grid, dim3(256), 0, stream,            \
                       (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride, (const uint8_t*)wq, \
                       (const uint8_t*)ws, (int)ws_stride, alpha, (const uint16_t*)bias,           \
                       (uint16_t*)y, (int)M, (int)N, (int)K);                                      \
    return (int)hipGetLastError();                                                                 \
  } while (0)
  // K % 2048 == 0: every wave's K quarter is a whole number of 4-step batches and every 16-byte
  // scale load is aligned (scale strides and bases must be 16-byte multiples too)
#define FPQ_SPLITK_NV(TNN, TMM)                                                                    \
  do {                                                                                             \
    const dim3 grid((unsigned)((N + TNN * 16 - 1) / (TNN * 16)),                                   \
                    (unsigned)((M + TMM * 16 - 1) / (TMM * 16)));                                  \
    hipLaunchKernelGGL((gemm_nvf4_splitk_kernel<TNN, TMM>), grid, dim3(256), 0, stream,            \
                       (const uint8_t*)xq, (const uint8_t*)xs, (int)xs_stride, (const uint8_t*)wq, \
                       (const uint8_t*)ws, (int)ws_stride, alpha, (const uint16_t*)bias,           \
                       (uint16_t*)y, (int)M, (int)N, (int)K);                                      \
    return (int)hipGetLastError();                                                                 \
  } while (0)
  if (FMT == 1 && K % 2048 == 0 && M <= 64 && xs_stride % 16 == 0 && ws_stride % 16 == 0 &&
      !((uintptr_t)xs & 15u) && !((uintptr_t)ws & 15u)) {
    if (M == 1) FPQ_SPLITK_NV(1, 1);
    if (M <= 16) FPQ_SPLITK_NV(2, 1);
    if (M <= 32) FPQ_SPLITK_NV(2, 2);
    FPQ_SPLITK_NV(2, 4);
  }
#undef FPQ_SPLITK_NV
  if (FMT == 0 && K % 2048 == 0 && M <= FPQ_SPLITK_MAX_M && xs_stride % 16 == 0 && ws_stride % 16 == 0 &&
      !((uintptr_t)xs & 15u) && !((uintptr_t)ws & 15u)) {
    // 32 weight rows per workgroup once there is more than one activation row: halves the
    // re-reading of the activations from L2 (measured best among 16 / 32 / 64 rows)
    if (M == 1) FPQ_SPLITK(1, 1);
    if (M <= 16) FPQ_SPLITK(2, 1);
    if (M <= 32) FPQ_SPLITK(2, 2);
    FPQ_SPLITK(2, 4);
  }
#undef FPQ_SPLITK
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
