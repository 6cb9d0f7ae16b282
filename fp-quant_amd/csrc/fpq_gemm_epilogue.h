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
int device_cus();   // fpq_capi.hip: compute units of the current device (256 where none answers)

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

// Which output tile a workgroup of a large-M kernel computes, and its number in the tile list (returned).
// Consecutive workgroup ids land on different XCDs (8 of them, each with its own L2), so every XCD gets a
// contiguous run of the list.  The list walks bands of kBandRows activation rows: inside a band the
// activation row tiles run fastest, then the weight strips, so the workgroups an XCD holds at a time (32 or
// 64) form a block that shares about as many weight strips as activation tiles through the XCD's L2, and a
// band's activations stay there while its strips stream past.  Measured against activation tiles fastest
// over the whole of M (256 x 128 tiles, K = 4096): 4096 rows, N = 14336 127.1 -> 120.0 us; 8192 rows, N = 4096 /
// 14336 / 28672 75.1 -> 70.3 / 245.1 -> 232.2 / 493.9 -> 463.0 us; 2048 rows unchanged; bands of 512 or 2048 rows
// 1-2 % behind 1024.  The row-major NVFP4 kernel (256 x 256 tiles) gains 2.4 % at 8192 rows, nothing at 4096.
constexpr int kBandRows = 1024;
template <int BM>
__device__ __forceinline__ int banded_tile(int tiles_m, int& tile_m, int& tile_n) {
  int logical = blockIdx.x;
  const int nb = gridDim.x, per = nb / 8;
  if (blockIdx.x < (unsigned)(per * 8)) logical = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  constexpr int kBand = kBandRows / BM > 0 ? kBandRows / BM : 1;   // activation row tiles per band
  if (tiles_m > kBand) {
    const int tiles_n = nb / tiles_m;
    const int band = logical / (kBand * tiles_n), within = logical - band * (kBand * tiles_n);
    const int first_m = band * kBand, rows = min(tiles_m - first_m, kBand);
    tile_m = first_m + within % rows;
    tile_n = within / rows;
  } else {
    tile_m = logical % tiles_m;
    tile_n = logical / tiles_m;
  }
  return logical;
}

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

// The four E4M3 bytes of a dword at once: bytes 0 and 2 (low / high half of `even`) and bytes 1 and 3 (of `odd`)
// as fp16 (value * 2^-8), two instructions each; a multiply then takes one half for both of its lanes.
// (The empty asm keeps the compiler from splitting the dword operation into one 16-bit pair per half.)
__device__ __forceinline__ v2h e4m3_even_f16(uint32_t d) {
  uint32_t e = (d << 7) & 0x3f803f80u;
  asm("" : "+v"(e));
  return __builtin_bit_cast(v2h, e);
}
__device__ __forceinline__ v2h e4m3_odd_f16(uint32_t d) {
  uint32_t e = (d >> 1) & 0x3f803f80u;
  asm("" : "+v"(e));
  return __builtin_bit_cast(v2h, e);
}
__device__ __forceinline__ _Float16 e4m3_byte_f16(uint32_t d, int byte) {   // byte: a constant once unrolled
  const v2h h = (byte & 1) ? e4m3_odd_f16(d) : e4m3_even_f16(d);
  return (byte & 2) ? h.y : h.x;
}
__device__ __forceinline__ v8h dequant8_f16_h(uint32_t codes, _Float16 s) { return dequant8_f16_s(codes, v2h{s, s}); }
// ... and one half of that: codes 4 part .. 4 part + 3
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
__device__ __forceinline__ v4h dequant4_f16_h(uint32_t codes, _Float16 s, int part) {
  const v2h s2 = {s, s};
  const v2h p0 = (part ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 2)
                       : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 0)) * s2;
  const v2h p1 = (part ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 3)
                       : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, 256.0f, 1)) * s2;
  return v4h{p0.x, p0.y, p1.x, p1.y};
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// Output of a GEMM whose weight operand is several layers' weights laid end to end along N: columns
// [end[i-1], end[i]) of the product go to y[i], a dense [M, end[i] - end[i-1]] matrix of its own
// (end[-1] = 0).  count == 0: one output [M, N].  Every boundary is a multiple of kSegmentAlign, so
// that no workgroup tile of any kernel lies across one.
constexpr int kMaxSegments = 4;
constexpr int kSegmentAlign = 256;
struct OutSegments {
  int count;
  int end[kMaxSegments];
  uint16_t* y[kMaxSegments];
};

// Where a tile whose first column is n0 (workgroup- or wave-uniform) is stored: the output matrix,
// its width, the tile's first column in it, and the bias moved to the matrix's first column.
struct OutView {
  uint16_t* y;
  const uint16_t* bias;
  int n0, N;
};
__device__ __forceinline__ OutView out_view(const OutSegments& seg, uint16_t* y, const uint16_t* bias, int n0,
                                            int N) {
  OutView v{y, bias, n0, N};
  if (seg.count > 0) {
    int start = 0, stop = seg.end[0];
    uint16_t* ys = seg.y[0];
#pragma unroll
    for (int i = 1; i < kMaxSegments; ++i)
      if (i < seg.count && n0 >= seg.end[i - 1]) {
        start = seg.end[i - 1];
        stop = seg.end[i];
        ys = seg.y[i];
      }
    v.y = ys;
    v.bias = bias ? bias + start : bias;
    v.n0 = n0 - start;
    v.N = stop - start;
  }
  return v;
}

// The epilogue for a wave tile that lies inside the output (no row or column of it is cut off) with
// N a multiple of 8 and an 8-byte aligned bias: same values as wave_tile_store below with as few
// instructions as possible, because a workgroup's four waves issue them alone -- one instruction every
// few cycles per wave, with the matrix pipes idle.  Bias values are fetched with 8-byte loads before
// the barrier, the staging addresses are one register plus immediates, the global addresses one
// uniform base plus a 32-bit lane offset, and nothing is bounds-checked.
template <int TN, int TM, int NWAVES, bool BIAS, bool RESID>
__device__ __forceinline__ void wave_tile_store_interior(const v16f (&acc)[TN][TM], uint8_t* smem,
                                                         uint16_t* __restrict__ y,
                                                         const uint16_t* __restrict__ bias, float alpha,
                                                         int n0, int m0, int wave, int lane, int N,
                                                         const uint16_t* __restrict__ residual) {
  const int r32 = lane & 31, kh = lane >> 5;
  constexpr int WT_N = TN * 32, WT_M = TM * 32;
  constexpr int kRowBytes = WT_N * 2;
  constexpr int kStride = kRowBytes + 16;
  // Wave tiles of 128 x 64 and more belong to the kernels for large outputs (tens of megabytes, far more
  // than the L2 holds): their stores do not ask the L2 to keep the lines (1.4 % on the whole kernel).
  constexpr bool kStreamOut = TN * TM >= 8;
  uint2 braw[BIAS ? TN * 4 : 1];
  if (BIAS) {
#pragma unroll
    for (int ig = 0; ig < TN * 4; ++ig) braw[ig] = *(const uint2*)(bias + n0 + ig * 8 + 4 * kh);
  }
  __syncthreads();                                   // every wave is done reading operands
  uint8_t* stg = smem + wave * (WT_M * kStride);
  uint8_t* lane_w = stg + r32 * kStride + kh * 8;
#pragma unroll
  for (int i = 0; i < TN; ++i) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        uint32_t lo = pack_bf16x2(acc[i][j][4 * g + 0] * alpha, acc[i][j][4 * g + 1] * alpha);
        uint32_t hi = pack_bf16x2(acc[i][j][4 * g + 2] * alpha, acc[i][j][4 * g + 3] * alpha);
        if (BIAS) {
          const uint2 b = braw[i * 4 + g];
          lo = pack_bf16x2(__uint_as_float(lo << 16) + __uint_as_float(b.x << 16),
                           __uint_as_float(lo & 0xffff0000u) + __uint_as_float(b.x & 0xffff0000u));
          hi = pack_bf16x2(__uint_as_float(hi << 16) + __uint_as_float(b.y << 16),
                           __uint_as_float(hi & 0xffff0000u) + __uint_as_float(b.y & 0xffff0000u));
        }
        *(uint2*)(lane_w + j * 32 * kStride + (i * 32 + 8 * g) * 2) = make_uint2(lo, hi);
      }
    }
  }
  constexpr int kLpr = kRowBytes / 16 <= 16 ? 16 : 32;
  constexpr int kRpi = 64 / kLpr;
  constexpr int kIters = WT_M / kRpi;
  constexpr int kBatch = kIters % 8 == 0 ? 8 : (kIters % 4 == 0 ? 4 : 1);
  static_assert(kRowBytes / 16 <= 32 && WT_M % kRpi == 0, "unsupported wave tile shape");
  const int rr = lane / kLpr, cc = lane % kLpr;
  if (cc * 16 >= kRowBytes) return;
  const uint8_t* lane_r = stg + rr * kStride + cc * 16;
  uint8_t* gbase = (uint8_t*)(y + (size_t)m0 * N + n0);                       // uniform
  const uint8_t* rbase = (const uint8_t*)(residual + (size_t)m0 * N + n0);    // uniform (unused without RESID)
  const uint32_t goff = (uint32_t)(rr * N + cc * 8) * 2u;                     // < WT_M * N * 2 < 2^31
  const uint32_t gstep = (uint32_t)(kRpi * N) * 2u;
#pragma unroll
  for (int p0 = 0; p0 < kIters; p0 += kBatch) {
    uint4 vb[kBatch], rb[RESID ? kBatch : 1];
#pragma unroll
    for (int q = 0; q < kBatch; ++q) vb[q] = *(const uint4*)(lane_r + (p0 + q) * kRpi * kStride);
    if (RESID) {
#pragma unroll
      for (int q = 0; q < kBatch; ++q) rb[q] = *(const uint4*)(rbase + goff + (uint32_t)(p0 + q) * gstep);
    }
#pragma unroll
    for (int q = 0; q < kBatch; ++q) {
      uint4 v = vb[q];
      if (RESID) {  // a separate bf16 add after the GEMM: one more rounding
        const uint32_t a[4] = {v.x, v.y, v.z, v.w}, b[4] = {rb[q].x, rb[q].y, rb[q].z, rb[q].w};
        uint32_t o[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          o[u] = pack_bf16x2(__uint_as_float(a[u] << 16) + __uint_as_float(b[u] << 16),
                             __uint_as_float(a[u] & 0xffff0000u) + __uint_as_float(b[u] & 0xffff0000u));
        v = make_uint4(o[0], o[1], o[2], o[3]);
      }
      if constexpr (kStreamOut) {
        typedef unsigned v4u_nt __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(v4u_nt{v.x, v.y, v.z, v.w}, (v4u_nt*)(gbase + goff + (uint32_t)(p0 + q) * gstep));
      } else {
        *(uint4*)(gbase + goff + (uint32_t)(p0 + q) * gstep) = v;
      }
    }
  }
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
  // wave-uniform: the whole wave tile is inside the output and the vector paths apply
  if (m0 + WT_M <= M && n0 + WT_N <= N && (N & 7) == 0 && ((uintptr_t)bias & 7u) == 0) {
    if (bias) {
      if (residual) wave_tile_store_interior<TN, TM, NWAVES, true, true>(acc, smem, y, bias, alpha, n0, m0, wave, lane, N, residual);
      else wave_tile_store_interior<TN, TM, NWAVES, true, false>(acc, smem, y, bias, alpha, n0, m0, wave, lane, N, residual);
    } else {
      if (residual) wave_tile_store_interior<TN, TM, NWAVES, false, true>(acc, smem, y, bias, alpha, n0, m0, wave, lane, N, residual);
      else wave_tile_store_interior<TN, TM, NWAVES, false, false>(acc, smem, y, bias, alpha, n0, m0, wave, lane, N, residual);
    }
    return;
  }
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
  // Batches of kBatch rows-per-instruction groups: all LDS reads of a batch are issued before its
  // first store, so the stores do not each wait for an LDS round trip.
  constexpr int kIters = WT_M / kRpi;
  constexpr int kBatch = kIters % 8 == 0 ? 8 : (kIters % 4 == 0 ? 4 : 1);
  if (cc * 16 >= kRowBytes) return;
#pragma unroll 1
  for (int p0 = 0; p0 < kIters; p0 += kBatch) {
    uint4 vb[kBatch];
#pragma unroll
    for (int q = 0; q < kBatch; ++q) vb[q] = *(const uint4*)(stg + ((p0 + q) * kRpi + rr) * kStride + cc * 16);
#pragma unroll
    for (int q = 0; q < kBatch; ++q) {
      uint4 v = vb[q];
      const int ml = (p0 + q) * kRpi + rr;
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
