// Fused rotate + group-scale + E2M1 pack kernels (MXFP4 / NVFP4) for gfx950.
//
// The rotation is a block Walsh-Hadamard transform evaluated as fp32 radix-2 butterflies with
// strides 1, 2, ..., g/2 on the exact products x[i] * norm, i.e. x @ H for the +-norm Sylvester
// matrix the reference builds (inference_lib/src/fp_quant/module/linear.py:24-30) with a fixed
// summation tree, so that results can be reproduced bit for bit on a CPU.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/fpq.h"
#include "fpq_device.h"
#include "fpq_gemm_epilogue.h"  // LdsLimitOnce

namespace fpq {

#ifndef FPQ_EPL
#define FPQ_EPL 64  // elements owned by one lane in the streaming kernel (64 or 128)
#endif

constexpr int kFmtMx = 0;
constexpr int kFmtNv = 1;

// -------------------------------------------------------------------------------------------
// Generic kernel: one lane owns 8 consecutive elements (one 16-byte load, 4 bytes of codes).
// A rotation block of G elements spans G/8 neighbouring lanes; the butterflies with stride
// >= 8 exchange registers between lanes.  Works for any cols % max(G, GROUP) == 0.
//
// lane8_load_rotate leaves the lane's 8 rotated values of chunk `chunk` in p (zeros for an
// inactive lane).  Must be called by all 64 lanes of a wave with consecutive chunk indices
// (inactive lanes pass active = false).
//
// A prologue computes the tensor that is quantized from its producer's inputs, so that the bf16
// intermediate never travels through memory (src/utils/llama_utils.py:60-71: act_fn(gate) * up
// feeds down_proj's quantizer, the RMSNorm output feeds those of q/k/v and gate/up).  Each
// PyTorch operator of the unfused sequence rounds to bf16 once, and so do these:
//   kProRmsNorm  bf16(gamma[c] * bf16(x[r, c] * inv_rms[r]))
//   kProSiluMul  bf16(bf16(silu(x[r, c])) * second[r, c]),  silu(g) = g / (1 + exp_det(-g))
// with plain fp32 multiplies, adds and divisions in a fixed order (this file is built without
// contraction), so a CPU reproduces every bit.
constexpr int kProNone = 0;
constexpr int kProRmsNorm = 1;
constexpr int kProSiluMul = 2;

struct Prologue {
  const float* row_scale;   // kProRmsNorm: 1 / rms per row
  const uint4* col_scale;   // kProRmsNorm: bf16 weight per column
  const uint4* second;      // kProSiluMul: the multiplier ("up") tensor
  uint4* out;               // optional: the prologue's bf16 result, row-major [rows, cols]
  uint32_t chunks_per_row;  // cols / 8
  uint32_t ld_first;        // row stride of x in 8-element chunks
  uint32_t ld_second;       // row stride of `second` in 8-element chunks
  uint32_t packed_rows;     // generic kernel only: 0 = row-major codes and scales; otherwise the row count
                            // padded to a multiple of 32, and codes / scales are written in the packed
                            // operand layout of the GEMMs (padded rows: zero codes, zero scale bytes)
};

// Packed operand layout, as 32-bit word / byte indices: the 4 code bytes of the 8-element chunk `cc`
// of `row`, and the scale byte of its group (MXFP4: group of 32 = 4 chunks, NVFP4: 16 = 2 chunks).
__device__ __forceinline__ uint32_t packed_code_word(uint32_t row, uint32_t cc, uint32_t chunks_per_row) {
  const uint32_t rt = row >> 5, r = row & 31u, ks = cc >> 3, kh = (cc >> 2) & 1u;
  return ((rt * (chunks_per_row >> 3) + ks) * 64u + kh * 32u + r) * 4u + (cc & 3u);
}
template <int FMT>
__device__ __forceinline__ uint32_t packed_scale_byte(uint32_t row, uint32_t cc, uint32_t chunks_per_row) {
  const uint32_t rt = row >> 5, r = row & 31u, kb = cc >> 5;
  if (FMT == kFmtMx) {
    const uint32_t gi = (cc >> 2) & 7u;   // group of the 256-K block: byte q = gi / 2 of lane slot kh = gi % 2
    return ((rt * (chunks_per_row >> 5) + kb) * 64u + (gi & 1u) * 32u + r) * 4u + (gi >> 1);
  }
  const uint32_t gi = (cc >> 1) & 15u;    // gi = 4 q + 2 kh + b: byte 2 q + b of lane slot kh
  return ((rt * (chunks_per_row >> 5) + kb) * 64u + ((gi >> 1) & 1u) * 32u + r) * 8u + 2u * (gi >> 2) + (gi & 1u);
}

__device__ __forceinline__ float bf16_rne(float v) {
  uint32_t b = __float_as_uint(v);
  b += 0x7fffu + ((b >> 16) & 1u);
  return __uint_as_float(b & 0xffff0000u);
}

// exp(t): clamp to +-200, n = rint(t * log2e), r = (t - n*ln2_hi) - n*ln2_lo (n*ln2_hi is exact),
// degree-5 Horner polynomial with separate multiplies and adds, ldexp by n (overflows to inf,
// underflows gradually).  Within 1e-7 of exp over the whole range.
__device__ __forceinline__ float exp_det(float t) {
  t = t < -200.0f ? -200.0f : t;
  t = t > 200.0f ? 200.0f : t;
  const float n = __builtin_rintf(t * 1.44269504088896341f);
  const float r = (t - n * 0.693359375f) - n * -2.12194440e-4f;
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  const float y = (p * (r * r) + r) + 1.0f;
  return __builtin_ldexpf(y, (int)n);
}

// bf16(silu(g)) for every bf16 bit pattern g, filled once per device by silu_table_kernel: the
// activation costs one 2-byte lookup per element (the hot part of the table stays in the L1)
// instead of ~50 VALU operations, which would make the fused kernel compute-bound.
__device__ uint16_t g_silu_table[65536];

__global__ __launch_bounds__(256) void silu_table_kernel() {
  const uint32_t bits = blockIdx.x * 256u + threadIdx.x;
  const float g = __uint_as_float(bits << 16);
  g_silu_table[bits] = (uint16_t)(__float_as_uint(bf16_rne(g / (1.0f + exp_det(-g)))) >> 16);
}

__device__ __forceinline__ float silu_bf16(uint32_t bits) {
  return __uint_as_float((uint32_t)g_silu_table[bits] << 16);
}

__device__ __forceinline__ void unpack8(const uint4& raw, float (&p)[8]) {
  p[0] = bf16_lo(raw.x); p[1] = bf16_hi(raw.x);
  p[2] = bf16_lo(raw.y); p[3] = bf16_hi(raw.y);
  p[4] = bf16_lo(raw.z); p[5] = bf16_hi(raw.z);
  p[6] = bf16_lo(raw.w); p[7] = bf16_hi(raw.w);
}

template <int G, int ROT, int PRO = kProNone>
__device__ __forceinline__ void lane8_load_rotate(const uint4* __restrict__ x, uint32_t chunk, bool active,
                                                  uint32_t lane, float norm, float* __restrict__ stage,
                                                  const uint16_t* __restrict__ hmat, float (&p)[8],
                                                  const Prologue& pro = Prologue{}, float row_scale = 0.0f) {
  // kProRmsNorm: the row's 1 / rms is pro.row_scale[row]; a caller that computed it in this launch leaves
  // pro.row_scale null and passes the value as row_scale (any value, NaN and infinity included, is data)
  uint4 raw = make_uint4(0u, 0u, 0u, 0u);
  if (PRO == kProNone) {
    if (active) raw = x[chunk];
    unpack8(raw, p);
  } else {
    uint4 aux = make_uint4(0u, 0u, 0u, 0u);
    float rs = 0.0f;
    if (active) {
      const uint32_t row = chunk / pro.chunks_per_row, cc = chunk - row * pro.chunks_per_row;
      raw = x[(size_t)row * pro.ld_first + cc];
      if (PRO == kProRmsNorm) {
        aux = pro.col_scale[cc];
        rs = pro.row_scale ? pro.row_scale[row] : row_scale;
      } else {
        aux = pro.second[(size_t)row * pro.ld_second + cc];
      }
    }
    float q[8];
    unpack8(raw, p);
    unpack8(aux, q);
    if (PRO == kProSiluMul) {
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[2 * i] = silu_bf16(w[i] & 0xffffu);
        p[2 * i + 1] = silu_bf16(w[i] >> 16);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float t = PRO == kProRmsNorm ? bf16_rne(p[i] * rs) : p[i];
      p[i] = bf16_rne(t * q[i]);
    }
    if (active && pro.out) {
      pro.out[chunk] = make_uint4((__float_as_uint(p[0]) >> 16) | (__float_as_uint(p[1]) & 0xffff0000u),
                                  (__float_as_uint(p[2]) >> 16) | (__float_as_uint(p[3]) & 0xffff0000u),
                                  (__float_as_uint(p[4]) >> 16) | (__float_as_uint(p[5]) & 0xffff0000u),
                                  (__float_as_uint(p[6]) >> 16) | (__float_as_uint(p[7]) & 0xffff0000u));
    }
  }

  if (ROT == FPQ_ROT_HADAMARD || ROT == FPQ_ROT_GSR) {
#pragma unroll
    for (int i = 0; i < 8; ++i) p[i] = p[i] * norm;
#pragma unroll
    for (int s = 1; s < 8; s *= 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if ((i & s) == 0) {
          const float a = p[i], b = p[i + s];
          p[i] = a + b;
          p[i + s] = a - b;
        }
      }
    }
#pragma unroll
    for (int s = 8; s < G; s *= 2) {
      const int lm = s / 8;
      const bool upper = (lane & lm) != 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float other = __shfl_xor(p[i], lm, 64);
        p[i] = upper ? other - p[i] : p[i] + other;
      }
    }
  }
  if (ROT == FPQ_ROT_GSR) {
    // sequency order: output k of a block is Hadamard output bitreverse(k ^ (k >> 1))
    // (inference_lib/src/fp_quant/module/linear.py:37-41); gathered through the wave's LDS stage
    constexpr int LOG2G = G == 16 ? 4 : G == 32 ? 5 : G == 64 ? 6 : 7;
    const uint32_t first = lane & ~(uint32_t)(G / 8 - 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) stage[lane * 8u + i] = p[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t k = (lane - first) * 8u + i;
      const uint32_t j = __brev(k ^ (k >> 1)) >> (32 - LOG2G);
      p[i] = stage[first * 8u + j];
    }
  }
  if (ROT == FPQ_ROT_GENERAL) {
    // arbitrary matrix: y[j] = sum_i x[i] * H[i][j], fp32 fused multiply-adds in the order i = 0..G-1
    const uint32_t first = lane & ~(uint32_t)(G / 8 - 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) stage[lane * 8u + i] = p[i];
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const uint16_t* hcol = hmat + (lane - first) * 8u;
#pragma unroll 4
    for (int ii = 0; ii < G; ++ii) {
      const float xi = stage[first * 8u + ii];
      const uint4 hv = *(const uint4*)(hcol + ii * G);
      acc[0] = __builtin_fmaf(xi, bf16_lo(hv.x), acc[0]); acc[1] = __builtin_fmaf(xi, bf16_hi(hv.x), acc[1]);
      acc[2] = __builtin_fmaf(xi, bf16_lo(hv.y), acc[2]); acc[3] = __builtin_fmaf(xi, bf16_hi(hv.y), acc[3]);
      acc[4] = __builtin_fmaf(xi, bf16_lo(hv.z), acc[4]); acc[5] = __builtin_fmaf(xi, bf16_hi(hv.z), acc[5]);
      acc[6] = __builtin_fmaf(xi, bf16_lo(hv.w), acc[6]); acc[7] = __builtin_fmaf(xi, bf16_hi(hv.w), acc[7]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) p[i] = acc[i];
  }
}

// Rotates and quantizes the lane's 8 elements: abs-max scales, or with QUEST (MXFP4 only) the
// reference's "quest" rule (inference_lib/src/fp_quant/module/triton/mxfp4.py:51-59, constant from
// pseudoquant_linear_fns.py:20-22): s = 2^floor(log2(fl(2.92247856/6) * std + 1e-8)) with the
// population standard deviation of the 32 rotated values, values beyond +-6 s saturate, and the
// optional mask gets bit (element % 8) of byte [row, element / 8] set where |x / s| < 6
// (mxfp4.py:105-110, linear_fns.py:67-76).  fp32 evaluation order, fixed so that a CPU can
// reproduce it: per octet of consecutive elements the sums of x and of fl(x*x) run left to right,
// the four octet sums combine as (o0 + o1) + (o2 + o3); mean = sum/32, var = max(msq - fl(mean*mean), 0).
template <int G, int FMT, int ROT, int ZERO, bool QUEST = false, int PRO = kProNone>
__device__ __forceinline__ void lane8_process(const uint4* __restrict__ x, uint32_t* __restrict__ codes,
                                              uint8_t* __restrict__ scales, uint32_t chunk, bool active,
                                              uint32_t lane, uint32_t chunks_per_row,
                                              uint32_t scale_stride, float norm, float gscale, float rg,
                                              float* __restrict__ stage, const uint16_t* __restrict__ hmat,
                                              uint8_t* __restrict__ mask = nullptr,
                                              const Prologue& pro = Prologue{}, float row_scale = 0.0f) {
  static_assert(!QUEST || FMT == kFmtMx, "the quest rule exists for MXFP4 only");
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  float p[8];
  lane8_load_rotate<G, ROT, PRO>(x, chunk, active, lane, norm, stage, hmat, p, pro, row_scale);

  if (QUEST) {
    float sum = p[0], sq = p[0] * p[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) {
      sum = sum + p[i];
      sq = sq + p[i] * p[i];
    }
#pragma unroll
    for (int lm = 1; lm < 4; lm *= 2) {
      sum = sum + __shfl_xor(sum, lm, 64);
      sq = sq + __shfl_xor(sq, lm, 64);
    }
    const float mean = sum * 0.03125f, msq = sq * 0.03125f;
    float var = msq - mean * mean;
    var = var > 0.0f ? var : 0.0f;
    const float sc = __builtin_sqrtf(var) * 0.48707976f + 1e-8f;   // fl32(2.92247856 / 6)
    const uint32_t ex = (__float_as_uint(sc) >> 23) & 0xffu;        // sc >= 1e-8: a normal number
    const float inv = __builtin_ldexpf(1.0f, 127 - (int)ex);        // 1 / s, exact
    uint32_t packed = 0u, mbits = 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float q = p[i] * inv;                                    // exact unless it underflows
      packed |= e2m1_code<ZERO>(q) << (4 * i);
      mbits |= (uint32_t)(__builtin_fabsf(q) < 6.0f) << i;
    }
    if (pro.packed_rows != 0u) {   // packed operand layout (no mask there); pad rows get zeros
      if (chunk < pro.packed_rows * chunks_per_row) {
        const uint32_t row = chunk / chunks_per_row, cc = chunk - row * chunks_per_row;
        codes[packed_code_word(row, cc, chunks_per_row)] = active ? packed : 0u;
        if ((cc & 3u) == 0u) scales[packed_scale_byte<FMT>(row, cc, chunks_per_row)] = active ? (uint8_t)ex : (uint8_t)0;
      }
      return;
    }
    if (active) {
      codes[chunk] = packed;
      if (mask) mask[chunk] = (uint8_t)mbits;
      if ((chunk & 3u) == 0u) {
        const uint32_t row = chunk / chunks_per_row;
        const uint32_t col = (chunk - row * chunks_per_row) / 4u;
        scales[(size_t)row * scale_stride + col] = (uint8_t)ex;
      }
    }
    return;
  }

  float a = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) a = __builtin_fmaxf(a, __builtin_fabsf(p[i]));
#pragma unroll
  for (int lm = 1; lm < GROUP / 8; lm *= 2) a = __builtin_fmaxf(a, __shfl_xor(a, lm, 64));

  GroupScale gs;
  if (FMT == kFmtMx) {
    gs = mx_group_scale(a);
  } else {
    gs = nv_group_scale(a, gscale, rg);
  }

  uint32_t packed = 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float v = scale_element(p[i], gs);
    if (ZERO == kZeroSigned) v = __builtin_copysignf(v, p[i]);  // x / s keeps the sign of x, also for -0
    if (FMT == kFmtNv) v = gs.zero ? 0.0f : v;
    packed |= e2m1_code<ZERO>(v) << (4 * i);
  }

  if (!QUEST && pro.packed_rows != 0u) {
    if (chunk < pro.packed_rows * chunks_per_row) {
      const uint32_t row = chunk / chunks_per_row, cc = chunk - row * chunks_per_row;
      codes[packed_code_word(row, cc, chunks_per_row)] = active ? packed : 0u;
      if ((cc & (GROUP / 8 - 1)) == 0u) {
        scales[packed_scale_byte<FMT>(row, cc, chunks_per_row)] = active ? (uint8_t)gs.byte : (uint8_t)0;
      }
    }
    return;
  }
  if (active) {
    codes[chunk] = packed;
    if ((chunk & (GROUP / 8 - 1)) == 0u) {
      const uint32_t row = chunk / chunks_per_row;
      const uint32_t col = (chunk - row * chunks_per_row) / (GROUP / 8);
      scales[(size_t)row * scale_stride + col] = (uint8_t)gs.byte;
    }
  }
}

// zero-fill the padded part of a scale tensor (rows >= rows, columns >= valid_cols)
__device__ __forceinline__ void fill_scale_padding(uint8_t* __restrict__ scales, uint32_t rows,
                                                   uint32_t valid_cols, uint32_t scale_rows,
                                                   uint32_t scale_stride) {
  if (scale_rows != rows || scale_stride != valid_cols) {
    const uint32_t total = scale_rows * scale_stride;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
      const uint32_t r = i / scale_stride;
      const uint32_t c = i - r * scale_stride;
      if (r >= rows || c >= valid_cols) scales[i] = 0;
    }
  }
}

// Generic kernel: works for any cols % max(G, GROUP) == 0; one 8-element chunk per thread.
template <int G, int FMT, int ROT, int ZERO, bool QUEST = false, int PRO = kProNone>
__global__ __launch_bounds__(256) void quantize_lane8_kernel(
    const uint4* __restrict__ x, uint32_t* __restrict__ codes, uint8_t* __restrict__ scales,
    uint32_t n_chunks, uint32_t chunks_per_row, uint32_t rows, uint32_t scale_rows,
    uint32_t scale_stride, float norm, const float* __restrict__ global_scale,
    const uint16_t* __restrict__ h, uint8_t* __restrict__ mask = nullptr, Prologue pro = Prologue{}) {
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  constexpr bool kStage = ROT == FPQ_ROT_GSR || ROT == FPQ_ROT_GENERAL;
  __shared__ float stage[kStage ? 4 : 1][kStage ? 512 : 1];
  __shared__ __attribute__((aligned(16))) uint16_t hmat[ROT == FPQ_ROT_GENERAL ? G * G : 8];
  if (ROT == FPQ_ROT_GENERAL) {
    for (int i = threadIdx.x; i < G * G; i += 256) hmat[i] = h[i];
    __syncthreads();
  }
  const uint32_t chunk = blockIdx.x * 256u + threadIdx.x;
  float g = 1.0f, rg = 1.0f;
  if (FMT == kFmtNv) {
    g = *global_scale;
    rg = g == 0.0f ? 0.0f : 1.0f / g;
  }
  lane8_process<G, FMT, ROT, ZERO, QUEST, PRO>(x, codes, scales, chunk, chunk < n_chunks, threadIdx.x & 63u,
                                               chunks_per_row, scale_stride, norm, g, rg,
                                               stage[kStage ? (threadIdx.x >> 6) : 0], hmat, mask, pro);
  fill_scale_padding(scales, rows, chunks_per_row / (GROUP / 8), scale_rows, scale_stride);
}

template <int G, int FMT, int ROT>
static int launch_lane8(const void* x, int64_t rows, int64_t cols, float norm, const float* gsp,
                        void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                        int zero_policy, hipStream_t stream, const void* h = nullptr, bool packed = false) {
  const int64_t n_chunks = rows * cols / 8;
  Prologue pro{};
  pro.packed_rows = packed ? (uint32_t)((rows + 31) / 32 * 32) : 0u;
  const int64_t threads = packed ? (int64_t)pro.packed_rows * (cols / 8) : n_chunks;
  const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  auto args = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const uint4*)x, (uint32_t*)codes,
                       (uint8_t*)scales, (uint32_t)n_chunks, (uint32_t)(cols / 8), (uint32_t)rows,
                       (uint32_t)scale_rows, (uint32_t)scale_stride, norm, gsp, (const uint16_t*)h,
                       (uint8_t*)nullptr, pro);
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroReference>);
  } else {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroSigned>);
  }
  return (int)hipGetLastError();
}

// -------------------------------------------------------------------------------------------
// Streaming kernel for cols % 64 == 0 (EPL = 32, 64 or 128): one lane owns EPL consecutive elements
// (2*EPL bytes in, EPL/2 bytes of codes and EPL/32 or EPL/16 scale bytes out), so the butterfly
// stages with stride < EPL, every group maximum and the packing stay inside the lane's registers;
// a rotation wider than EPL adds one or two exchanges between neighbouring lanes.  Inputs below 2^24
// elements run with EPL = 32: every wave then owns at most a tile or two, all loads are issued at once
// and the arithmetic of the wave whose data arrive last is exposed -- half the tile, half that tail
// (2048 x 4096, Hadamard 128: 7.4 -> 6.5 us; from 2^24 elements on the two sizes measure alike).  A wave moves
// 64 such chunks per tile: direct global -> LDS loads in full contiguous runs, then each lane
// reads its own chunk back with 16-byte LDS reads.  The 16-byte pieces of a chunk are
// XOR-swizzled by the lane number (through the choice of the piece each DMA lane fetches) so
// those reads are bank-conflict free.  Codes return through the same LDS region so that global
// stores are contiguous.
constexpr float kKappa = -0x1.8p-26f;  // fma(x, 0.75, x * kKappa) rounds to the E2M1 code of x / fl(4/3)

// Hadamard output index that sequency-ordered output k of a g-block takes: bitreverse(k ^ (k >> 1))
__host__ __device__ constexpr int gsr_source(int k, int g) {
  int gray = k ^ (k >> 1), r = 0;
  for (int b = 1; b < g; b <<= 1) {
    r = (r << 1) | (gray & 1);
    gray >>= 1;
  }
  return r;
}

// 16-byte store that does not ask the L2 to keep the line: the streaming kernel's codes are written once
// and read by a later kernel (2-3 % on the whole kernel against plain stores).
__device__ __forceinline__ void store16_nt(uint8_t* p, uint4 v) {
  typedef unsigned v4u_nt __attribute__((ext_vector_type(4)));
  __builtin_nontemporal_store(v4u_nt{v.x, v.y, v.z, v.w}, (v4u_nt*)p);
}

template <int ZERO>
__device__ __forceinline__ uint32_t fix_zero_nibbles(uint32_t w) {
  if (ZERO == kZeroReference) {
    const uint32_t nz = ((w & 0x77777777u) + 0x77777777u) & 0x88888888u;  // bit 3 set where magnitude != 0
    w |= nz ^ 0x88888888u;
  }
  return w;
}

//
// PACKED (EPL = 64, or 32 without a prologue) writes the operand layout of fpq_gemm_mxf4_packed /
// fpq_gemm_nvf4_packed instead of row-major codes and scales.  A wave tile is then 32 rows x two
// neighbouring chunks (lane = 2 * row + chunk, so the lane pairing of a rotation wider than a chunk is
// unchanged): the loads are 256-byte (128-byte) row segments, and every 16 bytes of a lane's codes are
// exactly one lane slot of a packed kilobyte block, so codes are stored straight from registers in two
// 512-byte runs per store.
//
// PRO != kProNone (PACKED only) applies a producer's arithmetic to the values as they leave LDS (see
// Prologue): kProRmsNorm scales by the row's 1/rms and the column's weight (16-byte loads that hit
// the L1: a wave touches two 128-byte pieces of the weight) and can write the bf16 result;
// kProSiluMul streams a second tile (the multiplier) through LDS next to the first and looks the
// activation up in an LDS copy of the silu table's busy part (|g| in [2^-14, 128)), the rest in the
// global table.
constexpr uint32_t kSiluLdsFirst = 113u << 7;         // bf16 magnitude bits of 2^-14
constexpr uint32_t kSiluLdsCount = 21u * 128u;        // magnitudes up to (not including) 2^7

// QUEST (MXFP4, no prologue): the scale of a group comes from its standard deviation instead of its
// maximum (the rule and its fixed fp32 summation order are stated at lane8_process); a lane holds whole
// groups, so the statistic needs no cross-lane step, the scale is a power of two, and the conversion
// instruction divides by it exactly and saturates at +-6.
template <int EPL, int G, int FMT, int ROT, int ZERO, bool PACKED = false, int PRO = kProNone, bool QUEST = false>
__global__ __launch_bounds__(256, 2) void quantize_stream_kernel(
    const uint8_t* __restrict__ x, uint8_t* __restrict__ codes, uint8_t* __restrict__ scales,
    uint32_t n_chunks, uint32_t chunks_per_row, uint32_t rows, uint32_t scale_rows,
    uint32_t scale_stride, float norm, const float* __restrict__ global_scale, Prologue pro) {
  static_assert(!PACKED || EPL == 64 || (EPL == 32 && PRO == kProNone),
                "packed output: 64-element chunks; 32-element chunks without a prologue");
  static_assert(PRO == kProNone || PACKED, "prologues exist for the packed output only");
  static_assert(!QUEST || (FMT == kFmtMx && PRO == kProNone), "the quest rule exists for plain MXFP4 only");
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  constexpr int NG = EPL / GROUP;        // groups (= scale bytes) per chunk
  constexpr int PIECES = EPL / 8;        // 16-byte input pieces per chunk
  constexpr uint32_t CB = EPL * 2;       // input bytes per chunk
  constexpr uint32_t TILE = 64 * CB;     // input bytes per wave tile
  constexpr int CPI = 64 / PIECES;       // chunks filled by one DMA instruction
  constexpr int CW = EPL / 8;            // code dwords per chunk
  constexpr int CQ = CW / 4;             // 16-byte code pieces per chunk
  __shared__ __attribute__((aligned(128))) uint8_t smem[4][TILE];
  // kProSiluMul: the second tile of every wave and the table copy live in dynamic LDS (together
  // with the static part they exceed the 64 KB a kernel gets without asking); kProRmsNorm: a tile
  // per wave for regrouping the by-product
  extern __shared__ __attribute__((aligned(128))) uint8_t dyn_lds[];
  uint16_t* silu_lds = (uint16_t*)(dyn_lds + 4 * TILE);
  // lookups go through a pointer that names the LDS address space, so that they are LDS reads and
  // not flat loads (which take the texture path)
  typedef __attribute__((address_space(3))) const uint16_t lds_u16;
  lds_u16* silu_tab = (lds_u16*)silu_lds;
  __shared__ float2 lut[128];
  if (PRO == kProSiluMul) {
    for (uint32_t i = threadIdx.x; i < 2u * kSiluLdsCount; i += 256u) {
      const uint32_t sgn = i >= kSiluLdsCount ? 1u : 0u;
      silu_lds[i] = g_silu_table[(sgn << 15) | (kSiluLdsFirst + i - sgn * kSiluLdsCount)];
    }
    __syncthreads();
  }

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u;
  uint8_t* my = smem[wave];
  const uint32_t my_base = (uint32_t)(uintptr_t)my;
  uint8_t* my2 = dyn_lds + (PRO != kProNone ? wave : 0) * TILE;
  const uint32_t my2_base = (uint32_t)(uintptr_t)my2;

  float gs = 1.0f, rg = 1.0f;
  bool nv_fast = true;
  if (FMT == kFmtNv) {
    gs = *global_scale;
    rg = gs == 0.0f ? 0.0f : 1.0f / gs;
    // with 2^-60 <= gs <= 2^60 no product of an E4M3 value with gs or 1/gs leaves the normal range
    nv_fast = gs >= 8.673617379884035e-19f && gs <= 1.152921504606847e18f;
    if (threadIdx.x < 128) {
      const float s = e4m3_decode(threadIdx.x) * rg;
      float2 e = make_float2(0.0f, 0.0f);
      if (s != 0.0f && nv_fast) {
        const float y = 1.0f / s;
        e = make_float2(y, __builtin_fmaf(-s, y, 1.0f) / s);
      }
      lut[threadIdx.x] = e;
    }
    __syncthreads();
  }

  // DMA lane map: instruction i fills LDS pieces [64 i, 64 i + 64); piece p = PIECES * b + j
  // belongs to chunk b and holds that chunk's 16-byte piece j ^ sw(b).  sw(b) is chosen so that
  // the 16-byte reads "piece k of my own chunk" of all lanes hit every LDS bank group once per
  // pass (checked with the bank-conflict counter): b % 16 for 256-byte chunks,
  // (b % 8) ^ ((b / 8) & 1) for 128-byte chunks and (b / 4) % 4 for 64-byte chunks.
  auto sw = [](uint32_t b) -> uint32_t {
    return PIECES == 8 ? ((b & 7u) ^ ((b >> 3) & 1u)) : PIECES == 4 ? ((b >> 2) & 3u) : (b % PIECES);
  };
  const uint32_t b_lo = lane / PIECES, j_lo = lane % PIECES;
  constexpr int NV_OFF = PIECES == 8 ? 2 : 4;  // distinct swizzle phases over the instruction index
  // bytes from one row to the next (a prologue's inputs may sit in wider buffers)
  const uint32_t row_bytes = PRO == kProNone ? chunks_per_row * CB : pro.ld_first * 16u;
  const uint32_t row_bytes2 = PRO == kProSiluMul ? pro.ld_second * 16u : 0u;
  // PACKED: chunk b of the tile is row b / CPR of the tile, chunk b % CPR of its columns.  With 64-element
  // chunks a tile is the 32 rows of a row tile x 2 chunks; with 32-element chunks it is 16 rows (half a row
  // tile) x 4 chunks, so that the 128 columns of the widest rotation still sit in neighbouring lanes.
  constexpr bool P32 = PACKED && EPL == 32;
  constexpr uint32_t CPR = P32 ? 4u : 2u;     // chunks per row of a packed tile
  constexpr uint32_t RPI = CPI / CPR;         // rows filled by one DMA instruction
  const uint32_t b_off = PACKED ? (b_lo / CPR) * row_bytes + (b_lo % CPR) * CB : b_lo * CB;
  uint32_t voff[NV_OFF], voff2[PRO == kProSiluMul ? NV_OFF : 1];
#pragma unroll
  for (int m = 0; m < NV_OFF; ++m) {
    voff[m] = b_off + ((j_lo ^ sw(CPI * m + b_lo)) * 16u);
    if (PRO == kProSiluMul) voff2[m] = voff[m] - (b_lo >> 1) * row_bytes + (b_lo >> 1) * row_bytes2;
  }
  const uint32_t rd_base = lane * CB, l_sw = sw(lane);

  const uint32_t pairs = chunks_per_row / CPR;  // PACKED: tiles side by side in a row (half) tile
  const uint32_t n_tiles = PACKED ? ((rows + 31u) / 32u) * pairs * (P32 ? 2u : 1u) : (n_chunks + 63u) / 64u;
  const uint32_t total_waves = gridDim.x * 4u;
  for (uint32_t tile = blockIdx.x * 4u + wave; tile < n_tiles; tile += total_waves) {
    const uint32_t per_rt = pairs * (P32 ? 2u : 1u);
    const uint32_t rt = PACKED ? tile / per_rt : 0u;
    const uint32_t hh = P32 ? (tile - rt * per_rt) / pairs : 0u;             // which 16 rows of the row tile
    const uint32_t pr = PACKED ? tile - rt * per_rt - hh * pairs : 0u;
    // chunks (row-major) or rows (PACKED) of this tile that exist
    const uint32_t rows_rt = PACKED ? min(32u, rows - rt * 32u) : 0u;
    const uint32_t valid = P32      ? (rows_rt > 16u * hh ? min(16u, rows_rt - 16u * hh) : 0u)
                           : PACKED ? rows_rt
                                    : min(64u, n_chunks - tile * 64u);
    if (P32 && valid == 0u) {
      // sixteen padding rows of the last row tile: zero codes and scale bytes, nothing to read
      const uint32_t units = chunks_per_row / 2u, unit = 2u * pr + ((lane >> 1) & 1u);
      const uint32_t slot = (lane & 1u) * 32u + 16u * hh + (lane >> 2);
      store16_nt(codes + (((size_t)rt * units + unit) * 64u + slot) * 16u, make_uint4(0u, 0u, 0u, 0u));
      uint8_t* sblk = scales + ((size_t)rt * (units / 4u) + (unit >> 2)) * (FMT == kFmtMx ? 256u : 512u);
      if (FMT == kFmtMx) sblk[slot * 4u + (unit & 3u)] = 0;
      else *(uint16_t*)(sblk + slot * 8u + 2u * (unit & 3u)) = 0;
      continue;
    }
    const uint8_t* src = PACKED ? x + ((size_t)rt * 32u + 16u * hh) * row_bytes + (size_t)(CPR * pr) * CB
                                : x + (size_t)tile * TILE;
    const uint8_t* src2 = PRO == kProSiluMul
                              ? (const uint8_t*)pro.second + (size_t)rt * 32u * row_bytes2 + (size_t)(2u * pr) * CB
                              : nullptr;
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      // The lane offset is an unsigned 32-bit addend to a scalar base, so it must never be
      // negative.  Chunks past the end of the tensor re-read valid bytes instead: the first
      // chunk of this instruction if that one is valid, else the first chunk of the tile.
      uint32_t off = voff[i % NV_OFF];
      if (PACKED) {
        const bool instr_valid = (uint32_t)(RPI * i) < valid;              // wave-uniform
        const uint8_t* base_i = instr_valid ? src + (size_t)(RPI * i) * row_bytes : src;
        const bool past = RPI * i + b_lo / CPR >= valid;
        if (past) off = (b_lo % CPR) * CB + j_lo * 16u;
        lds_dma16_nt(base_i, off, my_base + i * 1024u);
        if (PRO == kProSiluMul) {
          const uint8_t* base2_i = instr_valid ? src2 + (size_t)(RPI * i) * row_bytes2 : src2;
          lds_dma16_nt(base2_i, past ? off : voff2[i % NV_OFF], my2_base + i * 1024u);
        }
      } else {
        const bool instr_valid = (uint32_t)(CPI * i) < valid;                // wave-uniform
        const uint8_t* base_i = instr_valid ? src + i * 1024 : src;          // scalar address arithmetic
        if (CPI * i + b_lo >= valid) off = j_lo * 16u;
        lds_dma16_nt(base_i, off, my_base + i * 1024u);  // read once: keep it out of the caches
      }
    }
    wait_vmem();

    // this lane's chunk: out of LDS, rotated
    // prologue operands of this lane: its row (clamped: padding rows of the last row tile compute on
    // a valid row's data and are zeroed before the store) and its first 8-element column chunk
    const uint32_t p_row = PRO == kProNone ? 0u : min(rt * 32u + (lane >> 1), rows - 1u);
    const uint32_t p_cc = PRO == kProNone ? 0u : (2u * pr + (lane & 1u)) * (uint32_t)PIECES;
    const float p_rs = PRO == kProRmsNorm ? pro.row_scale[p_row] : 0.0f;
    const bool p_store = PRO != kProNone && pro.out != nullptr && (lane >> 1) < valid;
    auto load_rotate = [&](float (&v)[EPL]) {
#pragma unroll
    for (int k = 0; k < PIECES; ++k) {
      const uint4 raw = *(const uint4*)(my + rd_base + ((k ^ l_sw) * 16u));
      float e[8];
      unpack8(raw, e);
      if (PRO != kProNone) {
        float q[8];
        if (PRO == kProRmsNorm) {
          unpack8(pro.col_scale[p_cc + k], q);
#pragma unroll
          for (int i = 0; i < 8; ++i) e[i] = bf16_rne(e[i] * p_rs);
        } else {
          unpack8(*(const uint4*)(my2 + rd_base + ((k ^ l_sw) * 16u)), q);
          const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const uint32_t bits = (i & 1) ? (w[i >> 1] >> 16) : (w[i >> 1] & 0xffffu);
            // the LDS read is unconditional (index clamped) and the rare global read separate, so that
            // neither turns into a flat load through a pointer that could be either
            const uint32_t idx = (bits & 0x7fffu) - kSiluLdsFirst;
            const bool in_lds = idx < kSiluLdsCount;
            uint32_t t = silu_tab[(bits >> 15) * kSiluLdsCount + (in_lds ? idx : 0u)];
            if (!in_lds) t = g_silu_table[bits];
            e[i] = __uint_as_float(t << 16);
          }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = bf16_rne(e[i] * q[i]);
        if (PRO == kProRmsNorm ? pro.out != nullptr : p_store) {
          const uint4 packed8 =
              make_uint4((__float_as_uint(e[0]) >> 16) | (__float_as_uint(e[1]) & 0xffff0000u),
                         (__float_as_uint(e[2]) >> 16) | (__float_as_uint(e[3]) & 0xffff0000u),
                         (__float_as_uint(e[4]) >> 16) | (__float_as_uint(e[5]) & 0xffff0000u),
                         (__float_as_uint(e[6]) >> 16) | (__float_as_uint(e[7]) & 0xffff0000u));
          if (PRO == kProRmsNorm) {
            // parked in the wave's second LDS tile at the input's (swizzled) place, stored below
            *(uint4*)(my2 + rd_base + ((k ^ l_sw) * 16u)) = packed8;
          } else {
            pro.out[(size_t)p_row * chunks_per_row * PIECES + p_cc + k] = packed8;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) v[8 * k + i] = e[i];
    }
    if (PRO == kProRmsNorm && pro.out != nullptr) {
      // the by-product leaves as 256-byte row segments: store i covers rows 4 i .. 4 i + 3 of the
      // tile, 16 lanes per row (the two chunks of the row, 8 pieces each)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t r = 4u * i + (lane >> 4), ls = 2u * r + ((lane >> 3) & 1u), kk = lane & 7u;
        const uint4 o = *(const uint4*)(my2 + ls * CB + ((kk ^ sw(ls)) * 16u));
        if (r < valid) {
          store16_nt((uint8_t*)(pro.out + ((size_t)rt * 32u + r) * chunks_per_row * PIECES + (size_t)(2u * pr) * PIECES +
                               (lane & 15u)), o);
        }
      }
    }
    if (ROT == FPQ_ROT_HADAMARD || ROT == FPQ_ROT_GSR) {
#pragma unroll
      for (int i = 0; i < EPL; ++i) v[i] *= norm;
#pragma unroll
      for (int s = 1; s < (G < EPL ? G : EPL); s *= 2) {
        __builtin_amdgcn_sched_barrier(0);  // keep the stages in place: EPL live values, no more
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
          if ((i & s) == 0) {
            const float a = v[i], b = v[i + s];
            v[i] = a + b;
            v[i + s] = a - b;
          }
        }
      }
      if (G > EPL) {
        // stride EPL: the two halves of a rotation block sit in lanes 2u and 2u + 1.  The even
        // lane needs a + b, the odd one a - b = (value of the even lane) + (-own value).
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t flip = (lane & 1u) << 31;
#pragma unroll
        for (int i = 0; i < EPL; ++i) {
          const float other = __uint_as_float((uint32_t)__builtin_amdgcn_mov_dpp(
              (int)__float_as_uint(v[i]), 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true));
          v[i] = other + __uint_as_float(__float_as_uint(v[i]) ^ flip);
        }
        if (G > 2 * EPL) {
          // stride 2 EPL (a 128-wide rotation with EPL = 32): the quarters of a block sit in lanes
          // 4u .. 4u + 3 and the partner is lane ^ 2
          static_assert(G <= 4 * EPL, "at most two exchanges between lanes");
          __builtin_amdgcn_sched_barrier(0);
          const uint32_t flip2 = (lane & 2u) << 30;
#pragma unroll
          for (int i = 0; i < EPL; ++i) {
            const float other = __uint_as_float((uint32_t)__builtin_amdgcn_mov_dpp(
                (int)__float_as_uint(v[i]), 0x4E /* quad_perm [2,3,0,1] */, 0xF, 0xF, true));
            v[i] = other + __uint_as_float(__float_as_uint(v[i]) ^ flip2);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (ROT == FPQ_ROT_GSR) {
      // sequency order inside every G-block (G <= EPL here): a compile-time renaming of registers
      static_assert(ROT != FPQ_ROT_GSR || G <= EPL, "GSR blocks must fit in one lane");
      float w[EPL];
#pragma unroll
      for (int k = 0; k < EPL; ++k) w[k] = v[(k & ~(G - 1)) | gsr_source(k & (G - 1), G)];
#pragma unroll
      for (int k = 0; k < EPL; ++k) v[k] = w[k];
    }
    };
    float v[EPL];
    load_rotate(v);

    uint32_t cw[CW];
    uint32_t sbytes = 0u, sb_lo = 0u;
    bool need_slow = false;
#pragma unroll
    for (int gi = 0; gi < NG; ++gi) {
      float a = 0.0f;
      if (!QUEST) {
#pragma unroll
        for (int i = 0; i < GROUP; ++i) a = __builtin_fmaxf(a, __builtin_fabsf(v[gi * GROUP + i]));
      }
      uint32_t byte;
      bool fast;
      float k1, k2, cvt_scale;
      if (QUEST) {
        float os[4], oq[4];
#pragma unroll
        for (int o = 0; o < 4; ++o) {
          const float* p = &v[gi * GROUP + 8 * o];
          float sum = p[0], sq = p[0] * p[0];
#pragma unroll
          for (int i = 1; i < 8; ++i) {
            sum = sum + p[i];
            sq = sq + p[i] * p[i];
          }
          os[o] = sum;
          oq[o] = sq;
        }
        const float sum = (os[0] + os[1]) + (os[2] + os[3]), sq = (oq[0] + oq[1]) + (oq[2] + oq[3]);
        const float mean = sum * 0.03125f, msq = sq * 0.03125f;
        float var = msq - mean * mean;
        var = var > 0.0f ? var : 0.0f;
        const float sc = __builtin_sqrtf(var) * 0.48707976f + 1e-8f;   // fl32(2.92247856 / 6); >= 1e-8: normal
        byte = (__float_as_uint(sc) >> 23) & 0xffu;
        fast = true;
        k1 = k2 = 0.0f;
        cvt_scale = __uint_as_float(byte << 23);                         // s = 2^floor(log2(sc))
      } else if (FMT == kFmtMx) {
        const uint32_t bits = __float_as_uint(a);
        byte = bits >> 23;
        fast = (byte - 29u) <= 198u || bits == 0u;                       // -98 <= e <= 100, or all zero
        k1 = 0.75f;
        k2 = kKappa;
        cvt_scale = __uint_as_float((bits & 0x7f800000u) - (2u << 23));  // 2^(e-2)
        if (bits == 0u) {  // a zero group stores 2^-126 and zero codes
          byte = 1u;
          cvt_scale = 1.0f;
        }
      } else {
        float t = div6_rn(a) * gs;
        t = t > 448.0f ? 448.0f : t;
        byte = e4m3_encode(t);
        fast = nv_fast;
        const float2 e = lut[byte & 0x7fu];
        k1 = e.x;
        k2 = e.y;
        cvt_scale = 1.0f;
      }
      need_slow |= !fast;
#pragma unroll
      for (int d = 0; d < GROUP / 8; ++d) {
        uint32_t w = 0u;
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          const float x0 = v[gi * GROUP + d * 8 + 2 * h], x1 = v[gi * GROUP + d * 8 + 2 * h + 1];
          float q0 = QUEST ? x0 : __builtin_fmaf(x0, k1, x0 * k2);
          float q1 = QUEST ? x1 : __builtin_fmaf(x1, k1, x1 * k2);
          if (ZERO == kZeroSigned && !QUEST) {  // x / s keeps the sign of x, also for -0
            q0 = __builtin_copysignf(q0, x0);
            q1 = __builtin_copysignf(q1, x1);
          }
          if (h == 0) w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, cvt_scale, 0);
          if (h == 1) w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, cvt_scale, 1);
          if (h == 2) w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, cvt_scale, 2);
          if (h == 3) w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q0, q1, cvt_scale, 3);
        }
        if (FMT == kFmtNv && ZERO == kZeroSigned) w = byte == 0u ? 0u : w;  // zero scale: +0 codes
        cw[gi * (GROUP / 8) + d] = fix_zero_nibbles<ZERO>(w);
      }
      sbytes |= (byte & 0xffu) << (8 * (gi & 3));
      if (NG == 8 && gi == 3) {  // eight scale bytes per chunk: park the first four
        sb_lo = sbytes;
        sbytes = 0u;
      }
      __builtin_amdgcn_sched_barrier(0);
    }

    if constexpr (PACKED) {
      // Scale exponents outside the fast range (tiny or huge values): redo the tile with the
      // generic per-element arithmetic; the input is still in LDS.
      if (__builtin_amdgcn_ballot_w64(need_slow) != 0ull) {
        float u[EPL];
        load_rotate(u);
        sbytes = 0u;
#pragma unroll 1
        for (int gi = 0; gi < NG; ++gi) {
          float a = 0.0f;
#pragma unroll
          for (int i = 0; i < GROUP; ++i) a = __builtin_fmaxf(a, __builtin_fabsf(u[gi * GROUP + i]));
          const GroupScale g = FMT == kFmtMx ? mx_group_scale(a) : nv_group_scale(a, gs, rg);
#pragma unroll
          for (int d = 0; d < GROUP / 8; ++d) {
            uint32_t w = 0u;
#pragma unroll
            for (int h = 0; h < 8; ++h) {
              const float xv = u[gi * GROUP + d * 8 + h];
              float q = scale_element(xv, g);
              if (ZERO == kZeroSigned) q = __builtin_copysignf(q, xv);
              if (FMT == kFmtNv) q = g.zero ? 0.0f : q;
              w |= e2m1_code<ZERO>(q) << (4 * h);
            }
            cw[gi * (GROUP / 8) + d] = w;
          }
          sbytes |= (g.byte & 0xffu) << (8 * gi);
        }
      }
      const uint32_t r = P32 ? lane >> 2 : lane >> 1, ksl = lane & 1u;
      const bool row_ok = r < valid;
      if (!row_ok) {  // padding rows of the last row tile: zero codes, zero scale bytes
#pragma unroll
        for (int k = 0; k < CW; ++k) cw[k] = 0u;
        sbytes = 0u;
      }
      if constexpr (EPL == 32) {
        // The lane (row 16 hh + r, chunk c = lane % 4 of the tile's 128 columns) holds K half c % 2 of
        // the 64-K unit 2 pr + c / 2, i.e. lane slot (c % 2) * 32 + row of that packed kilobyte block, and
        // one (MXFP4) or two (NVFP4) scale bytes: byte unit % 4 (bytes 2 (unit % 4), + 1) of that slot's
        // entry in scale block (rt, unit / 4).
        const uint32_t units = chunks_per_row / 2u, unit = 2u * pr + ((lane >> 1) & 1u);
        const uint32_t slot = ksl * 32u + 16u * hh + r;
        store16_nt(codes + (((size_t)rt * units + unit) * 64u + slot) * 16u, make_uint4(cw[0], cw[1], cw[2], cw[3]));
        if (FMT == kFmtMx) {
          uint8_t* sblk = scales + ((size_t)rt * (units / 4u) + (unit >> 2)) * 256u;
          sblk[slot * 4u + (unit & 3u)] = (uint8_t)sbytes;
        } else {
          uint8_t* sblk = scales + ((size_t)rt * (units / 4u) + (unit >> 2)) * 512u;
          *(uint16_t*)(sblk + slot * 8u + 2u * (unit & 3u)) = (uint16_t)sbytes;
        }
        asm volatile("" ::: "memory");
        continue;
      }
      const uint32_t ks = 2u * pr + ksl;
      uint8_t* blk = codes + (((size_t)rt * chunks_per_row + ks) * 64u + r) * 16u;
      store16_nt(blk, make_uint4(cw[0], cw[1], cw[2], cw[3]));              // K half 0
      store16_nt(blk + 512, make_uint4(cw[CW > 4 ? 4 : 0], cw[CW > 4 ? 5 : 1], cw[CW > 4 ? 6 : 2],
                                       cw[CW > 4 ? 7 : 3]));                // K half 1
      // scale bytes: byte (ks % 4) of dword (kh, r) in block (rt, ks / 4).  The pair of lanes
      // of a row holds bytes q and q + 1 of both dwords: the even lane stores the half-word of
      // K half 0, the odd lane that of K half 1.
      const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)sbytes, 0xB1, 0xF, 0xF, true);
      if (FMT == kFmtMx) {
        const uint32_t hw = ksl == 0u ? ((sbytes & 0xffu) | ((other & 0xffu) << 8))
                                      : (((other >> 8) & 0xffu) | (sbytes & 0xff00u));
        uint8_t* sblk = scales + ((size_t)rt * (chunks_per_row / 4u) + (pr >> 1)) * 256u;
        *(uint16_t*)(sblk + (ksl * 32u + r) * 4u + 2u * (pr & 1u)) = (uint16_t)hw;
      } else {
        // NVFP4: four E4M3 bytes per lane, two per K half.  The 8 bytes of (kh, r) in block
        // (rt, ks / 4) hold bytes 2 q, 2 q + 1 for K step q = ks % 4, so the lane pair of a row owns
        // one dword of each K half: the even lane stores that of K half 0, the odd lane that of 1.
        const uint32_t dw = ksl == 0u ? ((sbytes & 0xffffu) | (other << 16))
                                      : ((other >> 16) | (sbytes & 0xffff0000u));
        uint8_t* sblk = scales + ((size_t)rt * (chunks_per_row / 4u) + (pr >> 1)) * 512u;
        *(uint32_t*)(sblk + (ksl * 32u + r) * 8u + 4u * (pr & 1u)) = dw;
      }
      asm volatile("" ::: "memory");
      continue;
    }

    // codes: lane-major runs -> LDS (16-byte pieces swizzled so 8 neighbouring lanes hit 8
    // different bank groups) -> contiguous rows
#pragma unroll
    for (int k4 = 0; k4 < CQ; ++k4) {
      const uint32_t sw = CQ == 4 ? ((lane >> 1) & 3u) : CQ == 2 ? ((lane >> 2) & 1u) : 0u;
      *(uint4*)(my + (lane * CQ + (k4 ^ sw)) * 16u) =
          make_uint4(cw[4 * k4], cw[4 * k4 + 1], cw[4 * k4 + 2], cw[4 * k4 + 3]);
    }
    uint8_t* dst = codes + (size_t)tile * (64u * CW * 4u);
#pragma unroll
    for (int i = 0; i < CQ; ++i) {
      const uint32_t g = 64u * i + lane, l = g / CQ, k4 = g % CQ;
      const uint32_t sw = CQ == 4 ? ((l >> 1) & 3u) : CQ == 2 ? ((l >> 2) & 1u) : 0u;
      const uint4 o = *(const uint4*)(my + (l * CQ + (k4 ^ sw)) * 16u);
      if (l < valid) store16_nt(dst + g * 16u, o);
    }

    if (lane < valid) {
      const uint32_t chunk = tile * 64u + lane;
      constexpr uint32_t SB = NG;  // scale bytes per chunk: 1, 2, 4 or 8
      size_t so;
      if (scale_stride == chunks_per_row * SB) {
        so = (size_t)chunk * SB;
      } else {
        const uint32_t row = chunk / chunks_per_row;
        so = (size_t)row * scale_stride + (chunk - row * chunks_per_row) * SB;
      }
      if ((scale_stride & (SB - 1u)) == 0u) {
        if (SB == 1) scales[so] = (uint8_t)sbytes;
        else if (SB == 2) *(uint16_t*)(scales + so) = (uint16_t)sbytes;
        else if (SB == 4) *(uint32_t*)(scales + so) = sbytes;
        else *(uint2*)(scales + so) = make_uint2(sb_lo, sbytes);
      } else {
#pragma unroll
        for (uint32_t u = 0; u < SB; ++u) {
          const uint32_t word = (SB == 8 && u < 4) ? sb_lo : sbytes;
          scales[so + u] = (uint8_t)(word >> (8 * (u & 3)));
        }
      }
    }

    // Scale exponents outside the fast range (tiny, huge, or an out-of-range global scale): redo
    // the whole tile with the generic per-element arithmetic, after the stores above have landed.
    if (__builtin_amdgcn_ballot_w64(need_slow) != 0ull) {
      wait_vmem();
#pragma unroll 1
      for (uint32_t it = 0; it < (uint32_t)PIECES; ++it) {
        const uint32_t c8 = tile * (64u * PIECES) + it * 64u + lane;
        lane8_process<G, FMT, ROT, ZERO>((const uint4*)x, (uint32_t*)codes, scales, c8,
                                         c8 < n_chunks * PIECES, lane, chunks_per_row * PIECES,
                                         scale_stride, norm, gs, rg, (float*)my, nullptr);
      }
    }
    asm volatile("" ::: "memory");
  }
  if (!PACKED) fill_scale_padding(scales, rows, chunks_per_row * NG, scale_rows, scale_stride);
}

template <int EPL, int G, int FMT, int ROT, bool QUEST = false>
static int launch_stream(const void* x, int64_t rows, int64_t cols, float norm, const float* gsp,
                         void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                         int zero_policy, hipStream_t stream) {
  const int64_t n_chunks = rows * cols / EPL;
  const int64_t n_tiles = (n_chunks + 63) / 64;
  int64_t blocks = (n_tiles + 3) / 4;
  if (blocks > 1024) blocks = 1024;  // resident workgroups on 256 CUs; waves stride over the tiles
  const dim3 grid((unsigned)blocks), block(256);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const uint8_t*)x, (uint8_t*)codes,
                       (uint8_t*)scales, (uint32_t)n_chunks, (uint32_t)(cols / EPL), (uint32_t)rows,
                       (uint32_t)scale_rows, (uint32_t)scale_stride, norm, gsp, Prologue{});
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    go(quantize_stream_kernel<EPL, G, FMT, ROT, kZeroReference, false, kProNone, QUEST>);
  } else {
    go(quantize_stream_kernel<EPL, G, FMT, ROT, kZeroSigned, false, kProNone, QUEST>);
  }
  return (int)hipGetLastError();
}

// The streaming kernel with the chunk size that suits the input (see the kernel's head); a sequency-ordered
// block has to fit in one lane.
constexpr int64_t kHalfTileElements = (int64_t)1 << 24;
template <int G, int FMT, int ROT, bool QUEST = false>
static int launch_stream_sized(const void* x, int64_t rows, int64_t cols, float norm, const float* gsp,
                               void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                               int zero_policy, hipStream_t stream) {
  if constexpr (ROT != FPQ_ROT_GSR || G <= 32) {
    if (rows * cols < kHalfTileElements)
      return launch_stream<32, G, FMT, ROT, QUEST>(x, rows, cols, norm, gsp, codes, scales, scale_rows,
                                                   scale_stride, zero_policy, stream);
  }
  return launch_stream<FPQ_EPL, G, FMT, ROT, QUEST>(x, rows, cols, norm, gsp, codes, scales, scale_rows,
                                                    scale_stride, zero_policy, stream);
}

constexpr int kSiluDynLds = 4 * 64 * 128 + 2 * (int)kSiluLdsCount * 2;  // second tiles + table copy

template <int G, int ROT, int PRO = kProNone, int FMT = kFmtMx, bool QUEST = false, int EPL = 64>
static int launch_stream_packed(const void* x, int64_t rows, int64_t cols, float norm, void* codes,
                                void* scales, int zero_policy, hipStream_t stream,
                                const Prologue& pro = Prologue{}, const float* gsp = nullptr) {
  const int64_t n_tiles = ((rows + 31) / 32) * (cols / 128) * (EPL == 32 ? 2 : 1);
  int64_t blocks = (n_tiles + 3) / 4;
  // Waves stride over the tiles of a capped grid.  The SiLU*up prologue (two workgroups fit a CU, each
  // copies the table's busy part into LDS first) is best with one resident round; the RMSNorm prologue
  // measured 2 % better with a grid twice the plain kernel's (8192 x 4096 and 8192 x 14336 inputs).
  constexpr int64_t kCap = PRO == kProSiluMul ? 512 : PRO == kProRmsNorm ? 2048 : 1024;
  if (blocks > kCap) blocks = kCap;
  const dim3 grid((unsigned)blocks), block(256);
  // kProRmsNorm: one more tile per wave, in which the bf16 by-product is regrouped into row segments
  constexpr int kDyn = PRO == kProSiluMul ? kSiluDynLds : PRO == kProRmsNorm ? 4 * 64 * 128 : 0;
  int status = 0;
  auto go = [&](auto kernel) {
    if (kDyn) {
      static LdsLimitOnce limit;
      if ((status = limit.ensure((const void*)kernel, kDyn)) != 0) return;
    }
    hipLaunchKernelGGL(kernel, grid, block, kDyn, stream, (const uint8_t*)x, (uint8_t*)codes,
                       (uint8_t*)scales, (uint32_t)(rows * cols / EPL), (uint32_t)(cols / EPL),
                       (uint32_t)rows, 0u, 0u, norm, gsp, pro);
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    go(quantize_stream_kernel<EPL, G, FMT, ROT, kZeroReference, true, PRO, QUEST>);
  } else {
    go(quantize_stream_kernel<EPL, G, FMT, ROT, kZeroSigned, true, PRO, QUEST>);
  }
  if (status) return status;
  return (int)hipGetLastError();
}

// The packed streaming kernel (no prologue) with the chunk size that suits the input, as launch_stream_sized.
template <int G, int ROT, int FMT, bool QUEST = false>
static int launch_stream_packed_sized(const void* x, int64_t rows, int64_t cols, float norm, void* codes,
                                      void* scales, int zero_policy, hipStream_t stream, const float* gsp) {
  if constexpr (ROT != FPQ_ROT_GSR || G <= 32) {
    if (rows * cols < kHalfTileElements)
      return launch_stream_packed<G, ROT, kProNone, FMT, QUEST, 32>(x, rows, cols, norm, codes, scales, zero_policy,
                                                                    stream, Prologue{}, gsp);
  }
  return launch_stream_packed<G, ROT, kProNone, FMT, QUEST>(x, rows, cols, norm, codes, scales, zero_policy, stream,
                                                            Prologue{}, gsp);
}

constexpr int64_t kPackedFewRows = 64;

template <int FMT>
static int dispatch_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                           const float* gsp, void* codes, void* scales, int zero_policy, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (FMT == kFmtNv && !gsp) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 32;
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % 256 != 0) return FPQ_E_SHAPE;
  if (rows * cols >= (int64_t)1 << 34) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)codes & 15u) || ((uintptr_t)scales & 3u)) return FPQ_E_ALIGN;
  // A few rows (decode): the generic kernel spreads a row over 512 lanes and finishes sooner than the
  // streaming kernel, whose wave tile is 32 rows deep; it writes the same packed bytes.
  const bool few = rows <= kPackedFewRows;
  constexpr int64_t kGroupCols = FMT == kFmtMx ? 32 : 16;
#define FPQ_LAUNCH_PACKED(GG, RR)                                                                                 \
  {                                                                                                               \
    if (few)                                                                                                      \
      return launch_lane8<GG, FMT, RR>(x, rows, cols, norm, gsp, codes, scales, rows, cols / kGroupCols,          \
                                       zero_policy, stream, nullptr, true);                                       \
    return launch_stream_packed_sized<GG, RR, FMT>(x, rows, cols, norm, codes, scales, zero_policy, stream, gsp); \
  }
  if (rot_kind == FPQ_ROT_IDENTITY) {
    FPQ_LAUNCH_PACKED(32, FPQ_ROT_IDENTITY);
  } else if (rot_kind == FPQ_ROT_HADAMARD) {
    switch (g) {
      case 16: FPQ_LAUNCH_PACKED(16, FPQ_ROT_HADAMARD);
      case 32: FPQ_LAUNCH_PACKED(32, FPQ_ROT_HADAMARD);
      case 64: FPQ_LAUNCH_PACKED(64, FPQ_ROT_HADAMARD);
      case 128: FPQ_LAUNCH_PACKED(128, FPQ_ROT_HADAMARD);
    }
  } else if (rot_kind == FPQ_ROT_GSR) {
    switch (g) {
      case 16: FPQ_LAUNCH_PACKED(16, FPQ_ROT_GSR);
      case 32: FPQ_LAUNCH_PACKED(32, FPQ_ROT_GSR);
      case 64: FPQ_LAUNCH_PACKED(64, FPQ_ROT_GSR);
    }
    return FPQ_E_UNSUPPORTED;  // a 128-wide sequency-ordered block spans two lanes
  } else if (rot_kind == FPQ_ROT_GENERAL) {
    return FPQ_E_UNSUPPORTED;    // arbitrary matrices: quantize row-major, then fpq_pack_mxf4
  }
#undef FPQ_LAUNCH_PACKED
  return FPQ_E_ROTATION;
}

template <int G, int ROT>
static int launch_lane8_quest(const void* x, int64_t rows, int64_t cols, float norm, void* codes, void* scales,
                              int64_t scale_rows, int64_t scale_stride, void* mask, int zero_policy,
                              hipStream_t stream, const void* h, bool packed = false) {
  const int64_t n_chunks = rows * cols / 8;
  Prologue pro{};
  pro.packed_rows = packed ? (uint32_t)((rows + 31) / 32 * 32) : 0u;
  const int64_t threads = packed ? (int64_t)pro.packed_rows * (cols / 8) : n_chunks;
  const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  auto args = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const uint4*)x, (uint32_t*)codes,
                       (uint8_t*)scales, (uint32_t)n_chunks, (uint32_t)(cols / 8), (uint32_t)rows,
                       (uint32_t)scale_rows, (uint32_t)scale_stride, norm, (const float*)nullptr,
                       (const uint16_t*)h, (uint8_t*)mask, pro);
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    args(quantize_lane8_kernel<G, kFmtMx, ROT, kZeroReference, true>);
  } else {
    args(quantize_lane8_kernel<G, kFmtMx, ROT, kZeroSigned, true>);
  }
  return (int)hipGetLastError();
}

static int dispatch_quest(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                          const void* h, void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                          void* mask, int zero_policy, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 32;
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % g != 0 || cols % 32 != 0) return FPQ_E_SHAPE;
  if (scale_rows < rows || scale_stride < cols / 32) return FPQ_E_SHAPE;
  if (rows * cols >= (int64_t)1 << 34 || scale_rows * scale_stride >= (int64_t)1 << 32) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)codes & 3u)) return FPQ_E_ALIGN;
  // big inputs without a clip mask: the streaming kernel, under the conditions of the abs-max dispatch
  const bool stream_ok = !mask && cols % FPQ_EPL == 0 && rows * cols >= (int64_t)1 << 21 &&
                         !((uintptr_t)codes & 15u) && !((uintptr_t)scales & 7u);
#define FPQ_LAUNCH_QUEST(GG, RR)                                                                   \
  return launch_lane8_quest<GG, RR>(x, rows, cols, norm, codes, scales, scale_rows, scale_stride, \
                                    mask, zero_policy, stream, h)
#define FPQ_LAUNCH_QUEST_STREAM(GG, RR)                                                                        \
  {                                                                                                            \
    if (stream_ok)                                                                                             \
      return launch_stream_sized<GG, kFmtMx, RR, true>(x, rows, cols, norm, nullptr, codes, scales,           \
                                                       scale_rows, scale_stride, zero_policy, stream);        \
    FPQ_LAUNCH_QUEST(GG, RR);                                                                                  \
  }
  if (rot_kind == FPQ_ROT_GENERAL) {
    if (!h) return FPQ_E_NULL;
    if ((uintptr_t)h & 1u) return FPQ_E_ALIGN;
  }
  switch (rot_kind) {
    case FPQ_ROT_IDENTITY: FPQ_LAUNCH_QUEST_STREAM(32, FPQ_ROT_IDENTITY);
    case FPQ_ROT_HADAMARD:
      switch (g) {
        case 16: FPQ_LAUNCH_QUEST_STREAM(16, FPQ_ROT_HADAMARD);
        case 32: FPQ_LAUNCH_QUEST_STREAM(32, FPQ_ROT_HADAMARD);
        case 64: FPQ_LAUNCH_QUEST_STREAM(64, FPQ_ROT_HADAMARD);
        case 128: FPQ_LAUNCH_QUEST_STREAM(128, FPQ_ROT_HADAMARD);
      }
      break;
    case FPQ_ROT_GSR:
      switch (g) {
        case 16: FPQ_LAUNCH_QUEST_STREAM(16, FPQ_ROT_GSR);
        case 32: FPQ_LAUNCH_QUEST_STREAM(32, FPQ_ROT_GSR);
        case 64: FPQ_LAUNCH_QUEST_STREAM(64, FPQ_ROT_GSR);
        case 128: FPQ_LAUNCH_QUEST(128, FPQ_ROT_GSR);  // a block spans two lanes of the streaming kernel
      }
      break;
    case FPQ_ROT_GENERAL:
      switch (g) {
        case 16: FPQ_LAUNCH_QUEST(16, FPQ_ROT_GENERAL);
        case 32: FPQ_LAUNCH_QUEST(32, FPQ_ROT_GENERAL);
        case 64: FPQ_LAUNCH_QUEST(64, FPQ_ROT_GENERAL);
        case 128: FPQ_LAUNCH_QUEST(128, FPQ_ROT_GENERAL);
      }
      break;
  }
#undef FPQ_LAUNCH_QUEST_STREAM
#undef FPQ_LAUNCH_QUEST
  return FPQ_E_ROTATION;
}

// fpq_quantize_mx_quest writing the packed operand layout (no clip mask): the streaming kernel, or the
// generic kernel for a few rows, under the conditions of dispatch_packed.
static int dispatch_quest_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                 void* codes, void* scales, int zero_policy, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 32;
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % 256 != 0) return FPQ_E_SHAPE;
  if (rows * cols >= (int64_t)1 << 34) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)codes & 15u) || ((uintptr_t)scales & 3u)) return FPQ_E_ALIGN;
  const bool few = rows <= kPackedFewRows;
#define FPQ_LAUNCH_QUEST_PACKED(GG, RR)                                                                           \
  {                                                                                                               \
    if (few)                                                                                                      \
      return launch_lane8_quest<GG, RR>(x, rows, cols, norm, codes, scales, rows, cols / 32, nullptr,             \
                                        zero_policy, stream, nullptr, true);                                      \
    return launch_stream_packed_sized<GG, RR, kFmtMx, true>(x, rows, cols, norm, codes, scales, zero_policy,      \
                                                            stream, nullptr);                                     \
  }
  if (rot_kind == FPQ_ROT_IDENTITY) {
    FPQ_LAUNCH_QUEST_PACKED(32, FPQ_ROT_IDENTITY);
  } else if (rot_kind == FPQ_ROT_HADAMARD) {
    switch (g) {
      case 16: FPQ_LAUNCH_QUEST_PACKED(16, FPQ_ROT_HADAMARD);
      case 32: FPQ_LAUNCH_QUEST_PACKED(32, FPQ_ROT_HADAMARD);
      case 64: FPQ_LAUNCH_QUEST_PACKED(64, FPQ_ROT_HADAMARD);
      case 128: FPQ_LAUNCH_QUEST_PACKED(128, FPQ_ROT_HADAMARD);
    }
  } else if (rot_kind == FPQ_ROT_GSR) {
    switch (g) {
      case 16: FPQ_LAUNCH_QUEST_PACKED(16, FPQ_ROT_GSR);
      case 32: FPQ_LAUNCH_QUEST_PACKED(32, FPQ_ROT_GSR);
      case 64: FPQ_LAUNCH_QUEST_PACKED(64, FPQ_ROT_GSR);
    }
    return FPQ_E_UNSUPPORTED;  // a 128-wide sequency-ordered block spans two lanes
  } else if (rot_kind == FPQ_ROT_GENERAL) {
    return FPQ_E_UNSUPPORTED;    // arbitrary matrices: quantize row-major, then fpq_pack_mxf4
  }
#undef FPQ_LAUNCH_QUEST_PACKED
  return FPQ_E_ROTATION;
}

template <int FMT>
static int dispatch(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                    const void* h, const float* gsp, void* codes, void* scales,
                    int64_t scale_rows, int64_t scale_stride, int zero_policy, void* stream_) {
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (FMT == kFmtNv && !gsp) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = GROUP;
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % g != 0 || cols % GROUP != 0) return FPQ_E_SHAPE;
  if (scale_rows < rows || scale_stride < cols / GROUP) return FPQ_E_SHAPE;
  if (rows * cols >= (int64_t)1 << 34 || scale_rows * scale_stride >= (int64_t)1 << 32) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)codes & 3u)) return FPQ_E_ALIGN;

  // big inputs with cols % FPQ_EPL == 0 and aligned outputs: the streaming kernel; else the generic one
  const bool stream_ok = cols % FPQ_EPL == 0 && rows * cols >= (int64_t)1 << 21 &&
                         !((uintptr_t)codes & 15u) && !((uintptr_t)scales & 7u);
#define FPQ_LAUNCH(GG, RR)                                                                       \
  return stream_ok ? launch_stream_sized<GG, FMT, RR>(x, rows, cols, norm, gsp, codes, scales,   \
                                                  scale_rows, scale_stride, zero_policy, stream) \
                   : launch_lane8<GG, FMT, RR>(x, rows, cols, norm, gsp, codes, scales,          \
                                               scale_rows, scale_stride, zero_policy, stream)
#define FPQ_LAUNCH_GENERIC(GG, RR)                                                               \
  return launch_lane8<GG, FMT, RR>(x, rows, cols, norm, gsp, codes, scales, scale_rows,         \
                                   scale_stride, zero_policy, stream, h)
  if (rot_kind == FPQ_ROT_IDENTITY) {
    FPQ_LAUNCH(GROUP, FPQ_ROT_IDENTITY);
  } else if (rot_kind == FPQ_ROT_HADAMARD) {
    switch (g) {
      case 16: FPQ_LAUNCH(16, FPQ_ROT_HADAMARD);
      case 32: FPQ_LAUNCH(32, FPQ_ROT_HADAMARD);
      case 64: FPQ_LAUNCH(64, FPQ_ROT_HADAMARD);
      case 128: FPQ_LAUNCH(128, FPQ_ROT_HADAMARD);
    }
  } else if (rot_kind == FPQ_ROT_GSR) {
    switch (g) {
      case 16: FPQ_LAUNCH(16, FPQ_ROT_GSR);
      case 32: FPQ_LAUNCH(32, FPQ_ROT_GSR);
      case 64: FPQ_LAUNCH(64, FPQ_ROT_GSR);
      case 128: FPQ_LAUNCH_GENERIC(128, FPQ_ROT_GSR);  // a block spans two lanes of the streaming kernel
    }
  } else if (rot_kind == FPQ_ROT_GENERAL) {
    if (!h) return FPQ_E_NULL;
    if ((uintptr_t)h & 1u) return FPQ_E_ALIGN;
    switch (g) {
      case 16: FPQ_LAUNCH_GENERIC(16, FPQ_ROT_GENERAL);
      case 32: FPQ_LAUNCH_GENERIC(32, FPQ_ROT_GENERAL);
      case 64: FPQ_LAUNCH_GENERIC(64, FPQ_ROT_GENERAL);
      case 128: FPQ_LAUNCH_GENERIC(128, FPQ_ROT_GENERAL);
    }
  }
#undef FPQ_LAUNCH_GENERIC
#undef FPQ_LAUNCH
  return FPQ_E_ROTATION;
}

// ------------------------------------------------------------------------------------------
// Quantizers with a prologue (generic kernel).
template <int G, int FMT, int ROT, int PRO>
static int launch_lane8_prologue(const void* x, int64_t rows, int64_t cols, float norm, const float* gsp,
                                 void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                                 int zero_policy, hipStream_t stream, const Prologue& pro) {
  const int64_t n_chunks = rows * cols / 8;
  const int64_t threads = pro.packed_rows ? (int64_t)pro.packed_rows * (cols / 8) : n_chunks;
  const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  auto args = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const uint4*)x, (uint32_t*)codes,
                       (uint8_t*)scales, (uint32_t)n_chunks, (uint32_t)(cols / 8), (uint32_t)rows,
                       (uint32_t)scale_rows, (uint32_t)scale_stride, norm, gsp, (const uint16_t*)nullptr,
                       (uint8_t*)nullptr, pro);
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroReference, false, PRO>);
  } else {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroSigned, false, PRO>);
  }
  return (int)hipGetLastError();
}

// Fills g_silu_table once per device.  The first call on a device builds the table on the caller's
// stream and waits for it, so that calls on other streams can rely on it afterwards; while a stream
// is being captured the build is recorded into the capture instead and nothing is remembered.
int ensure_silu_table(hipStream_t stream) {   // also called by fpq_prepare_device (fpq_capi.hip)
  static std::atomic<uint64_t> built{0};  // bit d: device d holds the table (devices >= 64 rebuild every call)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
  if (bit && (built.load(std::memory_order_acquire) & bit)) return 0;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  e = hipStreamIsCapturing(stream, &cap);
  if (e != hipSuccess) return (int)e;
  hipLaunchKernelGGL(silu_table_kernel, dim3(256), dim3(256), 0, stream);
  e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (cap != hipStreamCaptureStatusNone) return 0;
  e = hipStreamSynchronize(stream);
  if (e != hipSuccess) return (int)e;
  if (bit) built.fetch_or(bit, std::memory_order_release);
  return 0;
}

// x: the prologue's first input with row stride ld_first elements (kProSiluMul: `second` with
// ld_second); Hadamard rotations of 16..128 and the identity only.
template <int FMT, int PRO>
static int dispatch_prologue(const void* x, int64_t ld_first, const void* second, int64_t ld_second,
                             const float* row_scale, const void* col_scale, void* out, int64_t rows,
                             int64_t cols, int rot_kind, int g, float norm, const float* gsp, void* codes,
                             void* scales, int64_t scale_rows, int64_t scale_stride, int zero_policy,
                             void* stream_) {
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (PRO == kProRmsNorm && (!row_scale || !col_scale)) return FPQ_E_NULL;
  if (PRO == kProSiluMul && !second) return FPQ_E_NULL;
  if (FMT == kFmtNv && !gsp) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = GROUP;
  if (rot_kind != FPQ_ROT_IDENTITY && rot_kind != FPQ_ROT_HADAMARD) {
    return (rot_kind == FPQ_ROT_GSR || rot_kind == FPQ_ROT_GENERAL) ? FPQ_E_UNSUPPORTED : FPQ_E_ROTATION;
  }
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % g != 0 || cols % GROUP != 0) return FPQ_E_SHAPE;
  if (ld_first < cols || ld_first % 8 != 0) return FPQ_E_SHAPE;
  if (PRO == kProSiluMul && (ld_second < cols || ld_second % 8 != 0)) return FPQ_E_SHAPE;
  if (scale_rows < rows || scale_stride < cols / GROUP) return FPQ_E_SHAPE;
  if (rows * ld_first >= (int64_t)1 << 34 || rows * ld_second >= (int64_t)1 << 34 ||
      scale_rows * scale_stride >= (int64_t)1 << 32) {
    return FPQ_E_SHAPE;
  }
  if (((uintptr_t)x & 15u) || ((uintptr_t)second & 15u) || ((uintptr_t)col_scale & 15u) ||
      ((uintptr_t)out & 15u) || ((uintptr_t)row_scale & 3u) || ((uintptr_t)codes & 3u)) {
    return FPQ_E_ALIGN;
  }
  if (PRO == kProSiluMul) {
    if (const int st = ensure_silu_table(stream)) return st;
  }
  Prologue pro{};
  pro.row_scale = row_scale;
  pro.col_scale = (const uint4*)col_scale;
  pro.second = (const uint4*)second;
  pro.out = (uint4*)out;
  pro.chunks_per_row = (uint32_t)(cols / 8);
  pro.ld_first = (uint32_t)(ld_first / 8);
  pro.ld_second = (uint32_t)(ld_second / 8);
#define FPQ_LAUNCH_PRO(GG, RR)                                                                            \
  return launch_lane8_prologue<GG, FMT, RR, PRO>(x, rows, cols, norm, gsp, codes, scales, scale_rows,    \
                                                 scale_stride, zero_policy, stream, pro)
  if (rot_kind == FPQ_ROT_IDENTITY) FPQ_LAUNCH_PRO(GROUP, FPQ_ROT_IDENTITY);
  switch (g) {
    case 16: FPQ_LAUNCH_PRO(16, FPQ_ROT_HADAMARD);
    case 32: FPQ_LAUNCH_PRO(32, FPQ_ROT_HADAMARD);
    case 64: FPQ_LAUNCH_PRO(64, FPQ_ROT_HADAMARD);
    case 128: FPQ_LAUNCH_PRO(128, FPQ_ROT_HADAMARD);
  }
#undef FPQ_LAUNCH_PRO
  return FPQ_E_ROTATION;
}

// The same with the packed operand layout as output (streaming kernel; cols % 256 == 0).
template <int PRO, int FMT = kFmtMx>
static int dispatch_prologue_packed(const void* x, int64_t ld_first, const void* second, int64_t ld_second,
                                    const float* row_scale, const void* col_scale, void* out, int64_t rows,
                                    int64_t cols, int rot_kind, int g, float norm, void* codes, void* scales,
                                    int zero_policy, void* stream_, const float* gsp = nullptr) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !codes || !scales) return FPQ_E_NULL;
  if (FMT == kFmtNv && !gsp) return FPQ_E_NULL;
  if (PRO == kProRmsNorm && (!row_scale || !col_scale)) return FPQ_E_NULL;
  if (PRO == kProSiluMul && !second) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 32;
  if (rot_kind != FPQ_ROT_IDENTITY && rot_kind != FPQ_ROT_HADAMARD) {
    return (rot_kind == FPQ_ROT_GSR || rot_kind == FPQ_ROT_GENERAL) ? FPQ_E_UNSUPPORTED : FPQ_E_ROTATION;
  }
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % 256 != 0) return FPQ_E_SHAPE;
  if (ld_first < cols || ld_first % 8 != 0) return FPQ_E_SHAPE;
  if (PRO == kProSiluMul && (ld_second < cols || ld_second % 8 != 0)) return FPQ_E_SHAPE;
  // 32-bit byte offsets inside a row tile, 32-bit chunk counts
  if (rows * cols >= (int64_t)1 << 34 || ld_first >= (int64_t)1 << 24 || ld_second >= (int64_t)1 << 24) {
    return FPQ_E_SHAPE;
  }
  if (((uintptr_t)x & 15u) || ((uintptr_t)second & 15u) || ((uintptr_t)col_scale & 15u) ||
      ((uintptr_t)out & 15u) || ((uintptr_t)row_scale & 3u) || ((uintptr_t)codes & 15u) ||
      ((uintptr_t)scales & (FMT == kFmtNv ? 7u : 3u)) || ((uintptr_t)gsp & 3u)) {
    return FPQ_E_ALIGN;
  }
  if (PRO == kProSiluMul) {
    if (const int st = ensure_silu_table(stream)) return st;
  }
  Prologue pro{};
  pro.row_scale = row_scale;
  pro.col_scale = (const uint4*)col_scale;
  pro.second = (const uint4*)second;
  pro.out = (uint4*)out;
  pro.chunks_per_row = (uint32_t)(cols / 8);
  pro.ld_first = (uint32_t)(ld_first / 8);
  pro.ld_second = (uint32_t)(ld_second / 8);
  pro.packed_rows = 0u;
  const bool few = rows <= kPackedFewRows;
  if (few) pro.packed_rows = (uint32_t)((rows + 31) / 32 * 32);
#define FPQ_LAUNCH_PRO_PACKED(GG, RR)                                                                          \
  {                                                                                                            \
    if (few)                                                                                                   \
      return launch_lane8_prologue<GG, FMT, RR, PRO>(x, rows, cols, norm, gsp, codes, scales, rows,            \
                                                     cols / (FMT == kFmtNv ? 16 : 32), zero_policy, stream, pro); \
    return launch_stream_packed<GG, RR, PRO, FMT>(x, rows, cols, norm, codes, scales, zero_policy, stream,    \
                                                  pro, gsp);                                                  \
  }
  if (rot_kind == FPQ_ROT_IDENTITY) FPQ_LAUNCH_PRO_PACKED(32, FPQ_ROT_IDENTITY);
  switch (g) {
    case 16: FPQ_LAUNCH_PRO_PACKED(16, FPQ_ROT_HADAMARD);
    case 32: FPQ_LAUNCH_PRO_PACKED(32, FPQ_ROT_HADAMARD);
    case 64: FPQ_LAUNCH_PRO_PACKED(64, FPQ_ROT_HADAMARD);
    case 128: FPQ_LAUNCH_PRO_PACKED(128, FPQ_ROT_HADAMARD);
  }
#undef FPQ_LAUNCH_PRO_PACKED
  return FPQ_E_ROTATION;
}

// 1 / sqrt(mean(x^2) + eps) of every row, one wave per row.  Fixed summation order: squares of 8
// consecutive elements left to right; lane l accumulates the octets l, l + 64, ... in that order;
// the 64 lane sums combine by the butterfly a += a[lane ^ m], m = 1, 2, ..., 32.
__global__ __launch_bounds__(256) void row_inv_rms_kernel(const uint4* __restrict__ x, uint32_t rows,
                                                          uint32_t chunks_per_row, uint32_t ld, float cols_f,
                                                          float eps, float* __restrict__ out) {
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
  if (row >= rows) return;
  const uint4* src = x + (size_t)row * ld;
  float a = 0.0f;
  for (uint32_t c = lane; c < chunks_per_row; c += 64u) {
    float p[8];
    unpack8(src[c], p);
    float s = p[0] * p[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) s = s + p[i] * p[i];
    a = a + s;
  }
#pragma unroll
  for (int lm = 1; lm < 64; lm *= 2) a = a + __shfl_xor(a, lm, 64);
  if (lane == 0u) out[row] = 1.0f / __builtin_sqrtf(a / cols_f + eps);
}

// RMSNorm + rotate + quantize of a few rows in ONE launch (decode): a workgroup per row computes the
// row's 1 / rms exactly as row_inv_rms_kernel does (the octet sums go through LDS, then one wave adds
// them in that kernel's order) and quantizes the row with the generic kernel's arithmetic into the
// packed operand layout.  Workgroups past `rows` (the padding of the last 32-row tile) write zeros.
constexpr uint32_t kRowsKernelMaxChunks = 2048;   // cols <= 16384
template <int G, int FMT, int ROT, int ZERO>
__global__ __launch_bounds__(1024) void rmsnorm_rows_quantize_kernel(const uint4* __restrict__ x,
                                                                    uint32_t* __restrict__ codes,
                                                                    uint8_t* __restrict__ scales, uint32_t rows,
                                                                    float norm, float cols_f, float eps,
                                                                    float* __restrict__ inv_rms_out,
                                                                    const float* __restrict__ global_scale,
                                                                    Prologue pro) {
  __shared__ float oct[kRowsKernelMaxChunks];
  __shared__ float inv_shared;
  const uint32_t row = blockIdx.x, cpr = pro.chunks_per_row, lane = threadIdx.x & 63u, nthr = blockDim.x;
  const bool real = row < rows;
  if (real) {
    const uint4* src = x + (size_t)row * pro.ld_first;
    for (uint32_t c = threadIdx.x; c < cpr; c += nthr) {
      float p[8];
      unpack8(src[c], p);
      float s = p[0] * p[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) s = s + p[i] * p[i];
      oct[c] = s;
    }
  }
  __syncthreads();
  if (real && threadIdx.x < 64u) {
    float a = 0.0f;
    for (uint32_t c = lane; c < cpr; c += 64u) a = a + oct[c];
#pragma unroll
    for (int lm = 1; lm < 64; lm *= 2) a = a + __shfl_xor(a, lm, 64);
    if (lane == 0u) {
      const float inv = 1.0f / __builtin_sqrtf(a / cols_f + eps);
      inv_shared = inv;
      if (inv_rms_out) inv_rms_out[row] = inv;
    }
  }
  __syncthreads();
  const float rs = real ? inv_shared : 0.0f;
  float gs = 1.0f, rg = 1.0f;
  if (FMT == kFmtNv) {
    gs = *global_scale;
    rg = gs == 0.0f ? 0.0f : 1.0f / gs;
  }
  for (uint32_t c0 = 0; c0 < cpr; c0 += nthr) {   // the same trip count for every thread: lanes exchange values
    const uint32_t cc = c0 + threadIdx.x;
    const bool in = cc < cpr;
    // a chunk index past the packed output makes the generic kernel skip the store
    const uint32_t chunk = in ? row * cpr + cc : 0xffffffffu;
    lane8_process<G, FMT, ROT, ZERO, false, kProRmsNorm>(x, codes, scales, chunk, real && in, lane, cpr, 0u, norm, gs,
                                                         rg, nullptr, nullptr, nullptr, pro, rs);
  }
}

// ------------------------------------------------------------------------------------------
// max |rotate(x)| over a whole tensor, folded into *amax with an atomic maximum on the bit
// pattern (non-negative floats order like unsigned integers).  The rotation is the quantizers'
// own, so the value is the one their group maxima are taken from.
template <int G, int ROT>
__global__ __launch_bounds__(256) void rotated_absmax_kernel(const uint4* __restrict__ x, uint32_t n_chunks,
                                                             float norm, const uint16_t* __restrict__ h,
                                                             uint32_t* __restrict__ amax) {
  constexpr bool kStage = ROT == FPQ_ROT_GSR || ROT == FPQ_ROT_GENERAL;
  __shared__ float stage[kStage ? 4 : 1][kStage ? 512 : 1];
  __shared__ __attribute__((aligned(16))) uint16_t hmat[ROT == FPQ_ROT_GENERAL ? G * G : 8];
  if (ROT == FPQ_ROT_GENERAL) {
    for (int i = threadIdx.x; i < G * G; i += 256) hmat[i] = h[i];
    __syncthreads();
  }
  float a = 0.0f;
  for (uint32_t base = blockIdx.x * 256u; base < n_chunks; base += gridDim.x * 256u) {
    const uint32_t chunk = base + threadIdx.x;
    float p[8];
    lane8_load_rotate<G, ROT>(x, chunk, chunk < n_chunks, threadIdx.x & 63u, norm,
                              stage[kStage ? (threadIdx.x >> 6) : 0], hmat, p);
#pragma unroll
    for (int i = 0; i < 8; ++i) a = __builtin_fmaxf(a, __builtin_fabsf(p[i]));
  }
#pragma unroll
  for (int lm = 1; lm < 64; lm *= 2) a = __builtin_fmaxf(a, __shfl_xor(a, lm, 64));
  if ((threadIdx.x & 63u) == 0u) atomicMax(amax, __float_as_uint(a));
}

template <int G, int ROT>
static int launch_absmax(const void* x, int64_t rows, int64_t cols, float norm, const void* h, float* amax,
                         hipStream_t stream) {
  const int64_t n_chunks = rows * cols / 8;
  const int64_t blocks = (n_chunks + 255) / 256;
  hipLaunchKernelGGL((rotated_absmax_kernel<G, ROT>), dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256),
                     0, stream, (const uint4*)x, (uint32_t)n_chunks, norm, (const uint16_t*)h, (uint32_t*)amax);
  return (int)hipGetLastError();
}

static int dispatch_absmax(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                           const void* h, float* amax, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (!amax) return FPQ_E_NULL;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x) return FPQ_E_NULL;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 16;
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % g != 0) return FPQ_E_SHAPE;
  if (rows * cols >= (int64_t)1 << 34) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)amax & 3u)) return FPQ_E_ALIGN;
  if (rot_kind == FPQ_ROT_GENERAL) {
    if (!h) return FPQ_E_NULL;
    if ((uintptr_t)h & 1u) return FPQ_E_ALIGN;
  }
#define FPQ_LAUNCH_ABSMAX(GG, RR) return launch_absmax<GG, RR>(x, rows, cols, norm, h, amax, stream)
#define FPQ_ABSMAX_BY_G(RR)                       \
  switch (g) {                                    \
    case 16: FPQ_LAUNCH_ABSMAX(16, RR);           \
    case 32: FPQ_LAUNCH_ABSMAX(32, RR);           \
    case 64: FPQ_LAUNCH_ABSMAX(64, RR);           \
    case 128: FPQ_LAUNCH_ABSMAX(128, RR);         \
  }                                               \
  break
  switch (rot_kind) {
    case FPQ_ROT_IDENTITY: FPQ_LAUNCH_ABSMAX(16, FPQ_ROT_IDENTITY);
    case FPQ_ROT_HADAMARD: FPQ_ABSMAX_BY_G(FPQ_ROT_HADAMARD);
    case FPQ_ROT_GSR: FPQ_ABSMAX_BY_G(FPQ_ROT_GSR);
    case FPQ_ROT_GENERAL: FPQ_ABSMAX_BY_G(FPQ_ROT_GENERAL);
  }
#undef FPQ_ABSMAX_BY_G
#undef FPQ_LAUNCH_ABSMAX
  return FPQ_E_ROTATION;
}

// ------------------------------------------------------------------------------------------
template <int ZERO>
__global__ void e2m1_test_kernel(const float* in, uint8_t* out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (uint8_t)e2m1_code<ZERO>(in[i]);
}

}  // namespace fpq

extern "C" int fpq_quantize_mx(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                               float norm, const void* h, void* codes, void* scales,
                               int64_t scale_rows, int64_t scale_stride, int zero_policy,
                               void* stream) {
  return fpq::dispatch<fpq::kFmtMx>(x, rows, cols, rot_kind, g, norm, h, nullptr, codes, scales,
                                    scale_rows, scale_stride, zero_policy, stream);
}

extern "C" int fpq_quantize_mx_quest_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                                            float norm, void* packed_codes, void* packed_scales, int zero_policy,
                                            void* stream) {
  return fpq::dispatch_quest_packed(x, rows, cols, rot_kind, g, norm, packed_codes, packed_scales, zero_policy,
                                    stream);
}

extern "C" int fpq_quantize_mx_quest(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                                     float norm, const void* h, void* codes, void* scales,
                                     int64_t scale_rows, int64_t scale_stride, void* mask, int zero_policy,
                                     void* stream) {
  return fpq::dispatch_quest(x, rows, cols, rot_kind, g, norm, h, codes, scales, scale_rows, scale_stride,
                             mask, zero_policy, stream);
}

extern "C" int fpq_quantize_mx_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                                      float norm, void* packed_codes, void* packed_scales,
                                      int zero_policy, void* stream) {
  return fpq::dispatch_packed<fpq::kFmtMx>(x, rows, cols, rot_kind, g, norm, nullptr, packed_codes, packed_scales,
                                           zero_policy, stream);
}

extern "C" int fpq_quantize_nv_packed(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                                      float norm, const float* global_scale, void* packed_codes,
                                      void* packed_scales, int zero_policy, void* stream) {
  return fpq::dispatch_packed<fpq::kFmtNv>(x, rows, cols, rot_kind, g, norm, global_scale, packed_codes,
                                           packed_scales, zero_policy, stream);
}

extern "C" int fpq_quantize_nv(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                               float norm, const void* h, const float* global_scale, void* codes,
                               void* scales, int64_t scale_rows, int64_t scale_stride,
                               int zero_policy, void* stream) {
  return fpq::dispatch<fpq::kFmtNv>(x, rows, cols, rot_kind, g, norm, h, global_scale, codes,
                                    scales, scale_rows, scale_stride, zero_policy, stream);
}

extern "C" int fpq_row_inv_rms(const void* x, int64_t ld, int64_t rows, int64_t cols, float eps, float* inv_rms,
                               void* stream) {
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0) return FPQ_OK;
  if (!x || !inv_rms) return FPQ_E_NULL;
  if (cols == 0 || cols % 8 != 0 || ld < cols || ld % 8 != 0 || rows * ld >= (int64_t)1 << 34) return FPQ_E_SHAPE;
  if (((uintptr_t)x & 15u) || ((uintptr_t)inv_rms & 3u)) return FPQ_E_ALIGN;
  hipLaunchKernelGGL(fpq::row_inv_rms_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)x, (uint32_t)rows, (uint32_t)(cols / 8), (uint32_t)(ld / 8), (float)cols, eps,
                     inv_rms);
  return (int)hipGetLastError();
}

extern "C" int fpq_rmsnorm_quantize_mx(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                       int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                       void* normed, void* codes, void* scales, int64_t scale_rows,
                                       int64_t scale_stride, int zero_policy, void* stream) {
  return fpq::dispatch_prologue<fpq::kFmtMx, fpq::kProRmsNorm>(x, ld, nullptr, 0, inv_rms, weight, normed, rows,
                                                               cols, rot_kind, g, norm, nullptr, codes, scales,
                                                               scale_rows, scale_stride, zero_policy, stream);
}

extern "C" int fpq_rmsnorm_quantize_nv(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                       int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                       const float* global_scale, void* normed, void* codes, void* scales,
                                       int64_t scale_rows, int64_t scale_stride, int zero_policy, void* stream) {
  return fpq::dispatch_prologue<fpq::kFmtNv, fpq::kProRmsNorm>(x, ld, nullptr, 0, inv_rms, weight, normed, rows,
                                                               cols, rot_kind, g, norm, global_scale, codes,
                                                               scales, scale_rows, scale_stride, zero_policy,
                                                               stream);
}

extern "C" int fpq_silu_mul_quantize_mx(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                        int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                        void* product, void* codes, void* scales, int64_t scale_rows,
                                        int64_t scale_stride, int zero_policy, void* stream) {
  return fpq::dispatch_prologue<fpq::kFmtMx, fpq::kProSiluMul>(gate, ld_gate, up, ld_up, nullptr, nullptr, product,
                                                               rows, cols, rot_kind, g, norm, nullptr, codes,
                                                               scales, scale_rows, scale_stride, zero_policy,
                                                               stream);
}

extern "C" int fpq_silu_mul_quantize_nv(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                        int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                        const float* global_scale, void* product, void* codes, void* scales,
                                        int64_t scale_rows, int64_t scale_stride, int zero_policy,
                                        void* stream) {
  return fpq::dispatch_prologue<fpq::kFmtNv, fpq::kProSiluMul>(gate, ld_gate, up, ld_up, nullptr, nullptr, product,
                                                               rows, cols, rot_kind, g, norm, global_scale, codes,
                                                               scales, scale_rows, scale_stride, zero_policy,
                                                               stream);
}

extern "C" int fpq_rmsnorm_quantize_mx_packed(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                              int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                              void* normed, void* packed_codes, void* packed_scales,
                                              int zero_policy, void* stream) {
  return fpq::dispatch_prologue_packed<fpq::kProRmsNorm>(x, ld, nullptr, 0, inv_rms, weight, normed, rows, cols,
                                                         rot_kind, g, norm, packed_codes, packed_scales,
                                                         zero_policy, stream);
}

namespace fpq {
template <int FMT>
static int dispatch_rmsnorm_rows(const void* x, int64_t ld, const void* weight, int64_t rows, int64_t cols, float eps,
                                 int rot_kind, int g, float norm, float* inv_rms, void* normed, void* codes,
                                 void* scales, int zero_policy, void* stream_, const float* gsp = nullptr) {
  hipStream_t stream = (hipStream_t)stream_;
  if (rows < 0 || cols < 0) return FPQ_E_SHAPE;
  if (rows == 0 || cols == 0) return FPQ_OK;
  if (!x || !weight || !codes || !scales) return FPQ_E_NULL;
  if (FMT == kFmtNv && !gsp) return FPQ_E_NULL;
  if (zero_policy != FPQ_ZERO_REFERENCE && zero_policy != FPQ_ZERO_SIGNED) return FPQ_E_POLICY;
  if (rot_kind == FPQ_ROT_IDENTITY) g = 32;
  if (rot_kind != FPQ_ROT_IDENTITY && rot_kind != FPQ_ROT_HADAMARD) {
    return (rot_kind == FPQ_ROT_GSR || rot_kind == FPQ_ROT_GENERAL) ? FPQ_E_UNSUPPORTED : FPQ_E_ROTATION;
  }
  if (g != 16 && g != 32 && g != 64 && g != 128) return FPQ_E_ROTATION;
  if (cols % 256 != 0 || ld < cols || ld % 8 != 0 || ld >= (int64_t)1 << 24) return FPQ_E_SHAPE;
  if (rows > kPackedFewRows || cols / 8 > (int64_t)kRowsKernelMaxChunks) return FPQ_E_LIMIT;
  if (((uintptr_t)x & 15u) || ((uintptr_t)weight & 15u) || ((uintptr_t)normed & 15u) || ((uintptr_t)inv_rms & 3u) ||
      ((uintptr_t)codes & 15u) || ((uintptr_t)scales & (FMT == kFmtNv ? 7u : 3u)) || ((uintptr_t)gsp & 3u)) {
    return FPQ_E_ALIGN;
  }
  Prologue pro{};
  pro.col_scale = (const uint4*)weight;
  pro.out = (uint4*)normed;
  pro.chunks_per_row = (uint32_t)(cols / 8);
  pro.ld_first = (uint32_t)(ld / 8);
  pro.packed_rows = (uint32_t)((rows + 31) / 32 * 32);
  // a row is one workgroup's work: wider rows get more waves (the row statistic does not depend on the count)
  const dim3 grid(pro.packed_rows), block(pro.chunks_per_row >= 1024u ? 1024 : pro.chunks_per_row >= 512u ? 512 : 256);
#define FPQ_LAUNCH_ROWS(GG, RR)                                                                                 \
  {                                                                                                             \
    if (zero_policy == FPQ_ZERO_REFERENCE)                                                                      \
      hipLaunchKernelGGL((rmsnorm_rows_quantize_kernel<GG, FMT, RR, kZeroReference>), grid, block, 0, stream,   \
                         (const uint4*)x, (uint32_t*)codes, (uint8_t*)scales, (uint32_t)rows, norm, (float)cols, \
                         eps, inv_rms, gsp, pro);                                                               \
    else                                                                                                        \
      hipLaunchKernelGGL((rmsnorm_rows_quantize_kernel<GG, FMT, RR, kZeroSigned>), grid, block, 0, stream,      \
                         (const uint4*)x, (uint32_t*)codes, (uint8_t*)scales, (uint32_t)rows, norm, (float)cols, \
                         eps, inv_rms, gsp, pro);                                                               \
    return (int)hipGetLastError();                                                                              \
  }
  if (rot_kind == FPQ_ROT_IDENTITY) FPQ_LAUNCH_ROWS(32, FPQ_ROT_IDENTITY);
  switch (g) {
    case 16: FPQ_LAUNCH_ROWS(16, FPQ_ROT_HADAMARD);
    case 32: FPQ_LAUNCH_ROWS(32, FPQ_ROT_HADAMARD);
    case 64: FPQ_LAUNCH_ROWS(64, FPQ_ROT_HADAMARD);
    case 128: FPQ_LAUNCH_ROWS(128, FPQ_ROT_HADAMARD);
  }
#undef FPQ_LAUNCH_ROWS
  return FPQ_E_ROTATION;
}
}  // namespace fpq

extern "C" int64_t fpq_rmsnorm_rows_max_rows(void) { return fpq::kPackedFewRows; }

extern "C" int fpq_rmsnorm_rows_quantize_mx_packed(const void* x, int64_t ld, const void* weight, int64_t rows,
                                                   int64_t cols, float eps, int rot_kind, int g, float norm,
                                                   float* inv_rms, void* normed, void* packed_codes,
                                                   void* packed_scales, int zero_policy, void* stream) {
  return fpq::dispatch_rmsnorm_rows<fpq::kFmtMx>(x, ld, weight, rows, cols, eps, rot_kind, g, norm, inv_rms, normed,
                                                 packed_codes, packed_scales, zero_policy, stream);
}

extern "C" int fpq_rmsnorm_rows_quantize_nv_packed(const void* x, int64_t ld, const void* weight, int64_t rows,
                                                   int64_t cols, float eps, int rot_kind, int g, float norm,
                                                   const float* global_scale, float* inv_rms, void* normed,
                                                   void* packed_codes, void* packed_scales, int zero_policy,
                                                   void* stream) {
  return fpq::dispatch_rmsnorm_rows<fpq::kFmtNv>(x, ld, weight, rows, cols, eps, rot_kind, g, norm, inv_rms, normed,
                                                 packed_codes, packed_scales, zero_policy, stream, global_scale);
}

extern "C" int fpq_rmsnorm_quantize_nv_packed(const void* x, int64_t ld, const float* inv_rms, const void* weight,
                                              int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                              const float* global_scale, void* normed, void* packed_codes,
                                              void* packed_scales, int zero_policy, void* stream) {
  return fpq::dispatch_prologue_packed<fpq::kProRmsNorm, fpq::kFmtNv>(x, ld, nullptr, 0, inv_rms, weight, normed, rows,
                                                                      cols, rot_kind, g, norm, packed_codes,
                                                                      packed_scales, zero_policy, stream, global_scale);
}

extern "C" int fpq_silu_mul_quantize_nv_packed(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                               int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                               const float* global_scale, void* product, void* packed_codes,
                                               void* packed_scales, int zero_policy, void* stream) {
  return fpq::dispatch_prologue_packed<fpq::kProSiluMul, fpq::kFmtNv>(gate, ld_gate, up, ld_up, nullptr, nullptr,
                                                                      product, rows, cols, rot_kind, g, norm,
                                                                      packed_codes, packed_scales, zero_policy,
                                                                      stream, global_scale);
}

extern "C" int fpq_silu_mul_quantize_mx_packed(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                               int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                               void* product, void* packed_codes, void* packed_scales,
                                               int zero_policy, void* stream) {
  return fpq::dispatch_prologue_packed<fpq::kProSiluMul>(gate, ld_gate, up, ld_up, nullptr, nullptr, product, rows,
                                                         cols, rot_kind, g, norm, packed_codes, packed_scales,
                                                         zero_policy, stream);
}

extern "C" int fpq_rotated_absmax(const void* x, int64_t rows, int64_t cols, int rot_kind, int g, float norm,
                                  const void* h, float* amax, void* stream) {
  return fpq::dispatch_absmax(x, rows, cols, rot_kind, g, norm, h, amax, stream);
}

extern "C" int fpq_test_e2m1(const float* in, uint8_t* out, int64_t n, int zero_policy,
                             void* stream) {
  if (!in || !out) return FPQ_E_NULL;
  if (n <= 0) return n == 0 ? FPQ_OK : FPQ_E_SHAPE;
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    hipLaunchKernelGGL(fpq::e2m1_test_kernel<fpq::kZeroReference>, grid, block, 0,
                       (hipStream_t)stream, in, out, n);
  } else if (zero_policy == FPQ_ZERO_SIGNED) {
    hipLaunchKernelGGL(fpq::e2m1_test_kernel<fpq::kZeroSigned>, grid, block, 0,
                       (hipStream_t)stream, in, out, n);
  } else {
    return FPQ_E_POLICY;
  }
  return (int)hipGetLastError();
}
