// Fused rotate + group-scale + E2M1 pack kernels (MXFP4 / NVFP4) for gfx950.
//
// The rotation is a block Walsh-Hadamard transform evaluated as fp32 radix-2 butterflies with
// strides 1, 2, ..., g/2 on the exact products x[i] * norm, i.e. x @ H for the +-norm Sylvester
// matrix the reference builds (inference_lib/src/fp_quant/module/linear.py:24-30) with a fixed
// summation tree, so that results can be reproduced bit for bit on a CPU.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fpq.h"
#include "fpq_device.h"

namespace fpq {

constexpr int kFmtMx = 0;
constexpr int kFmtNv = 1;

// -------------------------------------------------------------------------------------------
// Generic kernel: one lane owns 8 consecutive elements (one 16-byte load, 4 bytes of codes).
// A rotation block of G elements spans G/8 neighbouring lanes; the butterflies with stride
// >= 8 exchange registers between lanes.  Works for any cols % max(G, GROUP) == 0.
template <int G, int FMT, int ROT, int ZERO>
__global__ __launch_bounds__(256) void quantize_lane8_kernel(
    const uint4* __restrict__ x, uint32_t* __restrict__ codes, uint8_t* __restrict__ scales,
    uint32_t n_chunks, uint32_t chunks_per_row, uint32_t rows, uint32_t scale_rows,
    uint32_t scale_stride, float norm, const float* __restrict__ global_scale) {
  constexpr int GROUP = FMT == kFmtMx ? 32 : 16;
  const uint32_t chunk = blockIdx.x * 256u + threadIdx.x;
  const uint32_t lane = threadIdx.x & 63u;
  const bool active = chunk < n_chunks;

  uint4 raw = make_uint4(0u, 0u, 0u, 0u);
  if (active) raw = x[chunk];

  float p[8];
  p[0] = bf16_lo(raw.x); p[1] = bf16_hi(raw.x);
  p[2] = bf16_lo(raw.y); p[3] = bf16_hi(raw.y);
  p[4] = bf16_lo(raw.z); p[5] = bf16_hi(raw.z);
  p[6] = bf16_lo(raw.w); p[7] = bf16_hi(raw.w);

  if (ROT == FPQ_ROT_HADAMARD) {
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

  float a = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) a = __builtin_fmaxf(a, __builtin_fabsf(p[i]));
#pragma unroll
  for (int lm = 1; lm < GROUP / 8; lm *= 2) a = __builtin_fmaxf(a, __shfl_xor(a, lm, 64));

  GroupScale gs;
  if (FMT == kFmtMx) {
    gs = mx_group_scale(a);
  } else {
    const float g = *global_scale;
    const float rg = g == 0.0f ? 0.0f : 1.0f / g;
    gs = nv_group_scale(a, g, rg);
  }

  uint32_t packed = 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float v = scale_element(p[i], gs);
    if (FMT == kFmtNv) v = gs.zero ? 0.0f : v;
    packed |= e2m1_code<ZERO>(v) << (4 * i);
  }

  if (active) {
    codes[chunk] = packed;
    if ((chunk & (GROUP / 8 - 1)) == 0u) {
      const uint32_t row = chunk / chunks_per_row;
      const uint32_t col = (chunk - row * chunks_per_row) / (GROUP / 8);
      scales[(size_t)row * scale_stride + col] = (uint8_t)gs.byte;
    }
  }

  // zero-fill the padded part of the scale tensor (rows >= rows, columns >= cols / GROUP)
  const uint32_t valid_cols = chunks_per_row / (GROUP / 8);
  if (scale_rows != rows || scale_stride != valid_cols) {
    const uint32_t total = scale_rows * scale_stride;
    for (uint32_t i = chunk; i < total; i += gridDim.x * 256u) {
      const uint32_t r = i / scale_stride;
      const uint32_t c = i - r * scale_stride;
      if (r >= rows || c >= valid_cols) scales[i] = 0;
    }
  }
}

template <int G, int FMT, int ROT>
static int launch_lane8(const void* x, int64_t rows, int64_t cols, float norm, const float* gsp,
                        void* codes, void* scales, int64_t scale_rows, int64_t scale_stride,
                        int zero_policy, hipStream_t stream) {
  const int64_t n_chunks = rows * cols / 8;
  const dim3 grid((unsigned)((n_chunks + 255) / 256)), block(256);
  auto args = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, (const uint4*)x, (uint32_t*)codes,
                       (uint8_t*)scales, (uint32_t)n_chunks, (uint32_t)(cols / 8), (uint32_t)rows,
                       (uint32_t)scale_rows, (uint32_t)scale_stride, norm, gsp);
  };
  if (zero_policy == FPQ_ZERO_REFERENCE) {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroReference>);
  } else {
    args(quantize_lane8_kernel<G, FMT, ROT, kZeroSigned>);
  }
  return (int)hipGetLastError();
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
  (void)h;

#define FPQ_LAUNCH(GG, RR)                                                                       \
  return launch_lane8<GG, FMT, RR>(x, rows, cols, norm, gsp, codes, scales, scale_rows,         \
                                   scale_stride, zero_policy, stream)
  if (rot_kind == FPQ_ROT_IDENTITY) {
    FPQ_LAUNCH(GROUP, FPQ_ROT_IDENTITY);
  } else if (rot_kind == FPQ_ROT_HADAMARD) {
    switch (g) {
      case 16: FPQ_LAUNCH(16, FPQ_ROT_HADAMARD);
      case 32: FPQ_LAUNCH(32, FPQ_ROT_HADAMARD);
      case 64: FPQ_LAUNCH(64, FPQ_ROT_HADAMARD);
      case 128: FPQ_LAUNCH(128, FPQ_ROT_HADAMARD);
    }
  } else if (rot_kind == FPQ_ROT_GSR || rot_kind == FPQ_ROT_GENERAL) {
    return FPQ_E_UNSUPPORTED;
  }
#undef FPQ_LAUNCH
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

extern "C" int fpq_quantize_nv(const void* x, int64_t rows, int64_t cols, int rot_kind, int g,
                               float norm, const void* h, const float* global_scale, void* codes,
                               void* scales, int64_t scale_rows, int64_t scale_stride,
                               int zero_policy, void* stream) {
  return fpq::dispatch<fpq::kFmtNv>(x, rows, cols, rot_kind, g, norm, h, global_scale, codes,
                                    scales, scale_rows, scale_stride, zero_policy, stream);
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
