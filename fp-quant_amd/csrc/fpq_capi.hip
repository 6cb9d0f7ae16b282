// Library-level entry points of the C ABI: version, status strings, device check.
#include <hip/hip_runtime.h>
#include <string.h>

#include "../../include/fpq.h"

extern "C" int fpq_version(void) { return FPQ_VERSION; }

extern "C" const char* fpq_status_string(int status) {
  switch (status) {
    case FPQ_OK: return "ok";
    case FPQ_E_NULL: return "a required pointer is null";
    case FPQ_E_SHAPE: return "sizes violate the documented divisibility or range rules";
    case FPQ_E_ROTATION: return "unknown rotation kind or unsupported rotation block size";
    case FPQ_E_ALIGN: return "a pointer is not aligned as documented";
    case FPQ_E_POLICY: return "unknown zero-nibble policy";
    case FPQ_E_UNSUPPORTED: return "no kernel in this build for the requested combination";
    case FPQ_E_LIMIT: return "a size is beyond the stated maximum of this entry point";
    default: break;
  }
  if (status > 0) return hipGetErrorString((hipError_t)status);
  return "unknown fpq status";
}

extern "C" int fpq_device_supported(int device) {
  hipDeviceProp_t prop;
  const hipError_t err = hipGetDeviceProperties(&prop, device);
  if (err != hipSuccess) return (int)err;
  return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

#include <atomic>

namespace fpq {
// Compute units of the current device, asked once per device; 256 (one MI355X) where no device answers, so
// that the size helpers stay host arithmetic.  Every shape threshold of the GEMM dispatch that stands for
// "one round of workgroups" or a fraction of it is derived from this number.
int device_cus() {
  constexpr int kDefault = 256, kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
    (void)hipGetLastError();
    return kDefault;
  }
  if (dev < kMaxDevices) {
    const int hit = cached[dev].load(std::memory_order_acquire);
    if (hit > 0) return hit;
  }
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
    (void)hipGetLastError();
    return kDefault;
  }
  if (dev < kMaxDevices) cached[dev].store(cus, std::memory_order_release);
  return cus;
}

int ensure_silu_table(hipStream_t stream);   // fpq_quantize.hip
int scratch_address(void** out);             // fpq_gemm_stream.hip
}  // namespace fpq

extern "C" int fpq_compute_units(void) { return fpq::device_cus(); }

extern "C" int fpq_prepare_device(void* stream) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  const hipError_t err = hipStreamIsCapturing((hipStream_t)stream, &cap);
  if (err != hipSuccess) return (int)err;
  if (cap != hipStreamCaptureStatusNone) return FPQ_E_UNSUPPORTED;   // it has to run, not be recorded
  if (const int st = fpq::ensure_silu_table((hipStream_t)stream)) return st;
  void* scratch = nullptr;
  return fpq::scratch_address(&scratch);
}

extern "C" int fpq_stream_capture_id(void* stream, unsigned long long* id) {
  if (!id) return FPQ_E_NULL;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long cid = 0;
  const hipError_t err = hipStreamGetCaptureInfo((hipStream_t)stream, &status, &cid);
  if (err != hipSuccess) return (int)err;
  *id = status == hipStreamCaptureStatusNone ? 0ull : (cid ? cid : ~0ull);
  return FPQ_OK;
}

// ---------------------------------------------------------------------------------------------
// Measurement hook: the rate at which the matrix pipes execute the FP4 block-scaled MFMA on
// operands that never leave registers -- no memory traffic, no LDS, no barriers -- so the only
// limits left are the issue rate and the clock the chip sustains for the given operand bits.
namespace fpq {
typedef int probe_v8i __attribute__((ext_vector_type(8)));
typedef float probe_v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_rate_kernel(const int* __restrict__ words, int iters,
                                                        float* __restrict__ sink,
                                                        unsigned long long* __restrict__ clocks) {
  const int t = threadIdx.x + blockIdx.x * 256;
  probe_v8i a[4], b[4];
  for (int i = 0; i < 4; ++i) {
    const int* w = words + (size_t)t * 32 + i * 4;
    a[i] = probe_v8i{w[0], w[1], w[2], w[3], 0, 0, 0, 0};
    b[i] = probe_v8i{w[16], w[17], w[18], w[19], 0, 0, 0, 0};
  }
  const int sa = 0x7f7f7f7f, sb = 0x7f7f7f7f;  // scale 1.0 in every byte
  probe_v16f acc[4][4];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 4, 4, 0, sa, 0, sb);
  }
  const unsigned long long c1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  sink[t] = s;
  if (threadIdx.x == 0) {
    clocks[blockIdx.x * 2] = c1 - c0;       // shader clock cycles
    clocks[blockIdx.x * 2 + 1] = r1 - r0;   // 100 MHz ticks
  }
}
}  // namespace fpq

extern "C" int fpq_test_mfma_rate(const int* words, int blocks, int iters, float* sink,
                                  unsigned long long* clocks, void* stream) {
  if (!words || !sink || !clocks) return FPQ_E_NULL;
  if (blocks <= 0 || iters <= 0) return FPQ_E_SHAPE;
  hipLaunchKernelGGL(fpq::mfma_rate_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, words,
                     iters, sink, clocks);
  return (int)hipGetLastError();
}
