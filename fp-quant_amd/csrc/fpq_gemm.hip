// W4A4 GEMM entry points (placeholder until the MFMA kernels land).
#include <hip/hip_runtime.h>

#include "../../include/fpq.h"

extern "C" int fpq_gemm_mxf4(const void*, const void*, int64_t, const void*, const void*, int64_t,
                             const float*, const void*, void*, int64_t, int64_t, int64_t, void*) {
  return FPQ_E_UNSUPPORTED;
}

extern "C" int fpq_gemm_nvf4(const void*, const void*, int64_t, const void*, const void*, int64_t,
                             const float*, const void*, void*, int64_t, int64_t, int64_t, void*) {
  return FPQ_E_UNSUPPORTED;
}
