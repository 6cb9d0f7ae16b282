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
