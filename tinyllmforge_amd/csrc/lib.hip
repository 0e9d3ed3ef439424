// Library-level entry points of libtlf_hip.so.
#include "common.h"

extern "C" int tlf_version(void) { return TLF_ABI_VERSION; }

extern "C" const char *tlf_error_string(int code) {
  switch (code) {
    case TLF_OK: return "ok";
    case TLF_E_NULL: return "a required pointer is NULL";
    case TLF_E_SHAPE: return "a size or stride is out of range";
    case TLF_E_ALIGN: return "a pointer or stride is not 16-byte aligned";
    case TLF_E_WORKSPACE: return "workspace missing, misaligned or too small";
    case TLF_E_UNSUPPORTED: return "no kernel for this combination";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

extern "C" int tlf_device_info(int32_t *num_cus, int32_t *lds_bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (num_cus) *num_cus = prop.multiProcessorCount;
  if (lds_bytes) *lds_bytes = static_cast<int32_t>(prop.sharedMemPerBlock);
  return TLF_OK;
}
