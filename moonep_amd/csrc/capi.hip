// Version and error strings of the C ABI.
#include "mep_common.h"

extern "C" int mep_version(void) { return 100; }  // major*10000 + minor*100 + patch

extern "C" const char* mep_strerror(int code) {
  switch (code) {
    case MEP_OK: return "ok";
    case MEP_ERR_INVALID_ARG: return "invalid argument (null pointer, size or rank out of range)";
    case MEP_ERR_UNSUPPORTED: return "shape not supported by the gfx950 kernels";
    case MEP_ERR_SCRATCH: return "scratch buffer missing or too small";
    case MEP_ERR_ALIGNMENT: return "pointer or stride not 16-byte aligned";
    case MEP_ERR_STATIC_LIMIT:
      return "input exceeds the fixed scratch of the allocation-free entry point (use the variant "
             "that takes a scratch buffer)";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}
