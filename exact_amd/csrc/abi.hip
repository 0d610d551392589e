// Version and error strings of the C ABI.
#include "exact_common.hpp"

extern "C" {

int exact_abi_version(void) { return EXACT_ABI_VERSION; }

const char* exact_strerror(int code) {
  switch (code) {
    case EXACT_OK: return "ok";
    case EXACT_E_NULL: return "EXACT_E_NULL: a required pointer is NULL";
    case EXACT_E_BITS: return "EXACT_E_BITS: bits must be 1, 2, 4 or 8";
    case EXACT_E_SHAPE: return "EXACT_E_SHAPE: negative, overflowing or unsupported size";
    case EXACT_E_ALIGN: return "EXACT_E_ALIGN: pointer alignment";
    case EXACT_E_ARG: return "EXACT_E_ARG: bad argument";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error code";
}

}  // extern "C"
