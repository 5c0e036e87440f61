// Version and error naming of the C ABI.
#include "aq_common.h"

extern "C" int aq_version(void) { return AQ_VERSION; }

extern "C" const char* aq_error_string(int code) {
  switch (code) {
    case AQ_OK: return "ok";
    case AQ_E_NULL: return "a required pointer is NULL";
    case AQ_E_SHAPE: return "bad shape (negative size, K not a multiple of 16, M > 16 for the decode path, ldx < K)";
    case AQ_E_DTYPE: return "unknown dtype code";
    case AQ_E_ALIGN: return "pointer or leading dimension is not 16-byte aligned";
    case AQ_E_WORKSPACE: return "workspace too small";
    case AQ_E_RANGE: return "size beyond what the kernels index, or beyond the array of the no-allocation entry point";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}
