// ABI version and error strings of the katz_hip C ABI.
#include "kh_common.h"

KH_EXPORT int kh_version(void) { return 1; }

KH_EXPORT const char* kh_error_string(int code) {
  switch (code) {
    case KH_OK: return "ok";
    case KH_ERR_INVALID_ARG: return "katz_hip: invalid argument (null pointer, non-positive size or inconsistent shape)";
    case KH_ERR_UNSUPPORTED: return "katz_hip: shape not supported by the kernels";
    case KH_ERR_ALIGNMENT: return "katz_hip: pointer or stride not 16-byte aligned";
    case KH_ERR_TOO_LARGE: return "katz_hip: size beyond the documented maximum";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "katz_hip: unknown error code";
}
