// Version and error-string entry points of the C ABI.
#include "adh_common.h"

extern "C" {

int adh_version(void) { return ADH_VERSION; }

const char *adh_error_string(int code) {
  switch (code) {
    case ADH_OK: return "ok";
    case ADH_EINVAL: return "invalid argument (extent, window bounds, H % K, tile count or beta)";
    case ADH_EUNIMPL: return "unimplemented combination (grid with both dimensions > 1, or dtype)";
    case ADH_ENULL: return "required pointer is NULL";
    case ADH_EALIGN: return "pointer not aligned to its element size";
    case ADH_EWORKSPACE: return "workspace too small";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown adh error";
}

}  // extern "C"
