// Library-level entry points of libmi_moe.so: ABI version and error text.
#include "common.h"

extern "C" int mi_moe_abi_version(void) { return MI_MOE_ABI_VERSION; }

extern "C" const char* mi_moe_strerror(int rc) {
  switch (rc) {
    case MI_MOE_OK: return "ok";
    case MI_MOE_ENULL: return "mi_moe: a required pointer is NULL";
    case MI_MOE_ESHAPE: return "mi_moe: a dimension is outside the supported range";
    case MI_MOE_EDTYPE: return "mi_moe: unsupported element type for this entry point";
    case MI_MOE_EALIGN: return "mi_moe: a pointer or leading dimension is not aligned as required";
    case MI_MOE_EWORKSPACE: return "mi_moe: workspace missing or too small";
    case MI_MOE_EUNSUPPORTED: return "mi_moe: shape / option combination not supported by this entry point";
    case MI_MOE_ETOOLARGE: return "mi_moe: input needs more scratch memory than this non-allocating entry point holds";
    default: break;
  }
  if (rc > 0) return hipGetErrorString(static_cast<hipError_t>(rc));
  return "mi_moe: unknown error code";
}
