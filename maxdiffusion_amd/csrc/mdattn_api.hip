// Version / error-string entry points of the C ABI.
#include "mdattn_common.h"

extern "C" int mdattn_version(void) { return MDATTN_VERSION; }

extern "C" const char* mdattn_strerror(int code) {
  switch (code) {
    case MDATTN_OK: return "ok";
    case MDATTN_E_BADARG: return "bad argument (null pointer, non-positive size or inconsistent shape)";
    case MDATTN_E_UNSUPPORTED: return "unsupported configuration for this build";
    case MDATTN_E_ALIGN: return "pointer or stride not aligned (16-byte pointers, strides multiple of 8 elements)";
    case MDATTN_E_LAUNCH: return "HIP runtime rejected the kernel launch";
    case MDATTN_E_TOOBIG: return "request exceeds the static scratch array of this no-allocation entry point";
    default: return "unknown mdattn error code";
  }
}
