// Version / error-string entry points of the C ABI.
#include "mdattn_common.h"

namespace mdattn {
namespace {
std::atomic<int> g_fwd_schedule{0};
}
int forced_fwd_schedule() { return g_fwd_schedule.load(std::memory_order_relaxed); }
}  // namespace mdattn

extern "C" int mdattn_set_fwd_schedule(int schedule) {
  if (schedule < 0 || schedule > MDATTN_FWD_SCHEDULE_LAST) return MDATTN_E_BADARG;
  return mdattn::g_fwd_schedule.exchange(schedule, std::memory_order_relaxed);
}

#ifndef MDATTN_BUILD_ID
#define MDATTN_BUILD_ID "unknown"
#endif
// The id sits behind a marker so that it can be read from the file without loading the library (a process that has
// mapped a stale build cannot load the fresh one from the same path any more).
static const char kBuildIdRecord[] = "mdattn-build-id:" MDATTN_BUILD_ID;
extern "C" const char* mdattn_build_id(void) { return kBuildIdRecord + 16; }

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
