// Host-side error bookkeeping for libbrt_hip.so.
#include <cstdarg>
#include <cstdio>

#include "common.hpp"

namespace brt {
namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return BRT_OK;
  return fail(BRT_E_LAUNCH, "%s: %s", what, hipGetErrorString(err));
}
}  // namespace brt

extern "C" const char* brt_hip_last_error(void) { return brt::g_error; }
extern "C" const char* brt_hip_version(void) { return "0.1"; }
