// Host-side error bookkeeping for libbrt_hip.so.
#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <set>
#include <utility>

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

int allow_dynamic_lds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(BRT_E_LAUNCH, "no current device");
  std::lock_guard<std::mutex> guard(mu);
  if (done.count({kernel, dev}) != 0) return BRT_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return fail(BRT_E_LAUNCH, "cannot reserve %d bytes of LDS", bytes);
  }
  done.insert({kernel, dev});
  return BRT_OK;
}
}  // namespace brt

extern "C" const char* brt_hip_last_error(void) { return brt::g_error; }
extern "C" const char* brt_hip_version(void) { return "0.1"; }
