// Thread-local error text and the version entry point.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

#include <mutex>
#include <set>
#include <utility>

namespace moe {
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

void clear_error() { g_error[0] = '\0'; }

int num_cus() {
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices] = {};  // 0 = not asked yet; written once per device with the same value
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail(MOE_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(err)), -1;
  if (dev >= 0 && dev < kMaxDevices && cached[dev] > 0) return cached[dev];
  int n = 0;
  err = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
  if (err != hipSuccess || n <= 0)
    return fail(MOE_ERR_HIP, "hipDeviceGetAttribute(multiprocessor count): %s", hipGetErrorString(err)), -1;
  if (dev >= 0 && dev < kMaxDevices) cached[dev] = n;
  return n;
}

int allow_dynamic_lds(const void* kernel, size_t bytes) {
  static std::mutex lock;
  static std::set<std::pair<const void*, int>> done;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail(MOE_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(err));
  std::lock_guard<std::mutex> hold(lock);
  if (done.find({kernel, dev}) != done.end()) return MOE_OK;
  err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
  if (err != hipSuccess)
    return fail(MOE_ERR_HIP, "hipFuncSetAttribute(%zu bytes of LDS): %s", bytes, hipGetErrorString(err));
  done.insert({kernel, dev});
  return MOE_OK;
}

}  // namespace moe

extern "C" int moe_version(void) { return 100; }

extern "C" const char* moe_last_error_string(void) { return moe::g_error; }
