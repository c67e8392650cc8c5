// Library-wide pieces of the C ABI: version, thread-local error text, cached device facts.
#include <stdarg.h>

#include <mutex>

#include "common.h"

namespace vamd {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int device_cu_count() {
  // One value per device id; the count cannot change while the process lives.
  static std::mutex mu;
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lock(mu);
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

}  // namespace vamd

extern "C" int vamd_abi_version(void) { return 1; }
extern "C" const char* vamd_last_error(void) { return vamd::g_error; }
