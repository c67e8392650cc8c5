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

// Plain streaming copy, 16 bytes per lane and grid-stride: the yardstick the memory counters of
// the other kernels are scaled by.
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

}  // namespace vamd

extern "C" int vamd_copy_bytes(const void* src, void* dst, int64_t bytes, void* stream) {
  using namespace vamd;
  VAMD_REQUIRE(src && dst && bytes > 0 && bytes % 16 == 0, "copy_bytes: need non-null pointers and a multiple of 16 bytes");
  VAMD_REQUIRE((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 == 0,
               "copy_bytes: pointers must be 16-byte aligned");
  const int64_t n16 = bytes / 16;
  int64_t blocks = (n16 + 255) / 256;
  const int64_t cap = (int64_t)device_cu_count() * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                     (uint4*)dst, n16);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_abi_version(void) { return 3; }
extern "C" const char* vamd_last_error(void) { return vamd::g_error; }
