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

// out = a + b + c + d, 16 bytes per lane from each input: the traffic of a fused loss kernel with its gradient
// (four tensors in, one out) without any of its arithmetic or its reduction, as a second yardstick.
__global__ __launch_bounds__(256) void sum4_kernel(const float4* __restrict__ a, const float4* __restrict__ b,
                                                   const float4* __restrict__ c, const float4* __restrict__ d,
                                                   float4* __restrict__ out, int64_t n4) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    const float4 x = a[i], y = b[i], z = c[i], w = d[i];
    out[i] = make_float4(x.x + y.x + z.x + w.x, x.y + y.y + z.y + w.y, x.z + y.z + z.z + w.z, x.w + y.w + z.w + w.w);
  }
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

extern "C" int vamd_sum4(const float* a, const float* b, const float* c, const float* d, float* out, int64_t n,
                         void* stream) {
  using namespace vamd;
  VAMD_REQUIRE(a && b && c && d && out && n > 0 && n % 4 == 0, "sum4: need non-null pointers and a multiple of 4 elements");
  VAMD_REQUIRE((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c) |
                reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(out)) % 16 == 0,
               "sum4: pointers must be 16-byte aligned");
  const int64_t n4 = n / 4;
  int64_t blocks = (n4 + 255) / 256;
  const int64_t cap = (int64_t)device_cu_count() * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(sum4_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const float4*)a,
                     (const float4*)b, (const float4*)c, (const float4*)d, (float4*)out, n4);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_abi_version(void) { return VAMD_ABI_VERSION; }
extern "C" const char* vamd_last_error(void) { return vamd::g_error; }
