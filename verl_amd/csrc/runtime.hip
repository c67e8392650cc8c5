// Library-wide pieces of the C ABI: version, thread-local error text, cached device facts.
#include <stdarg.h>
#include <stdlib.h>

#include <map>
#include <tuple>
#include <mutex>
#include <utility>

#include "common.h"

#include <atomic>

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

int resident_workgroups(const void* kernel, int threads, size_t dynamic_lds_bytes) {
  static std::mutex mu;
  static std::map<std::tuple<int, const void*, size_t>, int> cache;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find({dev, kernel, dynamic_lds_bytes});
  if (it != cache.end()) return it->second;
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, dynamic_lds_bytes) != hipSuccess || per_cu < 1)
    per_cu = 1;
  // The runtime's figure follows vector registers and LDS; a kernel with close to a hundred scalar registers was
  // seen to fit one wavefront per SIMD fewer than it says (2048 workgroups of 256 threads did not all become
  // resident, 1792 would have).  Waiting kernels must never overestimate, so two waves per SIMD are held back.
  const int waves_per_wg = (threads + 63) / 64;
  const int cap = (6 * 4) / waves_per_wg;  // 6 of the 8 wavefront slots of each of the 4 SIMDs
  if (cap >= 1 && per_cu > cap) per_cu = cap;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 1;
  const int n = per_cu * cus;
  cache[{dev, kernel, dynamic_lds_bytes}] = n;
  return n;
}

// Process-wide switch over the environment variable: -1 = not set (the variable decides), 0 / 1 = set by
// vamd_set_waiting_kernels().  A host that has seen one waiting kernel time out switches all of them off at once.
static std::atomic<int> g_waiting_override{-1};

bool waiting_kernels_allowed() {
  const int o = g_waiting_override.load(std::memory_order_relaxed);
  if (o >= 0) return o != 0;
  const char* e = getenv("VAMD_WAITING_KERNELS");
  return !(e && e[0] == '0' && e[1] == 0);
}

unsigned gate_spin_limit(unsigned standard) {
  if (const char* e = getenv("VAMD_GATE_SPIN_LIMIT")) {
    char* end = nullptr;
    const unsigned long v = strtoul(e, &end, 10);
    if (end != e) return (unsigned)v;
  }
  return standard;
}

// Plain streaming copy, 16 bytes per lane and grid-stride: the yardstick the memory counters of
// the other kernels are scaled by.  STREAM: non-temporal loads and stores, the policy the [B, L] kernels use for
// tensors beyond the caches.
typedef unsigned ys_u32x4 __attribute__((ext_vector_type(4)));
typedef float ys_f32x4 __attribute__((ext_vector_type(4)));
template <bool STREAM>
__global__ __launch_bounds__(256) void copy_kernel(const ys_u32x4* __restrict__ src, ys_u32x4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
    if (STREAM) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
    else dst[i] = src[i];
  }
}

// out = a + b + c + d, 16 bytes per lane from each input: the traffic of a fused loss kernel with its gradient
// (four tensors in, one out) without any of its arithmetic or its reduction, as a second yardstick.
template <bool STREAM>
__global__ __launch_bounds__(256) void sum4_kernel(const ys_f32x4* __restrict__ a, const ys_f32x4* __restrict__ b,
                                                   const ys_f32x4* __restrict__ c, const ys_f32x4* __restrict__ d,
                                                   ys_f32x4* __restrict__ out, int64_t n4) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
    if (STREAM) {
      const ys_f32x4 x = __builtin_nontemporal_load(a + i), y = __builtin_nontemporal_load(b + i),
                     z = __builtin_nontemporal_load(c + i), w = __builtin_nontemporal_load(d + i);
      __builtin_nontemporal_store(x + y + z + w, out + i);
    } else {
      out[i] = a[i] + b[i] + c[i] + d[i];
    }
  }
}

constexpr int64_t kStreamingBytes = 64ll << 20;  // per tensor: the size from which the [B, L] kernels stream

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
  if (bytes >= kStreamingBytes)
    hipLaunchKernelGGL(copy_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const ys_u32x4*)src, (ys_u32x4*)dst, n16);
  else
    hipLaunchKernelGGL(copy_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const ys_u32x4*)src, (ys_u32x4*)dst, n16);
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
  if (n * 4 >= kStreamingBytes)
    hipLaunchKernelGGL(sum4_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const ys_f32x4*)a, (const ys_f32x4*)b, (const ys_f32x4*)c, (const ys_f32x4*)d, (ys_f32x4*)out, n4);
  else
    hipLaunchKernelGGL(sum4_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const ys_f32x4*)a, (const ys_f32x4*)b, (const ys_f32x4*)c, (const ys_f32x4*)d, (ys_f32x4*)out, n4);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// Pure matrix-instruction loop, no memory traffic: what the matrix pipes deliver under the board's power management
// when nothing else draws power.  Every wavefront keeps 4 + 4 operand fragments (from `seed`, so the caller chooses
// how much they toggle) and 128 accumulator registers, and issues independent MFMAs round robin.
typedef __bf16 ys_bf16x8 __attribute__((ext_vector_type(8)));
typedef float ys_f32x16 __attribute__((ext_vector_type(16)));
template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_yardstick_kernel(const uint32_t* __restrict__ seed, float* __restrict__ out,
                                                             int iters) {
  ys_bf16x8 a[4], b[4];
  const uint32_t* s = seed + ((size_t)blockIdx.x * 512 + threadIdx.x) * 32;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    union {
      uint32_t u[4];
      ys_bf16x8 v;
    } ua, ub;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ua.u[j] = s[i * 8 + j];
      ub.u[j] = s[i * 8 + 4 + j];
    }
    a[i] = ua.v;
    b[i] = ub.v;
  }
  float sum = 0.f;
  if constexpr (SHAPE == VAMD_MFMA_32X32X16) {
    ys_f32x16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 3], b[i >> 1], acc[i], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 16; ++j) sum += acc[i][j];
  } else {
    vamd::ys_f32x4 acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = vamd::ys_f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 32; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 32; ++i) sum += (acc[i][0] + acc[i][1]) + (acc[i][2] + acc[i][3]);
  }
  out[(size_t)blockIdx.x * 512 + threadIdx.x] = sum;
}

extern "C" int64_t vamd_mfma_yardstick_flops(int shape, int workgroups, int iters) {
  if (workgroups <= 0 || iters <= 0) return 0;
  // per iteration and wavefront: 8 x 32768 flops, or 32 x 16384 flops
  const int64_t per_iter = shape == VAMD_MFMA_32X32X16 ? 8ll * 32768 : 32ll * 16384;
  return (int64_t)workgroups * 8 * iters * per_iter;
}

extern "C" int vamd_mfma_yardstick(int shape, const void* seed, float* out, int workgroups, int iters, void* stream) {
  using namespace vamd;
  VAMD_REQUIRE(seed && out && workgroups > 0 && iters > 0, "mfma_yardstick: need seed, out, workgroups > 0, iters > 0");
  VAMD_REQUIRE(shape == VAMD_MFMA_32X32X16 || shape == VAMD_MFMA_16X16X32, "mfma_yardstick: unknown shape %d", shape);
  if (shape == VAMD_MFMA_32X32X16)
    hipLaunchKernelGGL(mfma_yardstick_kernel<VAMD_MFMA_32X32X16>, dim3((unsigned)workgroups), dim3(512), 0,
                       (hipStream_t)stream, static_cast<const uint32_t*>(seed), out, iters);
  else
    hipLaunchKernelGGL(mfma_yardstick_kernel<VAMD_MFMA_16X16X32>, dim3((unsigned)workgroups), dim3(512), 0,
                       (hipStream_t)stream, static_cast<const uint32_t*>(seed), out, iters);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_abi_version(void) { return VAMD_ABI_VERSION; }
extern "C" const char* vamd_last_error(void) { return vamd::g_error; }

extern "C" void vamd_set_waiting_kernels(int allowed) {
  vamd::g_waiting_override.store(allowed < 0 ? -1 : (allowed != 0 ? 1 : 0), std::memory_order_relaxed);
}

extern "C" int vamd_waiting_kernels_enabled(void) { return vamd::waiting_kernels_allowed() ? 1 : 0; }
