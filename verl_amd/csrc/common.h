// Shared host-side helpers for the C-ABI entry points: error recording, argument checks,
// workspace carving, and small device-side reduction helpers used by the HBM-bound kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/verl_amd.h"

namespace vamd {

void set_error(const char* fmt, ...);

#define VAMD_REQUIRE(cond, ...)      \
  do {                               \
    if (!(cond)) {                   \
      ::vamd::set_error(__VA_ARGS__); \
      return VAMD_EINVAL;            \
    }                                \
  } while (0)

#define VAMD_HIP(expr)                                                                   \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      ::vamd::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
      return VAMD_EHIP;                                                                  \
    }                                                                                    \
  } while (0)

#define VAMD_LAUNCH_CHECK() VAMD_HIP(hipGetLastError())

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Bump allocator over the caller's workspace.
struct Carver {
  char* base;
  size_t off = 0;
  explicit Carver(void* p) : base(static_cast<char*>(p)) {}
  template <class T>
  T* take(size_t count) {
    off = align_up(off, 256);
    T* r = reinterpret_cast<T*>(base + off);
    off += count * sizeof(T);
    return r;
  }
  size_t used() const { return align_up(off, 256); }
};

int device_cu_count();

// mask element -> (weight, member) following masked_sum: weight = (float)m, member = m != 0
template <class M>
__device__ __forceinline__ float mask_weight(M m) {
  return static_cast<float>(m);
}

// ------------------------------------------------------------------------------------------
// wavefront / workgroup sums in double (deterministic: fixed tree, no atomics)
__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

// Sum NV doubles per thread over a workgroup of NT threads; result valid in thread 0.
template <int NV, int NT>
__device__ __forceinline__ void block_sum(double (&v)[NV], double* smem /* NV * NT/64 doubles */) {
  constexpr int NW = NT / 64;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    v[i] = wave_sum(v[i]);
    if (lane == 0) smem[i * NW + w] = v[i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      double s = 0;
      for (int j = 0; j < NW; ++j) s += smem[i * NW + j];
      v[i] = s;
    }
  }
  __syncthreads();
}

}  // namespace vamd

// Dispatch a templated launch over the mask element type.
#define VAMD_MASK_DISPATCH(code, M, ...)                      \
  switch (code) {                                             \
    case VAMD_MASK_F32: { using M = float; __VA_ARGS__; } break;   \
    case VAMD_MASK_I64: { using M = int64_t; __VA_ARGS__; } break; \
    case VAMD_MASK_U8: { using M = uint8_t; __VA_ARGS__; } break;  \
    case VAMD_MASK_I32: { using M = int32_t; __VA_ARGS__; } break; \
    default: ::vamd::set_error("unknown mask dtype code %d", code); return VAMD_EINVAL; \
  }
