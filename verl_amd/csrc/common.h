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
// Workgroups of `threads` threads of `kernel` (no dynamic LDS) that the current device holds at the same time:
// the grid limit of kernels whose workgroups wait for each other.  Cached per (device, kernel).
int resident_workgroups(const void* kernel, int threads, size_t dynamic_lds_bytes = 0);
// Grid for `items` units of work on a kernel whose workgroups wait for each other: at most `resident`, and chosen so
// that every workgroup walks the same number of items (2048 items on 1536 resident workgroups: 1024 x 2, not
// 1536 of which a third walk two).
inline int64_t balanced_waiting_grid(int64_t items, int64_t resident) {
  if (items <= resident) return items;
  const int64_t passes = (items + resident - 1) / resident;
  return (items + passes - 1) / passes;
}
// Poll limit of the launch-wide rendezvous: VAMD_GATE_SPIN_LIMIT in the environment (tests set 0 to force the
// timed-out path), else `standard`.
unsigned gate_spin_limit(unsigned standard);
// False when VAMD_WAITING_KERNELS=0 in the environment: the entry points then keep to launches whose workgroups
// never wait for each other (one or two launches more), for a GPU shared with long-running kernels of other streams
// or processes, where a launch's workgroups may not all be resident together.
bool waiting_kernels_allowed();

// mask element -> (weight, member) following masked_sum: weight = (float)m, member = m != 0
template <class M>
__device__ __forceinline__ float mask_weight(M m) {
  return static_cast<float>(m);
}

// ------------------------------------------------------------------------------------------
// wavefront / workgroup reductions in double (deterministic: fixed tree, no atomics).
//
// Every active wavefront calls these with all 64 lanes enabled.  The lane exchanges are data-parallel-primitive
// moves inside the vector ALU (a few cycles each) for the steps within a row of 16 lanes, and four lane reads for
// the rows; the same tree through the LDS crossbar (__shfl_xor) costs about a hundred cycles per dependent step,
// which is what a workgroup pays when it is the last one running and nothing hides the latency.
template <int CTRL>
__device__ __forceinline__ double lane_exchange(double x) {
  int lo = __double2loint(x), hi = __double2hiint(x);
  lo = __builtin_amdgcn_update_dpp(0, lo, CTRL, 0xF, 0xF, false);
  hi = __builtin_amdgcn_update_dpp(0, hi, CTRL, 0xF, 0xF, false);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double lane_read(double x, int lane) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(x), lane),
                          __builtin_amdgcn_readlane(__double2loint(x), lane));
}
struct SumOp {
  __device__ __forceinline__ double operator()(double a, double b) const { return a + b; }
  __device__ __forceinline__ double identity() const { return 0.0; }
};
struct MaxOp {
  __device__ __forceinline__ double operator()(double a, double b) const { return fmax(a, b); }
  __device__ __forceinline__ double identity() const { return -__longlong_as_double(0x7ff0000000000000ll); }
};
// Reduce NV values per lane over the wavefront, step-major so the NV chains overlap; the result is in every lane.
// Steps: partner lane ^ 1 and lane ^ 2 (quad permutes), then the mirrored half row and the mirrored row, whose
// partners hold the same value as lane ^ 4 and lane ^ 8 would since a quad / half row is uniform by then.
template <int NV, class Op>
__device__ __forceinline__ void row_reduce(double (&v)[NV], Op op) {  // over each row of 16 lanes
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = op(v[i], lane_exchange<0xB1>(v[i]));   // quad_perm [1,0,3,2]
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = op(v[i], lane_exchange<0x4E>(v[i]));   // quad_perm [2,3,0,1]
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = op(v[i], lane_exchange<0x141>(v[i]));  // row_half_mirror
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = op(v[i], lane_exchange<0x140>(v[i]));  // row_mirror
}
template <int NV, class Op>
__device__ __forceinline__ void wave_reduce(double (&v)[NV], Op op) {
  row_reduce<NV>(v, op);
#pragma unroll
  for (int i = 0; i < NV; ++i)
    v[i] = op(op(lane_read(v[i], 0), lane_read(v[i], 16)), op(lane_read(v[i], 32), lane_read(v[i], 48)));
}
__device__ __forceinline__ double wave_sum(double x) {
  double v[1] = {x};
  wave_reduce<1>(v, SumOp());
  return v[0];
}

// Reduce NV doubles per thread over a workgroup of NT threads; result valid in thread 0.  The wavefront results
// meet in LDS and the first wavefront combines them with one LDS read per value and a reduction over its first
// row of lanes: a single thread reading them one after the other would wait out every LDS round trip.
template <int NV, int NT, class Op>
__device__ __forceinline__ void block_reduce(double (&v)[NV], double* smem /* NV * NT/64 doubles */, Op op) {
  constexpr int NW = NT / 64;
  static_assert(NW <= 16, "the wavefront results are combined inside one row of 16 lanes");
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  wave_reduce<NV>(v, op);
  if (lane == 0)
#pragma unroll
    for (int i = 0; i < NV; ++i) smem[i * NW + w] = v[i];
  __syncthreads();
  if (w == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) v[i] = lane < NW ? smem[i * NW + lane] : op.identity();
    row_reduce<NV>(v, op);
  }
  __syncthreads();
}

// The same for a dozen values or more per thread.  Carrying every value through every exchange step costs
// NV x 6 dependent double operations per wavefront; here the wavefront stages its 64 x NV values in LDS and lane j
// adds up value j over the 64 lanes (in lane order), NV lanes at a time, so the chain is 64 additions whatever NV
// is.  stage: NT/64 * NV * kWidePitch doubles; the pitch of 65 keeps the lanes' rows on different banks and its
// last column takes the wavefront's result.  Result valid in thread 0.
constexpr int kWidePitch = 65;
template <int NV, int NT, class Op>
__device__ __forceinline__ void block_reduce_wide(double (&v)[NV], double* stage, Op op) {
  static_assert(NV <= 64, "one lane per value");
  constexpr int NW = NT / 64;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  double* mine = stage + (size_t)w * NV * kWidePitch;
#pragma unroll
  for (int i = 0; i < NV; ++i) mine[i * kWidePitch + lane] = v[i];
  __syncthreads();
  if (lane < NV) {
    const double* row = mine + lane * kWidePitch;
    double s = row[0];
#pragma unroll 8
    for (int l = 1; l < 64; ++l) s = op(s, row[l]);
    mine[lane * kWidePitch + 64] = s;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      double r = stage[i * kWidePitch + 64];
      for (int j = 1; j < NW; ++j) r = op(r, stage[(size_t)j * NV * kWidePitch + i * kWidePitch + 64]);
      v[i] = r;
    }
  }
  __syncthreads();
}

template <int NV, int NT>
__device__ __forceinline__ void block_sum(double (&v)[NV], double* smem) {
  block_reduce<NV, NT>(v, smem, SumOp());
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
