// Per-token log-prob / entropy from MATERIALISED logits, and clip_by_value: the unfused definitions the actor
// uses when the fused head is off (verl/utils/torch_functional.py:72-100 logprobs_from_logits, :148-200 _naive / _v2,
// :224-263 entropy_from_logits / _with_chunking, :203-221 clip_by_value).
//
// Forward: one pass over a row of logits with an online softmax (running max, sum e, sum e*z per thread, merged over
// the workgroup), one workgroup per row, 16-byte loads, four of them in flight per thread.  Algorithmic traffic: the
// logits once.  Backward: elementwise over [rows, vocab], d_logits = g_lp (onehot - p) - g_ent p (z - mean_z) with
// p = exp(z - lse): logits in, gradient out (in place if the caller passes the same buffer).
#include "common.h"

namespace vamd {
namespace {

constexpr int kRowThreads = 256;
constexpr int kInFlight = 4;  // 16-byte loads a thread issues before it consumes them
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;

// kVec: elements per 16-byte load; kBackwardLoads: such loads per thread in the backward kernel
struct F32 { using type = float; static constexpr int kVec = 4; static constexpr int kBackwardLoads = 2; };
struct BF16 { using type = uint16_t; static constexpr int kVec = 8; static constexpr int kBackwardLoads = 1; };
struct F16 { using type = _Float16; static constexpr int kVec = 8; static constexpr int kBackwardLoads = 1; };

__device__ __forceinline__ float to_float(float x, F32) { return x; }
__device__ __forceinline__ float to_float(uint16_t x, BF16) { return __uint_as_float((unsigned)x << 16); }
__device__ __forceinline__ float to_float(_Float16 x, F16) { return (float)x; }
__device__ __forceinline__ float from_float(float x, F32) { return x; }
__device__ __forceinline__ uint16_t from_float(float x, BF16) {
  const __bf16 b = (__bf16)x;  // round to nearest even
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ _Float16 from_float(float x, F16) { return (_Float16)x; }

typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

template <class D>
struct alignas(16) Pack {
  typename D::type v[D::kVec];
};

// Load the D::kVec elements starting at column c of a row (those at or beyond `cols` read as `fill`).
template <class D, bool VEC>
__device__ __forceinline__ void load_group(const typename D::type* __restrict__ row, int64_t c, int64_t cols,
                                           float fill, float (&x)[D::kVec]) {
  if (VEC && c + D::kVec <= cols) {
    // logits are read once and never again by this launch: non-temporal, which is worth 7 % of HBM bandwidth here
    const u32x4_t raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(row + c));
    const Pack<D> p = __builtin_bit_cast(Pack<D>, raw);
#pragma unroll
    for (int e = 0; e < D::kVec; ++e) x[e] = to_float(p.v[e], D());
  } else {
#pragma unroll
    for (int e = 0; e < D::kVec; ++e) x[e] = (c + e < cols) ? to_float(row[c + e], D()) : fill;
  }
}

template <class D, bool VEC>
__device__ __forceinline__ void store_group(typename D::type* __restrict__ row, int64_t c, int64_t cols,
                                            const float (&x)[D::kVec]) {
  if (VEC && c + D::kVec <= cols) {
    Pack<D> p;
#pragma unroll
    for (int e = 0; e < D::kVec; ++e) p.v[e] = from_float(x[e], D());
    __builtin_nontemporal_store(__builtin_bit_cast(u32x4_t, p), reinterpret_cast<u32x4_t*>(row + c));
  } else {
#pragma unroll
    for (int e = 0; e < D::kVec; ++e)
      if (c + e < cols) row[c + e] = from_float(x[e], D());
  }
}

__device__ __forceinline__ void merge(float& m, float& s, float& sz, float m2, float s2, float sz2) {
  const float mm = fmaxf(m, m2);
  const float a = __builtin_amdgcn_exp2f(m - mm), b = __builtin_amdgcn_exp2f(m2 - mm);
  s = s * a + s2 * b;
  sz = sz * a + sz2 * b;
  m = mm;
}

struct StatsArgs {
  const void* logits;
  int64_t ld;
  const int64_t* labels;
  int64_t cols;
  float* logprobs;
  float* entropy;
  float* lse;
  float* mean_z;
};

template <class D, bool VEC>
__global__ __launch_bounds__(kRowThreads) void row_softmax_stats_kernel(StatsArgs a) {
  using T = typename D::type;
  constexpr int G = D::kVec;
  const int64_t r = blockIdx.x;
  const T* __restrict__ row = static_cast<const T*>(a.logits) + r * a.ld;
  // running state in the log2 domain: m = max of z log2(e), s = sum 2^(y - m), sz = sum 2^(y - m) z
  float m = kNegBig, s = 0.f, sz = 0.f;
  const int64_t stride = (int64_t)kRowThreads * G;
  for (int64_t c0 = (int64_t)threadIdx.x * G; c0 < a.cols; c0 += stride * kInFlight) {
    // whole 16-byte groups are all requested first; a ragged last group is fetched element by element afterwards
    u32x4_t raw[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int64_t c = c0 + u * stride;
      if (VEC && c + G <= a.cols) raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(row + c));
    }
    float x[kInFlight][G];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int64_t c = c0 + u * stride;
      if (VEC && c + G <= a.cols) {
        const Pack<D> p = __builtin_bit_cast(Pack<D>, raw[u]);
#pragma unroll
        for (int e = 0; e < G; ++e) x[u][e] = to_float(p.v[e], D());
      } else if (c < a.cols) {
        load_group<D, false>(row, c, a.cols, kNegBig, x[u]);
      } else {
#pragma unroll
        for (int e = 0; e < G; ++e) x[u][e] = kNegBig;
      }
    }
    float gmax = kNegBig;
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int e = 0; e < G; ++e) gmax = fmaxf(gmax, x[u][e]);
    gmax *= kLog2e;
    if (gmax > m) {
      const float resc = __builtin_amdgcn_exp2f(m - gmax);
      s *= resc;
      sz *= resc;
      m = gmax;
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
#pragma unroll
      for (int e = 0; e < G; ++e) {
        const float z = x[u][e];
        const float ex = __builtin_amdgcn_exp2f(fmaf(z, kLog2e, -m));  // padding: 2^(-1e30 ...) = 0
        s += ex;
        sz = fmaf(ex, z, sz);  // padding: 0 * -1e30; a true -inf logit gives NaN, as softmax(z) * z does
      }
  }
  // wavefront, then workgroup
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64), sz2 = __shfl_xor(sz, off, 64);
    merge(m, s, sz, m2, s2, sz2);
  }
  __shared__ float red[3][kRowThreads / 64];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) {
    red[0][w] = m;
    red[1][w] = s;
    red[2][w] = sz;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int j = 1; j < kRowThreads / 64; ++j) merge(m, s, sz, red[0][j], red[1][j], red[2][j]);
    const float lse = (m + log2f(s)) * kLn2;
    const float mz = sz / s;
    if (a.lse) a.lse[r] = lse;
    if (a.mean_z) a.mean_z[r] = mz;
    if (a.entropy) a.entropy[r] = lse - mz;
    if (a.logprobs) {
      // a label outside [0, cols) (an ignore index such as -100, a padding id) reads nothing and yields 0
      const int64_t lab = a.labels[r];
      a.logprobs[r] = (lab >= 0 && lab < a.cols) ? to_float(row[lab], D()) - lse : 0.f;
    }
  }
}

struct BackwardArgs {
  const void* logits;
  int64_t ld;
  const int64_t* labels;  // needed with d_logprobs
  const float* lse;
  const float* mean_z;    // needed with d_entropy
  const float* d_logprobs;
  const float* d_entropy;
  void* d_logits;
  int64_t ld_out;
  int64_t cols;
  int chunks;
};

// One workgroup per (row, chunk of kRowThreads * G * F columns).  F = D::kBackwardLoads 16-byte loads per thread:
// small workgroups in large numbers keep more of the read and the write stream in flight than few workgroups that
// loop (4096 x 152064 fp32 logits: 798 us with 8 KiB per workgroup, 841 with 16 KiB, 913 with a resident grid that
// walks the items and requests the next one before it stores).  What counts is the elements per workgroup, about
// 2048: one load per thread for 16-bit logits (bf16, steady state: 461 us with four loads, 404 with two, 378 with
// one), two for fp32 (828 us; 863 with one).  Trimming the arithmetic per element changed nothing measurable.
template <class D, bool VEC>
__global__ __launch_bounds__(kRowThreads) void row_softmax_backward_kernel(BackwardArgs a) {
  using T = typename D::type;
  constexpr int G = D::kVec, F = D::kBackwardLoads;
  const int64_t r = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  const T* __restrict__ row = static_cast<const T*>(a.logits) + r * a.ld;
  T* __restrict__ out = static_cast<T*>(a.d_logits) + r * a.ld_out;
  const float lse2 = a.lse[r] * kLog2e;
  const float glp = a.d_logprobs ? a.d_logprobs[r] : 0.f;
  const float gent = a.d_entropy ? a.d_entropy[r] : 0.f;
  const float mz = a.d_entropy ? a.mean_z[r] : 0.f;
  const float t0 = fmaf(-gent, mz, glp);  // g_lp + g_ent (z - mean_z) = g_ent z + t0
  const int64_t label = a.d_logprobs ? a.labels[r] : -1;
  const int64_t stride = (int64_t)kRowThreads * G;
  const int64_t c0 = (int64_t)chunk * stride * F + (int64_t)threadIdx.x * G;
  // every whole 16-byte group is requested before anything else happens (the ragged last group of a row, if any,
  // is fetched element by element when its turn comes)
  u32x4_t raw[F];
#pragma unroll
  for (int u = 0; u < F; ++u) {
    const int64_t c = c0 + u * stride;
    if (VEC && c + G <= a.cols) raw[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(row + c));
  }
  float x[F][G];
#pragma unroll
  for (int u = 0; u < F; ++u) {
    const int64_t c = c0 + u * stride;
    if (c >= a.cols) continue;
    if (VEC && c + G <= a.cols) {
      const Pack<D> p = __builtin_bit_cast(Pack<D>, raw[u]);
#pragma unroll
      for (int e = 0; e < G; ++e) x[u][e] = to_float(p.v[e], D());
    } else {
      load_group<D, false>(row, c, a.cols, 0.f, x[u]);
    }
    // the label's place in this group as a 32-bit index (-1: not here): one 32-bit compare per element below
    const int64_t hit64 = label - c;
    const int hit = (hit64 >= 0 && hit64 < G) ? (int)hit64 : -1;
#pragma unroll
    for (int e = 0; e < G; ++e) {
      const float z = x[u][e];
      const float p = __builtin_amdgcn_exp2f(fmaf(z, kLog2e, -lse2));
      // fp32 logits keep the difference z - mean_z (exact where the two are close); for 16-bit logits, whose
      // output rounding is a thousand times coarser, the subtraction is folded into t0
      const float t = sizeof(T) == 4 ? fmaf(gent, z - mz, glp) : fmaf(gent, z, t0);
      x[u][e] = fmaf(-p, t, (hit == e) ? glp : 0.f);
    }
    store_group<D, VEC>(out, c, a.cols, x[u]);
  }
}

// min / max that hand a NaN operand on, like torch.min / torch.max of two tensors (fminf / fmaxf drop it)
__device__ __forceinline__ float min_nan(float a, float b) { return (a != a || b != b) ? a + b : fminf(a, b); }
__device__ __forceinline__ float max_nan(float a, float b) { return (a != a || b != b) ? a + b : fmaxf(a, b); }

// out = max(min(x, hi), lo)
__global__ __launch_bounds__(256) void clip_kernel(const float* __restrict__ x, const float* __restrict__ lo,
                                                   const float* __restrict__ hi, int64_t n, float* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    out[i] = max_nan(min_nan(x[i], hi[i]), lo[i]);
}

// Gradients of max(min(x, hi), lo) the way torch's binary min / max hand them out: the smaller (larger) operand
// takes the gradient, equal operands take half each; an operand loses its share only where the comparison says it
// lost, so where a NaN makes every comparison false both operands receive the whole gradient, as in torch.
__global__ __launch_bounds__(256) void clip_backward_kernel(const float* __restrict__ x, const float* __restrict__ lo,
                                                            const float* __restrict__ hi, const float* __restrict__ g,
                                                            int64_t n, float* __restrict__ dx, float* __restrict__ dlo,
                                                            float* __restrict__ dhi) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float xv = x[i], l = lo[i], h = hi[i], gv = g[i];
    const float a = min_nan(xv, h);
    const float tie1 = xv == h ? 0.5f : 1.f, tie2 = a == l ? 0.5f : 1.f;
    const float a_x = xv > h ? 0.f : tie1;  // d min(x, hi) / dx
    const float a_h = xv < h ? 0.f : tie1;  // d min(x, hi) / dhi
    const float o_a = a < l ? 0.f : tie2;   // d max(a, lo) / da
    const float o_l = a > l ? 0.f : tie2;   // d max(a, lo) / dlo
    if (dx) dx[i] = gv * o_a * a_x;
    if (dhi) dhi[i] = gv * o_a * a_h;
    if (dlo) dlo[i] = gv * o_l;
  }
}

template <class D>
bool rows_vectorizable(const void* base, int64_t ld) {
  return reinterpret_cast<uintptr_t>(base) % 16 == 0 && (ld * (int64_t)sizeof(typename D::type)) % 16 == 0;
}

int check_rows(const char* what, const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t ld) {
  VAMD_REQUIRE(logits != nullptr, "%s: null logits", what);
  VAMD_REQUIRE(dtype >= VAMD_DT_F32 && dtype <= VAMD_DT_F16, "%s: unknown element type code %d", what, dtype);
  VAMD_REQUIRE(n_rows > 0 && vocab > 0 && ld >= vocab, "%s: bad shape rows=%lld vocab=%lld ld=%lld", what,
               (long long)n_rows, (long long)vocab, (long long)ld);
  VAMD_REQUIRE(n_rows < (1ll << 31), "%s: too many rows", what);
  return VAMD_OK;
}

}  // namespace
}  // namespace vamd

using namespace vamd;

#define VAMD_DTYPE_DISPATCH(code, D, ...)                  \
  switch (code) {                                          \
    case VAMD_DT_F32: { using D = F32; __VA_ARGS__; } break;   \
    case VAMD_DT_BF16: { using D = BF16; __VA_ARGS__; } break; \
    default: { using D = F16; __VA_ARGS__; } break;            \
  }

extern "C" int vamd_row_softmax_stats(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t ld,
                                      const int64_t* labels, float* logprobs, float* entropy, float* lse,
                                      float* mean_z, void* stream) {
  int st = check_rows("row_softmax_stats", logits, dtype, n_rows, vocab, ld);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE((logprobs == nullptr) || labels, "row_softmax_stats: logprobs need labels");
  VAMD_REQUIRE(logprobs || entropy || lse || mean_z, "row_softmax_stats: no output requested");
  StatsArgs a{logits, ld, labels, vocab, logprobs, entropy, lse, mean_z};
  hipStream_t s = static_cast<hipStream_t>(stream);
  VAMD_DTYPE_DISPATCH(dtype, D, {
    if (rows_vectorizable<D>(logits, ld))
      hipLaunchKernelGGL((row_softmax_stats_kernel<D, true>), dim3((unsigned)n_rows), dim3(kRowThreads), 0, s, a);
    else
      hipLaunchKernelGGL((row_softmax_stats_kernel<D, false>), dim3((unsigned)n_rows), dim3(kRowThreads), 0, s, a);
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_row_softmax_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t ld,
                                         const int64_t* labels, const float* lse, const float* mean_z,
                                         const float* d_logprobs, const float* d_entropy, void* d_logits,
                                         int64_t ld_out, void* stream) {
  int st = check_rows("row_softmax_backward", logits, dtype, n_rows, vocab, ld);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(d_logits && ld_out >= vocab && lse, "row_softmax_backward: bad output or missing lse");
  VAMD_REQUIRE(d_logprobs || d_entropy, "row_softmax_backward: no upstream gradient");
  VAMD_REQUIRE(!d_logprobs || labels, "row_softmax_backward: d_logprobs needs labels");
  VAMD_REQUIRE(!d_entropy || mean_z, "row_softmax_backward: d_entropy needs mean_z");
  hipStream_t s = static_cast<hipStream_t>(stream);
  VAMD_DTYPE_DISPATCH(dtype, D, {
    const int64_t per_wg = (int64_t)kRowThreads * D::kVec * D::kBackwardLoads;
    const int64_t chunks = (vocab + per_wg - 1) / per_wg;
    VAMD_REQUIRE(n_rows * chunks < (1ll << 31), "row_softmax_backward: too many workgroups");
    BackwardArgs a{logits, ld, labels, lse, mean_z, d_logprobs, d_entropy, d_logits, ld_out, vocab, (int)chunks};
    const dim3 grid((unsigned)(n_rows * chunks));
    if (rows_vectorizable<D>(logits, ld) && rows_vectorizable<D>(d_logits, ld_out))
      hipLaunchKernelGGL((row_softmax_backward_kernel<D, true>), grid, dim3(kRowThreads), 0, s, a);
    else
      hipLaunchKernelGGL((row_softmax_backward_kernel<D, false>), grid, dim3(kRowThreads), 0, s, a);
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

static unsigned flat_grid(int64_t n) {
  int64_t blocks = (n + 255) / 256;
  const int64_t cap = (int64_t)device_cu_count() * 16;
  return (unsigned)(blocks < cap ? blocks : cap);
}

extern "C" int vamd_clip_by_value(const float* x, const float* lo, const float* hi, int64_t n, float* out,
                                  void* stream) {
  VAMD_REQUIRE(x && lo && hi && out && n > 0, "clip_by_value: bad argument");
  hipLaunchKernelGGL(clip_kernel, dim3(flat_grid(n)), dim3(256), 0, static_cast<hipStream_t>(stream), x, lo, hi, n, out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_clip_by_value_backward(const float* x, const float* lo, const float* hi, const float* grad_out,
                                           int64_t n, float* d_x, float* d_lo, float* d_hi, void* stream) {
  VAMD_REQUIRE(x && lo && hi && grad_out && n > 0 && (d_x || d_lo || d_hi), "clip_by_value_backward: bad argument");
  hipLaunchKernelGGL(clip_backward_kernel, dim3(flat_grid(n)), dim3(256), 0, static_cast<hipStream_t>(stream), x, lo,
                     hi, grad_out, n, d_x, d_lo, d_hi);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
