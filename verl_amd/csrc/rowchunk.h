// Shared skeleton of the HBM-bound [rows, cols] kernels (masked reductions, losses, GRPO).
//
// A launch covers the matrix with workgroups of 256 threads; workgroup (row, chunk) owns
// kChunk = 4096 consecutive columns of one row and each thread walks them in float4 steps that
// are contiguous across the wavefront (64 lanes x 16 B = 1 KiB per load instruction).  Partial
// sums leave the workgroup as doubles in a fixed tree order, one record per (row, chunk); a
// second, tiny kernel combines the records in index order, so results are bit-reproducible and
// no floating-point atomics are used.
#pragma once
#include "common.h"

namespace vamd {

constexpr int kRcThreads = 256;
constexpr int kChunk = 4096;  // columns per workgroup

inline int64_t chunks_of(int64_t cols) { return cols <= 0 ? 1 : (cols + kChunk - 1) / kChunk; }

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

template <bool VEC>
__device__ __forceinline__ void ld4(const float* __restrict__ p, int64_t i, int valid, float (&x)[4]) {
  if constexpr (VEC) {
    const float4 v = *reinterpret_cast<const float4*>(p + i);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = e < valid ? p[i + e] : 0.f;
  }
}

template <bool VEC>
__device__ __forceinline__ void st4(float* __restrict__ p, int64_t i, int valid, const float (&x)[4]) {
  if constexpr (VEC) {
    *reinterpret_cast<float4*>(p + i) = make_float4(x[0], x[1], x[2], x[3]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < valid) p[i + e] = x[e];
  }
}

// mask -> float weights; elements past `valid` read as 0 (excluded)
template <bool VEC, class M>
__device__ __forceinline__ void ldmask4(const M* __restrict__ p, int64_t i, int valid, float (&w)[4]) {
  if constexpr (VEC) {
    struct alignas(sizeof(M) * 4) Pack { M v[4]; };
    const Pack k = *reinterpret_cast<const Pack*>(p + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = static_cast<float>(k.v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = e < valid ? static_cast<float>(p[i + e]) : 0.f;
  }
}

// Iterate the 4-element groups of this workgroup's chunk: f(flat_index, valid_count)
template <class F>
__device__ __forceinline__ void for_each_group(int64_t row, int chunk, int64_t cols, F&& f) {
  const int64_t c_begin = (int64_t)chunk * kChunk;
  const int64_t c_end = (c_begin + kChunk) < cols ? (c_begin + kChunk) : cols;
  for (int64_t c = c_begin + (int64_t)threadIdx.x * 4; c < c_end; c += kRcThreads * 4) {
    const int64_t left = c_end - c;
    f(row * cols + c, left < 4 ? (int)left : 4);
  }
}

// The vector path needs 4-element groups that never straddle a row and 16-byte aligned rows.
inline bool can_vectorize(int64_t cols, std::initializer_list<const void*> f32_ptrs, const void* mask,
                          size_t mask_elem) {
  if (cols % 4 != 0) return false;
  for (const void* p : f32_ptrs)
    if (p && !aligned_to(p, 16)) return false;
  if (mask && !aligned_to(mask, mask_elem * 4)) return false;
  return true;
}

// ---------------------------------------------------------------------------------------------
// agg_loss combination of per-row sums (verl/trainer/ppo/core_algos.py:1025-1080).
struct AggParams {
  int mode;
  double dp_size, batch_num_tokens, global_batch_size, loss_scale_factor;  // < 0 : None
};

// Called by ONE workgroup of 256 threads.  partials: [rows][chunks][NV] doubles with slot 0 =
// sum(loss * w) and slot 1 = sum(w); slots >= 2 are summed over everything into extra[].
// Writes loss (double, thread 0) and coef[rows].
template <int NV>
__device__ void finalize_agg(const double* __restrict__ partials, int64_t rows, int chunks, int64_t cols,
                             const AggParams& ap, float* __restrict__ coef, double& loss_out, double& msum_out,
                             double (&extra)[NV > 2 ? NV - 2 : 1], double* smem) {
  // pass 1: totals
  double tot[NV + 1];  // slot NV: number of rows with a non-empty mask
#pragma unroll
  for (int i = 0; i <= NV; ++i) tot[i] = 0;
  double seq_mean_sum = 0;  // sum over kept rows of S_i / (M_i + 1e-8)
  double seq_sum = 0;       // sum over kept rows of S_i
  for (int64_t r = threadIdx.x; r < rows; r += kRcThreads) {
    double row[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) row[i] = 0;
    for (int c = 0; c < chunks; ++c)
#pragma unroll
      for (int i = 0; i < NV; ++i) row[i] += partials[(r * chunks + c) * NV + i];
#pragma unroll
    for (int i = 0; i < NV; ++i) tot[i] += row[i];
    if (row[1] > 0) {
      tot[NV] += 1;
      seq_sum += row[0];
      seq_mean_sum += (double)((float)row[0] / ((float)row[1] + 1e-8f));
    }
  }
  double red[NV + 3];
#pragma unroll
  for (int i = 0; i <= NV; ++i) red[i] = tot[i];
  red[NV + 1] = seq_mean_sum;
  red[NV + 2] = seq_sum;
  block_sum<NV + 3, kRcThreads>(red, smem);
  __shared__ double bc[NV + 3];
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < NV + 3; ++i) bc[i] = red[i];
  __syncthreads();
  const double S = bc[0], Msum = bc[1], kept = bc[NV], smean = bc[NV + 1], ssum = bc[NV + 2];
  double loss = 0, c_all = 0;
  double gbs = ap.global_batch_size < 0 ? kept : ap.global_batch_size;
  switch (ap.mode) {
    case VAMD_AGG_TOKEN_MEAN: {
      const double denom = ap.batch_num_tokens < 0 ? Msum : ap.batch_num_tokens;
      loss = S / denom * ap.dp_size;
      c_all = ap.dp_size / denom;
    } break;
    case VAMD_AGG_SEQ_MEAN_TOKEN_SUM:
      loss = ssum / gbs * ap.dp_size;
      break;
    case VAMD_AGG_SEQ_MEAN_TOKEN_MEAN:
      loss = smean / gbs * ap.dp_size;
      break;
    default: {
      const double f = ap.loss_scale_factor < 0 ? (double)cols : ap.loss_scale_factor;
      loss = S / f;
      c_all = 1.0 / f;
    } break;
  }
  if (coef) {
    for (int64_t r = threadIdx.x; r < rows; r += kRcThreads) {
      double c = c_all;
      if (ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_SUM || ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_MEAN) {
        double m = 0;
        for (int k = 0; k < chunks; ++k) m += partials[(r * chunks + k) * NV + 1];
        c = 0;
        if (m > 0) c = (ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_SUM ? 1.0 : 1.0 / (m + 1e-8)) * ap.dp_size / gbs;
      }
      coef[r] = (float)c;
    }
  }
  loss_out = loss;
  msum_out = Msum;
#pragma unroll
  for (int i = 2; i < NV; ++i) extra[i - 2] = bc[i];
}

}  // namespace vamd
