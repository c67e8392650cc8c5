// HBM-bound kernels of the PPO / GRPO policy math: masked moments and whitening, agg_loss,
// the clipped + dual-clip policy loss, the clipped value loss, GRPO group-normalised advantages.
// Reference semantics: verl/utils/torch_functional.py:266-339 and
// verl/trainer/ppo/core_algos.py:266-357, :1025-1080, :1159-1250, :1799-1838.
#include <initializer_list>

#include "rowchunk.h"

namespace vamd {

// =============================================================================================
// masked moments
// =============================================================================================
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void moments_kernel(const float* __restrict__ values,
                                                             const M* __restrict__ mask, int64_t cols, int chunks,
                                                             double* __restrict__ partials) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  float s0 = 0, s1 = 0, s2 = 0, cnt = 0;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float x[4], w[4];
    ld4<VEC>(values, i, valid, x);
    ldmask4<VEC>(mask, i, valid, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool in = w[e] != 0.f;
      const float v = in ? x[e] : 0.f;  // where(mask.bool(), values, 0)
      s0 += w[e];
      s1 += v * w[e];
      s2 += v * v * w[e];
      cnt += in ? 1.f : 0.f;
    }
  });
  __shared__ double smem[16];
  double acc[4] = {s0, s1, s2, cnt};
  block_sum<4, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    double* o = partials + (int64_t)blockIdx.x * 4;
    o[0] = acc[0]; o[1] = acc[1]; o[2] = acc[2]; o[3] = acc[3];
  }
}

// out[r][0..3] = sum over chunks (per_row) or out[0..3] = sum over everything
__global__ __launch_bounds__(kRcThreads) void moments_finalize_kernel(const double* __restrict__ partials,
                                                                      int64_t rows, int chunks, int per_row,
                                                                      double* __restrict__ out) {
  if (per_row) {
    const int64_t r = (int64_t)blockIdx.x * kRcThreads + threadIdx.x;
    if (r >= rows) return;
    double a[4] = {0, 0, 0, 0};
    for (int c = 0; c < chunks; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] += partials[(r * chunks + c) * 4 + i];
#pragma unroll
    for (int i = 0; i < 4; ++i) out[r * 4 + i] = a[i];
  } else {
    double a[4] = {0, 0, 0, 0};
    const int64_t n = rows * chunks;
    for (int64_t k = threadIdx.x; k < n; k += kRcThreads)
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] += partials[k * 4 + i];
    __shared__ double smem[16];
    block_sum<4, kRcThreads>(a, smem);
    if (threadIdx.x == 0)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = a[i];
  }
}

// stats = (mean, rsqrt(var_unbiased + 1e-8), shift) from the four moments, following
// masked_mean / masked_var / masked_whiten (torch_functional.py:287-339).
__global__ void whiten_stats_kernel(const double* __restrict__ mom, int shift_mean, float* __restrict__ stats) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const double s0 = mom[0], s1 = mom[1], s2 = mom[2];
  const float mean = (float)s1 / ((float)s0 + 1e-8f);
  const double md = (double)mean;
  // masked_mean((v - mean)^2) with the same epsilon in the denominator
  float var = (float)((s2 - 2.0 * md * s1 + md * md * s0)) / ((float)s0 + 1e-8f);
  var = var * ((float)s0 / ((float)s0 - 1.f));  // Bessel factor M / (M - 1)
  stats[0] = mean;
  stats[1] = rsqrtf(var + 1e-8f);
  stats[2] = shift_mean ? 0.f : mean;
}

__global__ __launch_bounds__(kRcThreads) void affine_kernel(const float* __restrict__ values,
                                                            const float* __restrict__ stats, int64_t n,
                                                            float* __restrict__ out, int vec) {
  const float mean = stats[0], rstd = stats[1], shift = stats[2];
  const int64_t stride = (int64_t)gridDim.x * kRcThreads * 4;
  for (int64_t i = ((int64_t)blockIdx.x * kRcThreads + threadIdx.x) * 4; i < n; i += stride) {
    const int64_t left = n - i;
    float x[4];
    if (vec) {
      ld4<true>(values, i, 4, x);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = (x[e] - mean) * rstd + shift;
      st4<true>(out, i, 4, x);
    } else {
      const int valid = left < 4 ? (int)left : 4;
      ld4<false>(values, i, valid, x);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = (x[e] - mean) * rstd + shift;
      st4<false>(out, i, valid, x);
    }
  }
}

// =============================================================================================
// agg_loss forward / backward
// =============================================================================================
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void agg_partial_kernel(const float* __restrict__ loss_mat,
                                                                 const M* __restrict__ mask, int64_t cols,
                                                                 int chunks, int token_mean,
                                                                 double* __restrict__ partials) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  float s = 0, m = 0;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float x[4], w[4];
    ld4<VEC>(loss_mat, i, valid, x);
    ldmask4<VEC>(mask, i, valid, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // token-mean goes through masked_sum (where() first); the seq-* modes multiply directly
      const float v = (token_mean && w[e] == 0.f) ? 0.f : x[e];
      if (e < valid) s += v * w[e];
      m += w[e];
    }
  });
  __shared__ double smem[8];
  double acc[2] = {s, m};
  block_sum<2, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    partials[(int64_t)blockIdx.x * 2] = acc[0];
    partials[(int64_t)blockIdx.x * 2 + 1] = acc[1];
  }
}

__global__ __launch_bounds__(kRcThreads) void agg_finalize_kernel(const double* __restrict__ partials, int64_t rows,
                                                                  int chunks, int64_t cols, AggParams ap,
                                                                  float* __restrict__ out_loss,
                                                                  float* __restrict__ coef) {
  __shared__ double smem[(2 + 3) * 4];
  double loss, msum, extra[1];
  finalize_agg<2>(partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
  if (threadIdx.x == 0) out_loss[0] = (float)loss;
}

// out[i][t] = coef[i] * (float)mask[i][t] * *d_loss
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void agg_backward_kernel(const float* __restrict__ d_loss,
                                                                  const float* __restrict__ coef,
                                                                  const M* __restrict__ mask, int64_t cols,
                                                                  int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const float c = coef[row] * d_loss[0];
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float w[4], o[4];
    ldmask4<VEC>(mask, i, valid, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = c * w[e];
    st4<VEC>(out, i, valid, o);
  });
}

// out[i][t] = g[i][t] * coef[i] * *d_loss * extra
template <bool VEC>
__global__ __launch_bounds__(kRcThreads) void scale_rows_kernel(const float* __restrict__ g,
                                                                const float* __restrict__ coef,
                                                                const float* __restrict__ d_loss, float extra,
                                                                int64_t cols, int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const float c = coef[row] * d_loss[0] * extra;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float x[4];
    ld4<VEC>(g, i, valid, x);
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] *= c;
    st4<VEC>(out, i, valid, x);
  });
}

// =============================================================================================
// policy loss (compute_policy_loss_vanilla, core_algos.py:1159-1250)
// =============================================================================================
struct PolicyParams {
  float ratio_lo, ratio_hi, clip_c;  // 1 - clip_low, 1 + clip_high, dual-clip constant
  int token_mean;
};

template <bool VEC, class M, bool GRAD, bool ISW>
__global__ __launch_bounds__(kRcThreads) void policy_partial_kernel(
    const float* __restrict__ old_lp, const float* __restrict__ lp, const float* __restrict__ adv,
    const M* __restrict__ mask, const float* __restrict__ isw, int64_t cols, int chunks, PolicyParams pp,
    double* __restrict__ partials, float* __restrict__ grad) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  float s_loss = 0, s_m = 0, s_kl = 0, s_cf = 0, s_cfl = 0;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float o[4], n[4], a[4], w[4], iw[4], g[4];
    ld4<VEC>(old_lp, i, valid, o);
    ld4<VEC>(lp, i, valid, n);
    ld4<VEC>(adv, i, valid, a);
    ldmask4<VEC>(mask, i, valid, w);
    if (ISW) ld4<VEC>(isw, i, valid, iw);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float d = n[e] - o[e];
      const float k = fminf(fmaxf(d, -20.f), 20.f);
      const float r = expf(k);
      const float l1 = -a[e] * r;
      const float rc = fminf(fmaxf(r, pp.ratio_lo), pp.ratio_hi);
      const float l2 = -a[e] * rc;
      const float c1 = fmaxf(l1, l2);
      const float l3 = -a[e] * pp.clip_c;
      const bool neg = a[e] < 0.f;
      float loss = neg ? fminf(l3, c1) : c1;
      if (ISW) loss *= iw[e];
      const bool in = w[e] != 0.f;
      const float we = w[e];
      if (e < valid) {
        s_loss += ((pp.token_mean && !in) ? 0.f : loss) * we;
        s_m += we;
        s_kl += in ? -k * we : 0.f;
        s_cf += (in && l2 > l1) ? we : 0.f;
        s_cfl += (in && c1 > l3 && neg) ? we : 0.f;
      }
      if (GRAD) {
        // autograd of maximum / minimum / clamp as PyTorch defines them (ties split 50/50,
        // clamp passes the gradient on its closed interval)
        const float in_k = (d >= -20.f && d <= 20.f) ? 1.f : 0.f;
        const float in_clip = (r >= pp.ratio_lo && r <= pp.ratio_hi) ? 1.f : 0.f;
        const float g1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
        const float g2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
        float dc1 = (g1 + g2 * in_clip) * (-a[e] * r) * in_k;
        if (neg) dc1 *= c1 < l3 ? 1.f : (c1 == l3 ? 0.5f : 0.f);
        if (ISW) dc1 *= iw[e];
        g[e] = dc1 * we;
      }
    }
    if (GRAD) st4<VEC>(grad, i, valid, g);
  });
  __shared__ double smem[20];
  double acc[5] = {s_loss, s_m, s_kl, s_cf, s_cfl};
  block_sum<5, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    double* p = partials + (int64_t)blockIdx.x * 5;
#pragma unroll
    for (int i = 0; i < 5; ++i) p[i] = acc[i];
  }
}

__global__ __launch_bounds__(kRcThreads) void policy_finalize_kernel(const double* __restrict__ partials,
                                                                     int64_t rows, int chunks, int64_t cols,
                                                                     AggParams ap, float* __restrict__ out,
                                                                     float* __restrict__ coef) {
  __shared__ double smem[(5 + 3) * 4];
  double loss, msum, extra[3];
  finalize_agg<5>(partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
  if (threadIdx.x == 0) {
    const float denom = (float)msum + 1e-8f;  // masked_mean's denominator
    out[0] = (float)loss;
    out[1] = (float)extra[1] / denom;  // pg_clipfrac
    out[2] = (float)extra[0] / denom;  // ppo_kl
    out[3] = (float)extra[2] / denom;  // pg_clipfrac_lower
  }
}

// =============================================================================================
// value loss (compute_value_loss, core_algos.py:1799-1838)
// =============================================================================================
template <bool VEC, class M, bool GRAD>
__global__ __launch_bounds__(kRcThreads) void value_partial_kernel(
    const float* __restrict__ vpreds, const float* __restrict__ returns, const float* __restrict__ values,
    const M* __restrict__ mask, int64_t cols, int chunks, float clip, int token_mean,
    double* __restrict__ partials, float* __restrict__ grad) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  float s_loss = 0, s_m = 0, s_cf = 0;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float vp[4], R[4], v[4], w[4], g[4];
    ld4<VEC>(vpreds, i, valid, vp);
    ld4<VEC>(returns, i, valid, R);
    ld4<VEC>(values, i, valid, v);
    ldmask4<VEC>(mask, i, valid, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = v[e] - clip, hi = v[e] + clip;
      const float inner = fminf(vp[e], hi);
      const float vc = fmaxf(inner, lo);
      const float d1 = vp[e] - R[e], d2 = vc - R[e];
      const float e1 = d1 * d1, e2 = d2 * d2;
      const float loss = fmaxf(e1, e2);
      const bool in = w[e] != 0.f;
      if (e < valid) {
        s_loss += ((token_mean && !in) ? 0.f : loss) * w[e];
        s_m += w[e];
        s_cf += (in && e2 > e1) ? w[e] : 0.f;
      }
      if (GRAD) {
        const float a = vp[e] < hi ? 1.f : (vp[e] == hi ? 0.5f : 0.f);
        const float b = inner > lo ? 1.f : (inner == lo ? 0.5f : 0.f);
        const float g1 = e1 > e2 ? 1.f : (e1 == e2 ? 0.5f : 0.f);
        const float g2 = e2 > e1 ? 1.f : (e1 == e2 ? 0.5f : 0.f);
        g[e] = (g1 * 2.f * d1 + g2 * 2.f * d2 * a * b) * w[e];
      }
    }
    if (GRAD) st4<VEC>(grad, i, valid, g);
  });
  __shared__ double smem[12];
  double acc[3] = {s_loss, s_m, s_cf};
  block_sum<3, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    double* p = partials + (int64_t)blockIdx.x * 3;
    p[0] = acc[0]; p[1] = acc[1]; p[2] = acc[2];
  }
}

__global__ __launch_bounds__(kRcThreads) void value_finalize_kernel(const double* __restrict__ partials,
                                                                    int64_t rows, int chunks, int64_t cols,
                                                                    AggParams ap, float* __restrict__ out,
                                                                    float* __restrict__ coef) {
  __shared__ double smem[(3 + 3) * 4];
  double loss, msum, extra[1];
  finalize_agg<3>(partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
  if (threadIdx.x == 0) {
    out[0] = 0.5f * (float)loss;
    out[1] = (float)extra[0] / ((float)msum + 1e-8f);
  }
}

// =============================================================================================
// GRPO
// =============================================================================================
// partial[row][chunk] = sum of rewards (the mask is NOT applied, core_algos.py:303)
template <bool VEC>
__global__ __launch_bounds__(kRcThreads) void rowsum_partial_kernel(const float* __restrict__ x, int64_t cols,
                                                                    int chunks, double* __restrict__ partials) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  float s = 0;
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float v[4];
    ld4<VEC>(x, i, valid, v);
    s += (v[0] + v[1]) + (v[2] + v[3]);
  });
  __shared__ double smem[4];
  double acc[1] = {s};
  block_sum<1, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) partials[blockIdx.x] = acc[0];
}

// scores[i] = (float) sum_c partial[i][c]
__global__ void rowsum_finalize_kernel(const double* __restrict__ partials, int64_t rows, int chunks,
                                       float* __restrict__ scores) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  double s = 0;
  for (int c = 0; c < chunks; ++c) s += partials[r * chunks + c];
  scores[r] = (float)s;
}

// One thread per group: count, mean, std over the group's members in index order.
// std_mode 0: unbiased torch.std (two-pass); 1: sqrt(clamp(var, min=eps)) of group_mean_std.
// Singleton groups get mean 0, std 1 (core_algos.py:314-316, groupwise.py:215-221).
__global__ void group_stats_kernel(const float* __restrict__ scores, const int64_t* __restrict__ gid, int64_t n,
                                   int64_t n_groups, float eps, int std_mode, float* __restrict__ mean,
                                   float* __restrict__ stdv, float* __restrict__ count) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n_groups) return;
  double s = 0;
  int64_t c = 0;
  for (int64_t i = 0; i < n; ++i)
    if (gid[i] == g) {
      s += scores[i];
      ++c;
    }
  float mu = 0.f, sd = 1.f;
  if (c > 1) {
    const double m = s / (double)c;
    double q = 0;
    for (int64_t i = 0; i < n; ++i)
      if (gid[i] == g) {
        const double d = (double)scores[i] - m;
        q += d * d;
      }
    const double var = q / (double)(c - 1);
    mu = (float)m;
    sd = std_mode == 0 ? (float)sqrt(var) : sqrtf(fmaxf((float)var, eps));
  }
  mean[g] = mu;
  stdv[g] = sd;
  if (count) count[g] = (float)c;
}

// scalars[i] = (score - mean_g) / (std_g + eps)   or   score - mean_g
__global__ void grpo_scalars_kernel(const float* __restrict__ scores, const int64_t* __restrict__ gid, int64_t n,
                                    const float* __restrict__ mean, const float* __restrict__ stdv, float eps,
                                    int norm_by_std, float* __restrict__ scalars) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t g = gid[i];
  const float c = scores[i] - mean[g];
  scalars[i] = norm_by_std ? c / (stdv[g] + eps) : c;
}

// adv[i][t] = scalars[i] * (float)mask[i][t]
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void broadcast_rows_kernel(const float* __restrict__ scalars,
                                                                    const M* __restrict__ mask, int64_t cols,
                                                                    int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const float a = scalars[row];
  for_each_group(row, chunk, cols, [&](int64_t i, int valid) {
    float w[4], o[4];
    ldmask4<VEC>(mask, i, valid, w);
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = a * w[e];
    st4<VEC>(out, i, valid, o);
  });
}

int launch_moments_finalize(const double* partials, int64_t rows, int chunks, int per_row, double* out,
                            hipStream_t stream) {
  const unsigned grid = per_row ? (unsigned)((rows + kRcThreads - 1) / kRcThreads) : 1u;
  hipLaunchKernelGGL(moments_finalize_kernel, dim3(grid), dim3(kRcThreads), 0, stream, partials, rows, chunks,
                     per_row, out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

static int check_matrix(const char* what, int64_t rows, int64_t cols) {
  VAMD_REQUIRE(rows > 0 && cols > 0, "%s: empty input (%lld x %lld)", what, (long long)rows, (long long)cols);
  VAMD_REQUIRE(rows * chunks_of(cols) < (1ll << 31), "%s: too many workgroups", what);
  return VAMD_OK;
}

static AggParams make_agg(int mode, double dp, double bnt, double gbs, double lsf) {
  AggParams a;
  a.mode = mode;
  a.dp_size = dp;
  a.batch_num_tokens = bnt;
  a.global_batch_size = gbs;
  a.loss_scale_factor = lsf;
  return a;
}

}  // namespace vamd

using namespace vamd;

#define VAMD_VEC_DISPATCH(vec, V, ...) \
  if (vec) { constexpr bool V = true; __VA_ARGS__; } else { constexpr bool V = false; __VA_ARGS__; }

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_masked_moments_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return align_up((size_t)rows * chunks_of(cols) * 4 * sizeof(double), 256);
}

extern "C" int vamd_masked_moments(const float* values, const void* mask, int mask_dtype, int64_t rows,
                                   int64_t cols, int per_row, double* out, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  int st = check_matrix("masked_moments", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(values && mask && out, "masked_moments: null pointer");
  if (!workspace || workspace_bytes < vamd_masked_moments_workspace_bytes(rows, cols)) {
    set_error("masked_moments: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  double* partials = static_cast<double*>(workspace);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {values}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((moments_kernel<V, M>), dim3((unsigned)(rows * chunks)),
                                                 dim3(kRcThreads), 0, s, values, static_cast<const M*>(mask), cols,
                                                 chunks, partials));
  });
  VAMD_LAUNCH_CHECK();
  return launch_moments_finalize(partials, rows, chunks, per_row, out, s);
}

extern "C" int vamd_whiten_stats(const double* moments, int shift_mean, float* stats, void* stream) {
  VAMD_REQUIRE(moments && stats, "whiten_stats: null pointer");
  hipLaunchKernelGGL(whiten_stats_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), moments,
                     shift_mean, stats);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_affine_by_stats(const float* values, const float* stats, int64_t n, float* out, void* stream) {
  VAMD_REQUIRE(values && stats && out && n > 0, "affine_by_stats: bad argument");
  const int vec = (n % 4 == 0) && aligned_to(values, 16) && aligned_to(out, 16);
  int64_t blocks = (n + kRcThreads * 16 - 1) / (kRcThreads * 16);
  if (blocks < 1) blocks = 1;
  if (blocks > 65535 * 16) blocks = 65535 * 16;
  hipLaunchKernelGGL(affine_kernel, dim3((unsigned)blocks), dim3(kRcThreads), 0, static_cast<hipStream_t>(stream),
                     values, stats, n, out, vec);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_agg_loss_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return align_up((size_t)rows * chunks_of(cols) * 2 * sizeof(double), 256);
}

extern "C" int vamd_agg_loss_forward(const float* loss_mat, const void* mask, int mask_dtype, int64_t rows,
                                     int64_t cols, int mode, double dp_size, double batch_num_tokens,
                                     double global_batch_size, double loss_scale_factor, float* out_loss,
                                     float* coef_out, void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_matrix("agg_loss", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(loss_mat && mask && out_loss, "agg_loss: null pointer");
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "agg_loss: invalid mode %d", mode);
  if (!workspace || workspace_bytes < vamd_agg_loss_workspace_bytes(rows, cols)) {
    set_error("agg_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  double* partials = static_cast<double*>(workspace);
  const int token_mean = mode == VAMD_AGG_TOKEN_MEAN;
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {loss_mat}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((agg_partial_kernel<V, M>), dim3((unsigned)(rows * chunks)),
                                                 dim3(kRcThreads), 0, s, loss_mat, static_cast<const M*>(mask),
                                                 cols, chunks, token_mean, partials));
  });
  VAMD_LAUNCH_CHECK();
  hipLaunchKernelGGL(agg_finalize_kernel, dim3(1), dim3(kRcThreads), 0, s, partials, rows, chunks, cols,
                     make_agg(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor), out_loss,
                     coef_out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_agg_loss_backward(const float* d_loss, const float* coef, const void* mask, int mask_dtype,
                                      int64_t rows, int64_t cols, float* d_loss_mat, void* stream) {
  int st = check_matrix("agg_loss_backward", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(d_loss && coef && mask && d_loss_mat, "agg_loss_backward: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {d_loss_mat}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((agg_backward_kernel<V, M>), dim3((unsigned)(rows * chunks)),
                                                 dim3(kRcThreads), 0, s, d_loss, coef,
                                                 static_cast<const M*>(mask), cols, chunks, d_loss_mat));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_scale_rows(const float* g, const float* coef, const float* d_loss, float extra_scale,
                               int64_t rows, int64_t cols, float* out, void* stream) {
  int st = check_matrix("scale_rows", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(g && coef && d_loss && out, "scale_rows: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  const bool vec = can_vectorize(cols, {g, out}, nullptr, 0);
  VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((scale_rows_kernel<V>), dim3((unsigned)(rows * chunks)),
                                               dim3(kRcThreads), 0, s, g, coef, d_loss, extra_scale, cols, chunks,
                                               out));
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_policy_loss_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return align_up((size_t)rows * chunks_of(cols) * 5 * sizeof(double), 256);
}

extern "C" int vamd_policy_loss_forward(const float* old_log_prob, const float* log_prob, const float* advantages,
                                        const void* mask, int mask_dtype, const float* is_weights, int64_t rows,
                                        int64_t cols, float clip_low, float clip_high, float clip_c, int mode,
                                        double dp_size, double batch_num_tokens, double global_batch_size,
                                        double loss_scale_factor, float* out, float* grad_unscaled, float* coef_out,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_matrix("policy_loss", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(old_log_prob && log_prob && advantages && mask && out, "policy_loss: null pointer");
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "policy_loss: invalid mode %d", mode);
  VAMD_REQUIRE(clip_c > 1.0f, "policy_loss: clip_ratio_c must be > 1.0, got %f", (double)clip_c);
  VAMD_REQUIRE(!grad_unscaled || coef_out, "policy_loss: grad output needs coef_out");
  if (!workspace || workspace_bytes < vamd_policy_loss_workspace_bytes(rows, cols)) {
    set_error("policy_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  double* partials = static_cast<double*>(workspace);
  PolicyParams pp;
  pp.ratio_lo = (float)(1.0 - (double)clip_low);
  pp.ratio_hi = (float)(1.0 + (double)clip_high);
  pp.clip_c = clip_c;
  pp.token_mean = mode == VAMD_AGG_TOKEN_MEAN;
  const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
#define VAMD_PL(V, G, W)                                                                                     \
  hipLaunchKernelGGL((policy_partial_kernel<V, M, G, W>), grid, block, 0, s, old_log_prob, log_prob, advantages, \
                     mk, is_weights, cols, chunks, pp, partials, grad_unscaled)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {old_log_prob, log_prob, advantages, is_weights, grad_unscaled}, mask,
                                   sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    if (vec) {
      if (grad_unscaled) { if (is_weights) VAMD_PL(true, true, true); else VAMD_PL(true, true, false); }
      else { if (is_weights) VAMD_PL(true, false, true); else VAMD_PL(true, false, false); }
    } else {
      if (grad_unscaled) { if (is_weights) VAMD_PL(false, true, true); else VAMD_PL(false, true, false); }
      else { if (is_weights) VAMD_PL(false, false, true); else VAMD_PL(false, false, false); }
    }
  });
#undef VAMD_PL
  VAMD_LAUNCH_CHECK();
  hipLaunchKernelGGL(policy_finalize_kernel, dim3(1), dim3(kRcThreads), 0, s, partials, rows, chunks, cols,
                     make_agg(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor), out, coef_out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_value_loss_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return align_up((size_t)rows * chunks_of(cols) * 3 * sizeof(double), 256);
}

extern "C" int vamd_value_loss_forward(const float* vpreds, const float* returns, const float* values,
                                       const void* mask, int mask_dtype, int64_t rows, int64_t cols,
                                       float cliprange_value, int mode, float* out, float* grad_unscaled,
                                       float* coef_out, void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_matrix("value_loss", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(vpreds && returns && values && mask && out, "value_loss: null pointer");
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "value_loss: invalid mode %d", mode);
  VAMD_REQUIRE(!grad_unscaled || coef_out, "value_loss: grad output needs coef_out");
  if (!workspace || workspace_bytes < vamd_value_loss_workspace_bytes(rows, cols)) {
    set_error("value_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  double* partials = static_cast<double*>(workspace);
  const int token_mean = mode == VAMD_AGG_TOKEN_MEAN;
  const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
#define VAMD_VL(V, G)                                                                                       \
  hipLaunchKernelGGL((value_partial_kernel<V, M, G>), grid, block, 0, s, vpreds, returns, values, mk, cols, \
                     chunks, cliprange_value, token_mean, partials, grad_unscaled)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {vpreds, returns, values, grad_unscaled}, mask, sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    if (vec) { if (grad_unscaled) VAMD_VL(true, true); else VAMD_VL(true, false); }
    else { if (grad_unscaled) VAMD_VL(false, true); else VAMD_VL(false, false); }
  });
#undef VAMD_VL
  VAMD_LAUNCH_CHECK();
  hipLaunchKernelGGL(value_finalize_kernel, dim3(1), dim3(kRcThreads), 0, s, partials, rows, chunks, cols,
                     make_agg(mode, 1.0, -1.0, -1.0, -1.0), out, coef_out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_grpo_workspace_bytes(int64_t batch, int64_t length, int64_t n_groups) {
  if (batch <= 0 || length <= 0 || n_groups <= 0) return 0;
  size_t b = align_up((size_t)batch * chunks_of(length) * sizeof(double), 256);
  b += 2 * align_up((size_t)batch * sizeof(float), 256);     // scores, scalars
  b += 2 * align_up((size_t)n_groups * sizeof(float), 256);  // mean, std
  return b;
}

extern "C" int vamd_group_mean_std(const float* scores, const int64_t* group_ids, int64_t n, int64_t n_groups,
                                   float eps, float* mean, float* std, float* count, void* stream) {
  VAMD_REQUIRE(scores && group_ids && mean && std && n > 0 && n_groups > 0, "group_mean_std: bad argument");
  hipLaunchKernelGGL(group_stats_kernel, dim3((unsigned)((n_groups + 63) / 64)), dim3(64), 0,
                     static_cast<hipStream_t>(stream), scores, group_ids, n, n_groups, eps, 1, mean, std, count);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_grpo_advantage(const float* rewards, const void* mask, int mask_dtype, const int64_t* group_ids,
                                   int64_t batch, int64_t length, int64_t n_groups, float epsilon, int norm_by_std,
                                   int std_mode, float* advantages, float* scores_out, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  int st = check_matrix("grpo", batch, length);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(rewards && mask && group_ids && advantages && n_groups > 0, "grpo: bad argument");
  if (!workspace || workspace_bytes < vamd_grpo_workspace_bytes(batch, length, n_groups)) {
    set_error("grpo: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(length);
  Carver carve(workspace);
  double* partials = carve.take<double>((size_t)batch * chunks);
  float* scores = carve.take<float>((size_t)batch);
  float* scalars = carve.take<float>((size_t)batch);
  float* mean = carve.take<float>((size_t)n_groups);
  float* stdv = carve.take<float>((size_t)n_groups);
  {
    const bool vec = can_vectorize(length, {rewards}, nullptr, 0);
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((rowsum_partial_kernel<V>), dim3((unsigned)(batch * chunks)),
                                                 dim3(kRcThreads), 0, s, rewards, length, chunks, partials));
    VAMD_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(rowsum_finalize_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, partials, batch,
                     chunks, scores);
  VAMD_LAUNCH_CHECK();
  hipLaunchKernelGGL(group_stats_kernel, dim3((unsigned)((n_groups + 63) / 64)), dim3(64), 0, s, scores, group_ids,
                     batch, n_groups, epsilon, std_mode, mean, stdv, (float*)nullptr);
  VAMD_LAUNCH_CHECK();
  hipLaunchKernelGGL(grpo_scalars_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, scores, group_ids,
                     batch, mean, stdv, epsilon, norm_by_std, scores_out ? scores_out : scalars);
  VAMD_LAUNCH_CHECK();
  const float* sc = scores_out ? scores_out : scalars;
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(length, {advantages}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((broadcast_rows_kernel<V, M>), dim3((unsigned)(batch * chunks)),
                                                 dim3(kRcThreads), 0, s, sc, static_cast<const M*>(mask), length,
                                                 chunks, advantages));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
