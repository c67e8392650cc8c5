// HBM-bound kernels of the PPO / GRPO policy math: masked moments and whitening, agg_loss,
// the clipped + dual-clip policy loss, the clipped value loss, GRPO group-normalised advantages.
// Reference semantics: verl/utils/torch_functional.py:266-339 and
// verl/trainer/ppo/core_algos.py:266-357, :1025-1080, :1159-1250, :1799-1838.
//
// Every reduction is ONE launch: workgroups stream their 4096-column chunk with all loads in
// flight at once, leave a record of double partial sums, and the workgroup that arrives last
// folds the records (in index order) into the outputs.
#include <initializer_list>

#include <type_traits>

#include "rowchunk.h"

namespace vamd {

struct Work {
  unsigned* ticket;  // workspace head: zero on entry, zero on exit
  double* partials;  // NV slots per (row, chunk) workgroup, slot-major (record_at)
  int totals;        // loss kernels built without the fold: take the launch totals here (totals_epilogue)
};

// The loss kernels of a large launch carry no fold of their own (FOLD = false).  Two of the four agg_loss modes,
// token-mean and seq-mean-token-sum-norm, need nothing but the launch totals, and those come cheaply in two
// levels (sum_all_records: a few dozen registers, no per-row pass), so such a launch finishes here; the per-row
// modes leave their records to fold_loss_kernel.  Same formulas as finalize_agg.
template <int NV, int EPI>
__device__ __forceinline__ void totals_epilogue(const Work& wk, int64_t rows, int chunks, int64_t cols,
                                                const AggParams& ap, float* __restrict__ coef,
                                                float* __restrict__ out, double* smem) {
  double tot[NV];
  if (!sum_all_records<NV>(wk.ticket, wk.partials, rows, chunks, tot, smem)) return;
  __shared__ float c_all;
  if (threadIdx.x == 0) {
    double loss, c;
    if (ap.mode == VAMD_AGG_TOKEN_MEAN) {
      const double denom = ap.batch_num_tokens < 0 ? tot[1] : ap.batch_num_tokens;
      loss = tot[0] / denom * ap.dp_size;
      c = ap.dp_size / denom;
    } else {
      const double f = ap.loss_scale_factor < 0 ? (double)cols : ap.loss_scale_factor;
      loss = tot[0] / f;
      c = 1.0 / f;
    }
    double extra[NV > 2 ? NV - 2 : 1] = {};
#pragma unroll
    for (int i = 2; i < NV; ++i) extra[i - 2] = tot[i];
    loss_epilogue<EPI>(loss, tot[1], extra, out);
    c_all = (float)c;
  }
  __syncthreads();
  if (coef)
    for (int64_t r = threadIdx.x; r < rows; r += kRcThreads) coef[r] = c_all;
  ticket_reset(wk.ticket);
}
__host__ __device__ inline bool totals_suffice(int mode) {
  return mode == VAMD_AGG_TOKEN_MEAN || mode == VAMD_AGG_SEQ_MEAN_TOKEN_SUM_NORM;
}

// =============================================================================================
// masked moments
// =============================================================================================
// Where the folded moments go: the four doubles (per row or for the whole launch) and, derived from them in the
// same launch, the fp32 results the callers are after.
struct MomentOuts {
  double* moments;  // [rows][4] or [4]; may be null
  float* sum;       // [rows] or [1]: masked_sum
  float* mean;      // [rows] or [1]: masked_mean = sum / (sum(mask) + 1e-8)
  float* denom;     // [rows] or [1]: sum(mask) + 1e-8 (what the gradient of masked_mean divides by)
  float* whiten;    // [4], whole launch only: mean, rsqrt(var + 1e-8), shift
  int shift_mean;
};
__device__ __forceinline__ void write_moment_outs(const MomentOuts& o, int64_t at, const double (&a)[4]) {
  if (o.moments)
#pragma unroll
    for (int i = 0; i < 4; ++i) o.moments[at * 4 + i] = a[i];
  const float denom = (float)a[0] + 1e-8f;
  if (o.sum) o.sum[at] = (float)a[1];
  if (o.mean) o.mean[at] = (float)a[1] / denom;
  if (o.denom) o.denom[at] = denom;
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void moments_kernel(const float* __restrict__ values,
                                                             const float* __restrict__ minus,
                                                             const M* __restrict__ mask, int64_t rows,
                                                             int64_t cols, int chunks, int span, int per_row, Work wk,
                                                             MomentOuts out) {
  // A workgroup walks `span` consecutive 4096-column chunks of its row and leaves one record (`chunks` counts those
  // spans): at 128 MB per tensor a quarter of the workgroup reductions and records, and few enough records for the
  // last workgroup to fold them itself.
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const bool streaming = streams_past_caches(rows * cols);  // the grid counts spans, not chunks
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  for (int u = 0; u < span; ++u) {
    const ChunkPos pos(row, chunk * span + u, cols);
    float x[kGroups][4], w[kGroups][4];
    load_groups<VEC>(values, pos, x, streaming);
    if (minus) {  // moments of values - minus
      float y[kGroups][4];
      load_groups<VEC>(minus, pos, y, streaming);
#pragma unroll
      for (int g = 0; g < kGroups; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) x[g][e] -= y[g][e];
    }
    load_mask_groups<VEC>(mask, pos, w, streaming);
    float s0 = 0, s1 = 0, s2 = 0, cnt = 0;
#pragma unroll
    for (int g = 0; g < kGroups; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool in = w[g][e] != 0.f;
        const float v = in ? x[g][e] : 0.f;  // where(mask.bool(), values, 0)
        s0 += w[g][e];
        s1 += v * w[g][e];
        s2 += v * v * w[g][e];
        cnt += in ? 1.f : 0.f;
      }
    acc[0] += (double)s0;
    acc[1] += (double)s1;
    acc[2] += (double)s2;
    acc[3] += (double)cnt;
  }
  __shared__ double smem[16];
  block_sum<4, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<4>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if (!per_row) {
    double a[4];
    if (!sum_all_records<4>(wk.ticket, wk.partials, rows, chunks, a, smem)) return;
    if (threadIdx.x == 0) {
      write_moment_outs(out, 0, a);
      if (out.whiten) whiten_stats_from_moments(a[0], a[1], a[2], out.shift_mean, out.whiten);
    }
    ticket_reset(wk.ticket);
    return;
  }
  if (!last_block_arrives(wk.ticket)) return;
  {
    for (int64_t r0 = threadIdx.x; r0 < rows; r0 += 2 * kRcThreads) {
      const int64_t rr[2] = {r0, r0 + kRcThreads};
      const bool have[2] = {true, rr[1] < rows};
      double a[2][4];
      fold_row_records<4, 4, 2>(wk.partials, rr, have, rows, chunks, a);
#pragma unroll
      for (int k = 0; k < 2; ++k)
        if (have[k]) write_moment_outs(out, rr[k], a[k]);
    }
  }
  ticket_reset(wk.ticket);
}

__global__ void whiten_stats_kernel(const double* __restrict__ mom, int shift_mean, float* __restrict__ stats) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  whiten_stats_from_moments(mom[0], mom[1], mom[2], shift_mean, stats);
}

template <bool VEC>
__global__ __launch_bounds__(kRcThreads) void affine_kernel(const float* __restrict__ values,
                                                            const float* __restrict__ stats, int64_t n,
                                                            float* __restrict__ out) {
  const float mean = stats[0], rstd = stats[1], shift = stats[2];
  const ChunkPos pos(0, blockIdx.x, n);  // the flat array as one long row
  float x[kGroups][4];
  load_groups<VEC>(values, pos, x);
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) x[g][e] = (x[g][e] - mean) * rstd + shift;
  store_groups<VEC>(out, pos, x);
}

// out = ((v - mean) * rstd + shift) * mask
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void affine_masked_kernel(const float* __restrict__ values,
                                                                   const float* __restrict__ stats,
                                                                   const M* __restrict__ mask, int64_t n,
                                                                   float* __restrict__ out) {
  const float mean = stats[0], rstd = stats[1], shift = stats[2];
  const ChunkPos pos(0, blockIdx.x, n);
  float x[kGroups][4], w[kGroups][4];
  load_groups<VEC>(values, pos, x);
  load_mask_groups<VEC>(mask, pos, w);
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) x[g][e] = ((x[g][e] - mean) * rstd + shift) * w[g][e];
  store_groups<VEC>(out, pos, x);
}

// =============================================================================================
// agg_loss forward / backward
// =============================================================================================
template <bool VEC, class M, bool FOLD>
__global__ __launch_bounds__(kRcThreads) void agg_kernel(const float* __restrict__ loss_mat,
                                                         const M* __restrict__ mask, int64_t rows, int64_t cols,
                                                         int chunks, AggParams ap, Work wk,
                                                         float* __restrict__ out_loss, float* __restrict__ coef) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float x[kGroups][4], w[kGroups][4];
  load_groups<VEC>(loss_mat, pos, x);
  load_mask_groups<VEC>(mask, pos, w);
  const bool token_mean = ap.mode == VAMD_AGG_TOKEN_MEAN;
  float s = 0, m = 0;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // token-mean goes through masked_sum (where() first); the seq-* modes multiply directly
      const float v = (token_mean && w[g][e] == 0.f) ? 0.f : x[g][e];
      if (e < pos.valid[g]) s += v * w[g][e];
      m += w[g][e];
    }
  __shared__ double smem[(2 + 3) * 4];
  double acc[2] = {s, m};
  block_sum<2, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<2>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if constexpr (FOLD) {
    if (totals_suffice(ap.mode)) {  // no per-row pass: the launch totals are all these modes need
      totals_epilogue<2, kEpiAgg>(wk, rows, chunks, cols, ap, coef, out_loss, smem);
      return;
    }
    if (!last_block_arrives(wk.ticket)) return;
    double loss, msum, extra[1];
    finalize_agg<2>(wk.partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
    if (threadIdx.x == 0) loss_epilogue<kEpiAgg>(loss, msum, extra, out_loss);
    ticket_reset(wk.ticket);
  } else {
    if (wk.totals) totals_epilogue<2, kEpiAgg>(wk, rows, chunks, cols, ap, coef, out_loss, smem);
  }
}

// out[i][t] = coef[i] * (float)mask[i][t] * *d_loss
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void agg_backward_kernel(const float* __restrict__ d_loss,
                                                                  const float* __restrict__ coef,
                                                                  const M* __restrict__ mask, int64_t cols,
                                                                  int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float w[kGroups][4];
  load_mask_groups<VEC>(mask, pos, w);
  const float c = coef[row] * d_loss[0];
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) w[g][e] *= c;
  store_groups<VEC>(out, pos, w);
}

// out[i][t] = g[i][t] * coef[i] * *d_loss * extra
template <bool VEC>
__global__ __launch_bounds__(kRcThreads) void scale_rows_kernel(const float* __restrict__ g,
                                                                const float* __restrict__ coef,
                                                                const float* __restrict__ d_loss, float extra,
                                                                int64_t cols, int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float x[kGroups][4];
  load_groups<VEC>(g, pos, x);
  const float c = coef[row] * d_loss[0] * extra;
#pragma unroll
  for (int k = 0; k < kGroups; ++k)
#pragma unroll
    for (int e = 0; e < 4; ++e) x[k][e] *= c;
  store_groups<VEC>(out, pos, x);
}

// =============================================================================================
// policy loss (compute_policy_loss_vanilla, core_algos.py:1159-1250)
// =============================================================================================
constexpr int kRowSyncChunks = 32;            // chunks of one row whose workgroups wait for each other (131072 columns)
constexpr unsigned kRowWaitSpins = 1u << 16;  // polls of about a microsecond; the neighbours normally arrive within a few
struct PolicyParams {
  float ratio_lo, ratio_hi, clip_c;  // 1 - clip_low, 1 + clip_high, dual-clip constant
  int variant;                       // VAMD_PL_*
  float tau_pos, tau_neg;            // SAPO gate temperatures
  const double* row_moments;         // GSPO: [rows][4], slot 0 = sum(m), slot 1 = sum((lp - old) m)
                                     // GEO_MEAN: [rows][chunks][4] partial sums of geo_rows_kernel
  float nkl_lo, nkl_hi;              // GEO_MEAN: clip range of the log-ratio, (-clip_low, +clip_high)
  double* row_partials;              // ROWS kernels: [rows][chunks][4] partial row sums, exchanged inside the launch
  unsigned spin_limit;               // ROWS kernels: polls a workgroup spends on its row's other chunks
};

// Per-token loss, its derivative with respect to log_prob and the metric contributions of the
// policy-loss variants (autograd conventions of PyTorch: maximum / minimum split ties 50/50,
// clamp passes the gradient on its closed interval, detached factors carry none).
//   VANILLA  clipped + dual-clip PPO                         core_algos.py:1159-1250
//   GPG      -log_prob A                                     :1414-1447
//   CISPO    -sg(clip(ratio)) A log_prob                     :1721-1779
//   SAPO     -4/tau sigmoid(tau (ratio - 1)) A               :1329-1411
//   GSPO     clipped objective on the sequence-level ratio   :1253-1326
//   REINFORCE  -log_prob A, KL metric against the rollout policy (compute_policy_loss_reinforce) :1984-2061
//   GEO_MEAN   -A_seq exp(mean_t clipped log-ratio) per sequence (GMPO)           :1635-1718
struct TokenLoss {
  float loss, dloss, kl, cf, cfl;  // kl: -(clamped or raw) log-ratio; cf / cfl: 1 where the clip counters fire
};

// VARIANT >= 0 fixes the variant at compile time: the per-token code is then straight-line and the 16 tokens of a
// thread interleave; VARIANT = -1 reads it from pp (one branch per token, every variant's code in the kernel).
template <int VARIANT>
__device__ __forceinline__ TokenLoss token_loss(const PolicyParams& pp, float old, float lp, float A, float seq_lr) {
  const int variant = VARIANT >= 0 ? VARIANT : pp.variant;
  TokenLoss t;
  t.cf = 0.f;
  t.cfl = 0.f;
  const float d = lp - old;
  const float k = fminf(fmaxf(d, -20.f), 20.f);
  const float in_k = (d >= -20.f && d <= 20.f) ? 1.f : 0.f;
  t.kl = -k;
  switch (variant) {
    case VAMD_PL_GPG:
      t.loss = -lp * A;
      t.dloss = -A;
      t.kl = 0.f;
      break;
    case VAMD_PL_REINFORCE:
      t.loss = -lp * A;
      t.dloss = -A;
      t.kl = -d;
      break;
    case VAMD_PL_GEO_MEAN: {
      // seq_lr carries q = -(A_seq ratio_seq w_seq) / (M + 1e-8): every valid token of the row holds the loss q
      // (their sum is the sequence loss), and d loss / d log_prob is q where the token's log-ratio enters the
      // geometric mean unclipped
      // written with & and | on purpose: short-circuit forms became a branch per token
      const bool up = A > 0.f, down = A < 0.f;
      const bool above = d > pp.nkl_hi, below = d < pp.nkl_lo;  // outside the clip range (d != clamp(d))
      const bool passes = (up & !above) | (down & !below);
      t.loss = seq_lr;
      t.dloss = passes ? seq_lr : 0.f;
      t.kl = -d;
      t.cf = (up & (above | below)) ? 1.f : 0.f;
      t.cfl = (down & (above | below)) ? 1.f : 0.f;
    } break;
    case VAMD_PL_CISPO: {
      const float r = expf(k);
      const float rc = fminf(fmaxf(r, pp.ratio_lo), pp.ratio_hi);
      t.loss = -rc * A * lp;
      t.dloss = -rc * A;
      t.cf = r != rc ? 1.f : 0.f;
    } break;
    case VAMD_PL_SAPO: {
      const float r = expf(k);
      const float tau = A > 0.f ? pp.tau_pos : pp.tau_neg;
      const float sg = 1.f / (1.f + expf(-tau * (r - 1.f)));
      t.loss = -(sg * (4.f / tau)) * A;
      t.dloss = -A * 4.f * sg * (1.f - sg) * r * in_k;
    } break;
    case VAMD_PL_GSPO: {
      const float lr = fminf(seq_lr, 10.f);
      const float pass = seq_lr <= 10.f ? 1.f : 0.f;
      const float r = expf(lr);
      const float l1 = -A * r;
      const float rc = fminf(fmaxf(r, pp.ratio_lo), pp.ratio_hi);
      const float l2 = -A * rc;
      t.loss = fmaxf(l1, l2);
      const float in_clip = (r >= pp.ratio_lo && r <= pp.ratio_hi) ? 1.f : 0.f;
      const float g1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
      const float g2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
      t.dloss = (g1 + g2 * in_clip) * (-A * r) * pass;
      t.cf = l2 > l1 ? 1.f : 0.f;
      t.kl = -d;  // the metric uses the unclamped log-ratio (:1317)
    } break;
    default: {
      const float r = expf(k);
      const float l1 = -A * r;
      const float rc = fminf(fmaxf(r, pp.ratio_lo), pp.ratio_hi);
      const float l2 = -A * rc;
      const float c1 = fmaxf(l1, l2);
      const float l3 = -A * pp.clip_c;
      const bool neg = A < 0.f;
      t.loss = neg ? fminf(l3, c1) : c1;
      t.cf = l2 > l1 ? 1.f : 0.f;
      t.cfl = (c1 > l3 && neg) ? 1.f : 0.f;
      const float in_clip = (r >= pp.ratio_lo && r <= pp.ratio_hi) ? 1.f : 0.f;
      const float g1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
      const float g2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
      float dc1 = (g1 + g2 * in_clip) * (-A * r) * in_k;
      if (neg) dc1 *= c1 < l3 ? 1.f : (c1 == l3 ? 0.5f : 0.f);
      t.dloss = dc1;
    } break;
  }
  return t;
}

// f(std::integral_constant<int, variant>): for a kernel built with the variant fixed, that variant; otherwise the
// runtime one, so that the caller's token loop exists once per variant instead of switching per token.
template <int VARIANT, class F>
__device__ __forceinline__ void with_policy_variant(int variant, F&& f) {
  if constexpr (VARIANT >= 0) {
    f(std::integral_constant<int, VARIANT>());
  } else {
    switch (variant) {
      case VAMD_PL_GPG: f(std::integral_constant<int, VAMD_PL_GPG>()); break;
      case VAMD_PL_CISPO: f(std::integral_constant<int, VAMD_PL_CISPO>()); break;
      case VAMD_PL_SAPO: f(std::integral_constant<int, VAMD_PL_SAPO>()); break;
      case VAMD_PL_GSPO: f(std::integral_constant<int, VAMD_PL_GSPO>()); break;
      case VAMD_PL_REINFORCE: f(std::integral_constant<int, VAMD_PL_REINFORCE>()); break;
      case VAMD_PL_GEO_MEAN: f(std::integral_constant<int, VAMD_PL_GEO_MEAN>()); break;
      default: f(std::integral_constant<int, VAMD_PL_VANILLA>()); break;
    }
  }
}

// The per-sequence quantity of the two losses that need one before their per-token pass, as four partial sums over
// one chunk of the row (fp32 over a thread's 16 tokens; the caller widens and reduces them):
//   GSPO (core_algos.py:1286-1294)      sum(m), sum((lp - old) m), 0, 0
//   GEO_MEAN (core_algos.py:1683-1704)  sum(m), sum(k m), sum(A m), sum(log(is_weight + 1e-10) m)
//                                       with k the log-ratio clipped on the side its advantage's sign names
// One function for whoever computes them -- the row pre-pass kernel, the loss kernel for its own chunk, a loss
// workgroup that has to stand in for a neighbour -- so that all arrive at the same bits.
template <bool ISW>
__device__ __forceinline__ void row_presums(int variant, const ChunkPos& pos, const float (&o)[kGroups][4],
                                            const float (&n)[kGroups][4], const float (&a)[kGroups][4],
                                            const float (&w)[kGroups][4], const float (&iw)[kGroups][4], float lo,
                                            float hi, double (&acc)[4]) {
  float s_m = 0, s_k = 0, s_a = 0, s_w = 0;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // elements past the end of the row were loaded as zeros with weight zero: they add nothing, and leaving the
      // test out keeps the sixteen tokens of a thread free of branches
      const float d = n[g][e] - o[g][e];
      const float we = w[g][e];
      s_m += we;
      if (variant == VAMD_PL_GSPO) {
        s_k += (we != 0.f ? d : 0.f) * we;  // where(mask, lp - old, 0) * mask
      } else {
        // min(d, clamp(d, lo, hi)) is min(d, hi) and max(d, clamp(d, lo, hi)) is max(d, lo) (lo <= hi)
        const float A = a[g][e];
        const float k = A > 0.f ? fminf(d, hi) : (A < 0.f ? fmaxf(d, lo) : 0.f);
        s_k += k * we;
        s_a += A * we;
        if (ISW) s_w += logf(iw[g][e] + 1e-10f) * we;
      }
    }
  acc[0] = s_m;
  acc[1] = s_k;
  acc[2] = s_a;
  acc[3] = s_w;
}

// Row pre-pass as a launch of its own (GMPO where the loss kernel cannot exchange the sums itself): per (row, chunk)
// the four partial sums.
template <bool VEC, class M, bool ISW>
__global__ __launch_bounds__(kRcThreads) void geo_rows_kernel(const float* __restrict__ old_lp,
                                                              const float* __restrict__ lp,
                                                              const float* __restrict__ adv,
                                                              const M* __restrict__ mask,
                                                              const float* __restrict__ isw, int64_t cols, int chunks,
                                                              float lo, float hi, double* __restrict__ partials) {
  const int64_t row = blockIdx.x / chunks;
  const ChunkPos pos(row, blockIdx.x % chunks, cols);
  float o[kGroups][4], n[kGroups][4], a[kGroups][4], w[kGroups][4], iw[kGroups][4];
  load_groups<VEC>(old_lp, pos, o);
  load_groups<VEC>(lp, pos, n);
  load_groups<VEC>(adv, pos, a);
  load_mask_groups<VEC>(mask, pos, w);
  if (ISW) load_groups<VEC>(isw, pos, iw);
  __shared__ double smem[4 * 4];
  double acc[4];
  row_presums<ISW>(VAMD_PL_GEO_MEAN, pos, o, n, a, w, iw, lo, hi, acc);
  block_sum<4, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    double* p = partials + (int64_t)blockIdx.x * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = acc[i];
  }
}

// ROWS: the kernel works out the per-sequence quantity of GSPO / GMPO itself instead of taking it from a pre-pass.
// Every workgroup reduces the four partial sums of its own chunk from the values it holds in registers anyway; with
// one chunk per row that is all.  With several, it leaves them in pp.row_partials, sets the ready byte of its
// (row, chunk) and waits -- a bounded number of polls -- for the bytes of the row's other chunks, whose workgroups
// have the neighbouring ids and start together with it.  A workgroup whose wait ran out computes the missing chunks'
// sums itself, to the same bits, so the result does not depend on what the device lets run at the same time.  The
// launch's last workgroup clears the ready bytes (ROWS launches always fold their own records).
template <bool VEC, class M, bool GRAD, bool ISW, bool FOLD, int VARIANT, bool ROWS = false>
__global__ __launch_bounds__(kRcThreads) void policy_kernel(
    const float* __restrict__ old_lp, const float* __restrict__ lp, const float* __restrict__ adv,
    const M* __restrict__ mask, const float* __restrict__ isw, int64_t rows, int64_t cols, int chunks,
    PolicyParams pp, AggParams ap, Work wk, float* __restrict__ out, float* __restrict__ grad,
    float* __restrict__ coef) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float o[kGroups][4], n[kGroups][4], a[kGroups][4], w[kGroups][4], iw[kGroups][4], gr[kGroups][4];
  load_groups<VEC>(old_lp, pos, o);
  load_groups<VEC>(lp, pos, n);
  load_groups<VEC>(adv, pos, a);
  load_mask_groups<VEC>(mask, pos, w);
  if (ISW) load_groups<VEC>(isw, pos, iw);
  const bool token_mean = ap.mode == VAMD_AGG_TOKEN_MEAN;
  float seq_lr = 0.f;
  const int variant = VARIANT >= 0 ? VARIANT : pp.variant;
  __shared__ double smem[(5 + 3) * 4];
  double r[4] = {0, 0, 0, 0};  // the row's four sums (GSPO, GEO_MEAN)
  if constexpr (ROWS) {
    __shared__ double row_sums[4];
    double own[4];
    row_presums<ISW>(variant, pos, o, n, a, w, iw, pp.nkl_lo, pp.nkl_hi, own);
    block_sum<4, kRcThreads>(own, smem);  // valid in thread 0
    bool open = true;
    if (chunks > 1) {
      if (threadIdx.x == 0) {
        double* mine = pp.row_partials + (row * chunks + chunk) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) peer_store(mine + i, own[i]);
        ready_byte_set(wk.ticket, row * chunks + chunk);
      }
      bool ready = true;
      unsigned polls = 0;
      if ((int)threadIdx.x < chunks && (int)threadIdx.x != chunk)
        ready = ready_byte_wait(wk.ticket, row * chunks + threadIdx.x, polls, pp.spin_limit);
      open = __syncthreads_and(ready) != 0;
      if (!open && threadIdx.x == 0) note_gave_up(wk.ticket);
    }
    if (open) {
      if (threadIdx.x == 0) {
        for (int c = 0; c < chunks; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            r[i] += c == chunk ? own[i] : peer_load(pp.row_partials + (row * chunks + c) * 4 + i);
      }
    } else {
      for (int c = 0; c < chunks; ++c) {  // uniform over the workgroup
        double part[4];
        if (c != chunk) {
          const ChunkPos p2(row, c, cols);
          float o2[kGroups][4], n2[kGroups][4], a2[kGroups][4], w2[kGroups][4], iw2[kGroups][4];
          load_groups<VEC>(old_lp, p2, o2);
          load_groups<VEC>(lp, p2, n2);
          load_groups<VEC>(adv, p2, a2);
          load_mask_groups<VEC>(mask, p2, w2);
          if (ISW) load_groups<VEC>(isw, p2, iw2);
          row_presums<ISW>(variant, p2, o2, n2, a2, w2, iw2, pp.nkl_lo, pp.nkl_hi, part);
          block_sum<4, kRcThreads>(part, smem);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] += c == chunk ? own[i] : part[i];  // thread 0's are the sums
      }
    }
    if (threadIdx.x == 0)
#pragma unroll
      for (int i = 0; i < 4; ++i) row_sums[i] = r[i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = row_sums[i];
  } else {
    if (variant == VAMD_PL_GSPO) {
      r[0] = pp.row_moments[row * 4];
      r[1] = pp.row_moments[row * 4 + 1];
    }
    if (variant == VAMD_PL_GEO_MEAN)
      for (int c = 0; c < chunks; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] += pp.row_moments[(row * chunks + c) * 4 + i];
  }
  if (variant == VAMD_PL_GSPO)  // sum((lp - old) m) / clamp(sum(m), min = 1)
    seq_lr = (float)r[1] / fmaxf((float)r[0], 1.f);
  if (variant == VAMD_PL_GEO_MEAN) {
    const float den = (float)r[0] + 1e-8f;
    const float ratio = expf((float)r[1] / den);
    const float a_seq = (float)r[2] / den;
    const float w_seq = expf((float)r[3] / den);  // 1 when no importance weights were given (sum of logs = 0)
    seq_lr = -a_seq * ratio * w_seq / den;
  }
  // GMPO's importance weights enter through the sequence weight above, not token by token
  const bool isw_per_token = ISW && variant != VAMD_PL_GEO_MEAN;
  float s_loss = 0, s_m = 0, s_kl = 0, s_cf = 0, s_cfl = 0;
  // a kernel built for every variant (VARIANT = -1) picks the variant once, here, and runs that variant's copy of
  // the token loop: chosen per token, the sixteen tokens of a thread were sixteen seven-way switches
  with_policy_variant<VARIANT>(variant, [&](auto which) {
    constexpr int V = decltype(which)::value;
#pragma unroll
    for (int g = 0; g < kGroups; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const TokenLoss t = token_loss<V>(pp, o[g][e], n[g][e], a[g][e], seq_lr);
        float loss = t.loss;
        if (isw_per_token) loss *= iw[g][e];
        const float we = w[g][e];
        const bool in = we != 0.f;
        // Elements past the end of the row were loaded as zeros with weight zero and add nothing, so the test is
        // redundant.  The small launches (FOLD) are faster without its sixteen branches (512 x 4096: 16.1 -> 15.8
        // us with the gradient); the large ones are faster with it (2048 x 16384: 115 against 117 us), where the
        // compiler then holds all of a thread's loads in registers at once.
        if (FOLD || e < pos.valid[g]) {
          s_loss += ((token_mean && !in) ? 0.f : loss) * we;
          s_m += we;
          s_kl += in ? t.kl * we : 0.f;
          s_cf += in ? t.cf * we : 0.f;
          s_cfl += in ? t.cfl * we : 0.f;
        }
        if (GRAD) gr[g][e] = (isw_per_token ? t.dloss * iw[g][e] : t.dloss) * we;
      }
  });
  if (GRAD) store_groups<VEC>(grad, pos, gr);
  static_assert(!ROWS || FOLD, "a launch that sets ready bytes has a last workgroup that clears them");
  double acc[5] = {s_loss, s_m, s_kl, s_cf, s_cfl};
  block_sum<5, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<5>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if constexpr (FOLD) {
    if (!ROWS && totals_suffice(ap.mode)) {  // no per-row pass: the launch totals are all these modes need
      totals_epilogue<5, kEpiPolicy>(wk, rows, chunks, cols, ap, coef, out, smem);
      return;
    }
    if (!last_block_arrives(wk.ticket)) return;
    double loss, msum, extra[3];
    finalize_agg<5>(wk.partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
    if (threadIdx.x == 0) loss_epilogue<kEpiPolicy>(loss, msum, extra, out);
    ticket_reset(wk.ticket);
    if (ROWS && chunks > 1) ready_bytes_clear<kRcThreads>(wk.ticket, rows * chunks);
  } else {
    if (wk.totals) totals_epilogue<5, kEpiPolicy>(wk, rows, chunks, cols, ap, coef, out, smem);
  }
}

// GSPO / GMPO on rows of two to four chunks when the workgroups of a row cannot wait for each other (more workgroups
// than the device holds at once, or waiting kernels switched off): one workgroup of 1024 threads holds the whole row
// in registers -- every 256 threads one chunk, 16 tokens of each input per thread -- so the per-sequence sums are a
// workgroup reduction and the inputs are read once, where a pre-pass launch reads three of the four a second time
// (2048 x 16384: 20 instead of 32 bytes per token; GSPO 180 -> 136 us, GMPO 192 -> 146 us).  The 64 - 80 values a
// thread holds leave room for one such workgroup per CU, so nothing streams on a CU while its workgroup reduces;
// squeezed into 64 registers for two per CU (log-probs kept as their difference, loads in two stages) the kernel
// spilled and took 199 / 252 us.  One record per row; a single-workgroup launch folds them (folding in the last
// workgroup to arrive measured the same).
constexpr int kWholeRowThreads = 1024;
constexpr int kWholeRowChunks = kWholeRowThreads / kRcThreads;
template <class M, bool GRAD, bool ISW, int VARIANT>
__global__ __launch_bounds__(kWholeRowThreads) void policy_whole_row_kernel(
    const float* __restrict__ old_lp, const float* __restrict__ lp, const float* __restrict__ adv,
    const M* __restrict__ mask, const float* __restrict__ isw, int64_t rows, int64_t cols, PolicyParams pp,
    int token_mean, double* __restrict__ records, float* __restrict__ grad) {
  static_assert(VARIANT == VAMD_PL_GSPO || VARIANT == VAMD_PL_GEO_MEAN, "the losses built on a per-sequence sum");
  const int64_t row = blockIdx.x;
  const ChunkPos pos(row, threadIdx.x / kRcThreads, cols, threadIdx.x % kRcThreads);
  const bool streaming = streams_past_caches(rows * cols);
  float o[kGroups][4], n[kGroups][4], a[kGroups][4], w[kGroups][4], iw[kGroups][4], gr[kGroups][4];
  load_groups<true>(old_lp, pos, o, streaming);
  load_groups<true>(lp, pos, n, streaming);
  load_groups<true>(adv, pos, a, streaming);
  load_mask_groups<true>(mask, pos, w, streaming);
  if (ISW) load_groups<true>(isw, pos, iw, streaming);
  __shared__ double smem[5 * (kWholeRowThreads / 64)];
  __shared__ double row_sums[4];
  double r[4];
  row_presums<ISW>(VARIANT, pos, o, n, a, w, iw, pp.nkl_lo, pp.nkl_hi, r);
  block_sum<4, kWholeRowThreads>(r, smem);
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) row_sums[i] = r[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = row_sums[i];
  float seq_lr;
  if (VARIANT == VAMD_PL_GSPO) {
    seq_lr = (float)r[1] / fmaxf((float)r[0], 1.f);
  } else {
    const float den = (float)r[0] + 1e-8f;
    seq_lr = -((float)r[2] / den) * expf((float)r[1] / den) * expf((float)r[3] / den) / den;
  }
  const bool isw_per_token = ISW && VARIANT != VAMD_PL_GEO_MEAN;
  float s_loss = 0, s_m = 0, s_kl = 0, s_cf = 0, s_cfl = 0;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const TokenLoss t = token_loss<VARIANT>(pp, o[g][e], n[g][e], a[g][e], seq_lr);
      float loss = t.loss;
      if (isw_per_token) loss *= iw[g][e];
      const float we = w[g][e];
      const bool in = we != 0.f;
      // no test for elements past the end of the row: they were loaded as zeros with weight zero and add nothing
      s_loss += ((token_mean && !in) ? 0.f : loss) * we;
      s_m += we;
      s_kl += in ? t.kl * we : 0.f;
      s_cf += in ? t.cf * we : 0.f;
      s_cfl += in ? t.cfl * we : 0.f;
      if (GRAD) gr[g][e] = (isw_per_token ? t.dloss * iw[g][e] : t.dloss) * we;
    }
  if (GRAD) store_groups<true>(grad, pos, gr, streaming);
  double acc[5] = {s_loss, s_m, s_kl, s_cf, s_cfl};
  block_sum<5, kWholeRowThreads>(acc, smem);
  if (threadIdx.x == 0) store_record<5>(records, row, 0, rows, 1, acc);
}

// =============================================================================================
// value loss (compute_value_loss, core_algos.py:1799-1838)
// =============================================================================================
template <bool VEC, class M, bool GRAD, bool FOLD>
__global__ __launch_bounds__(kRcThreads) void value_kernel(
    const float* __restrict__ vpreds, const float* __restrict__ returns, const float* __restrict__ values,
    const M* __restrict__ mask, int64_t rows, int64_t cols, int chunks, float clip, AggParams ap, Work wk,
    float* __restrict__ out, float* __restrict__ grad, float* __restrict__ coef) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float vp[kGroups][4], R[kGroups][4], v[kGroups][4], w[kGroups][4], gr[kGroups][4];
  load_groups<VEC>(vpreds, pos, vp);
  load_groups<VEC>(returns, pos, R);
  load_groups<VEC>(values, pos, v);
  load_mask_groups<VEC>(mask, pos, w);
  const bool token_mean = ap.mode == VAMD_AGG_TOKEN_MEAN;
  float s_loss = 0, s_m = 0, s_cf = 0;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float lo = v[g][e] - clip, hi = v[g][e] + clip;
      const float inner = fminf(vp[g][e], hi);
      const float vc = fmaxf(inner, lo);
      const float d1 = vp[g][e] - R[g][e], d2 = vc - R[g][e];
      const float e1 = d1 * d1, e2 = d2 * d2;
      const float loss = fmaxf(e1, e2);
      const float we = w[g][e];
      const bool in = we != 0.f;
      if (FOLD || e < pos.valid[g]) {  // redundant (zeros with weight zero past the end); see policy_kernel
        s_loss += ((token_mean && !in) ? 0.f : loss) * we;
        s_m += we;
        s_cf += (in && e2 > e1) ? we : 0.f;
      }
      if (GRAD) {
        const float ga = vp[g][e] < hi ? 1.f : (vp[g][e] == hi ? 0.5f : 0.f);
        const float gb = inner > lo ? 1.f : (inner == lo ? 0.5f : 0.f);
        const float g1 = e1 > e2 ? 1.f : (e1 == e2 ? 0.5f : 0.f);
        const float g2 = e2 > e1 ? 1.f : (e1 == e2 ? 0.5f : 0.f);
        gr[g][e] = (g1 * 2.f * d1 + g2 * 2.f * d2 * ga * gb) * we;
      }
    }
  if (GRAD) store_groups<VEC>(grad, pos, gr);
  __shared__ double smem[(3 + 3) * 4];
  double acc[3] = {s_loss, s_m, s_cf};
  block_sum<3, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<3>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if constexpr (FOLD) {
    if (totals_suffice(ap.mode)) {  // no per-row pass: the launch totals are all these modes need
      totals_epilogue<3, kEpiValue>(wk, rows, chunks, cols, ap, coef, out, smem);
      return;
    }
    if (!last_block_arrives(wk.ticket)) return;
    double loss, msum, extra[1];
    finalize_agg<3>(wk.partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
    if (threadIdx.x == 0) loss_epilogue<kEpiValue>(loss, msum, extra, out);
    ticket_reset(wk.ticket);
  } else {
    if (wk.totals) totals_epilogue<3, kEpiValue>(wk, rows, chunks, cols, ap, coef, out, smem);
  }
}

// =============================================================================================
// KL penalty (kl_penalty / kl_penalty_forward, core_algos.py:1841-1902)
// =============================================================================================
// kld and d kld / d logprob of one element.  straight: value of the chosen estimator, gradient of
// k2 (0.5 (lp - ref)^2), the reference's "+" variants.
// KIND >= 0 fixes the estimator at compile time (the sixteen tokens of a thread are then straight-line code that
// interleaves); KIND = -1 reads it from `kind`.
template <int KIND = -1>
__device__ __forceinline__ void kl_point(int kind, bool straight, float lp, float ref, float& kld, float& g) {
  const float d = lp - ref;
  switch (KIND >= 0 ? KIND : kind) {
    case VAMD_KL_K1:
      kld = d;
      g = 1.f;
      break;
    case VAMD_KL_ABS:
      kld = fabsf(d);
      g = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
      break;
    case VAMD_KL_K2:
      kld = 0.5f * d * d;
      g = d;
      break;
    default: {  // k3: exp(k) - k - 1 with k = clamp(ref - lp, -20, 20), result clamped to [-10, 10]
      const float k = ref - lp;
      const float kc = fminf(fmaxf(k, -20.f), 20.f);
      const float ratio = expf(kc);
      const float raw = ratio - kc - 1.f;
      kld = fminf(fmaxf(raw, -10.f), 10.f);
      const bool pass = k >= -20.f && k <= 20.f && raw >= -10.f && raw <= 10.f;  // clamp passes gradients on its bounds
      g = pass ? 1.f - ratio : 0.f;
    } break;
  }
  if (straight) g = d;
}
// f(std::integral_constant<int, kind>) for the runtime `kind`: one copy of the caller's token loop per estimator
// instead of a switch per token.
template <class F>
__device__ __forceinline__ void with_kl_kind(int kind, F&& f) {
  switch (kind) {
    case VAMD_KL_K1: f(std::integral_constant<int, VAMD_KL_K1>()); break;
    case VAMD_KL_ABS: f(std::integral_constant<int, VAMD_KL_ABS>()); break;
    case VAMD_KL_K2: f(std::integral_constant<int, VAMD_KL_K2>()); break;
    default: f(std::integral_constant<int, VAMD_KL_K3>()); break;
  }
}

__global__ __launch_bounds__(256) void kl_elementwise_kernel(const float* __restrict__ lp, const float* __restrict__ ref,
                                                             int64_t n, int kind, int straight,
                                                             float* __restrict__ kld, float* __restrict__ grad) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float k, g;
  kl_point(kind, straight != 0, lp[i], ref[i], k, g);
  if (kld) kld[i] = k;
  if (grad) grad[i] = g;
}

// agg_loss(kl_penalty(logprob, ref), mask, mode) in one pass, with the per-element gradient
// (times the mask weight, before the per-row agg_loss coefficient) on request.
template <bool VEC, class M, bool GRAD, bool FOLD>
__global__ __launch_bounds__(kRcThreads) void kl_loss_kernel(
    const float* __restrict__ logprob, const float* __restrict__ ref, const M* __restrict__ mask, int64_t rows,
    int64_t cols, int chunks, int kind, int straight, AggParams ap, Work wk, float* __restrict__ out,
    float* __restrict__ grad, float* __restrict__ coef) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float lp[kGroups][4], rf[kGroups][4], w[kGroups][4], gr[kGroups][4];
  load_groups<VEC>(logprob, pos, lp);
  load_groups<VEC>(ref, pos, rf);
  load_mask_groups<VEC>(mask, pos, w);
  const bool token_mean = ap.mode == VAMD_AGG_TOKEN_MEAN;
  float s_loss = 0, s_m = 0;
  with_kl_kind(kind, [&](auto which) {
    constexpr int KIND = decltype(which)::value;
#pragma unroll
    for (int g = 0; g < kGroups; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float kld, dk;
        kl_point<KIND>(kind, straight != 0, lp[g][e], rf[g][e], kld, dk);
        const float we = w[g][e];
        if (FOLD || e < pos.valid[g]) {  // redundant (zeros with weight zero past the end); see policy_kernel
          s_loss += ((token_mean && we == 0.f) ? 0.f : kld) * we;
          s_m += we;
        }
        if (GRAD) gr[g][e] = dk * we;
      }
  });
  if (GRAD) store_groups<VEC>(grad, pos, gr);
  __shared__ double smem[(2 + 3) * 4];
  double acc[2] = {s_loss, s_m};
  block_sum<2, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<2>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if constexpr (FOLD) {
    if (totals_suffice(ap.mode)) {  // no per-row pass: the launch totals are all these modes need
      totals_epilogue<2, kEpiKl>(wk, rows, chunks, cols, ap, coef, out, smem);
      return;
    }
    if (!last_block_arrives(wk.ticket)) return;
    double loss, msum, extra[1];
    finalize_agg<2>(wk.partials, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
    if (threadIdx.x == 0) loss_epilogue<kEpiKl>(loss, msum, extra, out);
    ticket_reset(wk.ticket);
  } else {
    if (wk.totals) totals_epilogue<2, kEpiKl>(wk, rows, chunks, cols, ap, coef, out, smem);
  }
}

// token_level_rewards = scores - beta * kld * mask and current_kl = mean over rows of
// masked_mean(kld * mask, mask, axis=-1), the two things apply_kl_penalty derives from the KL estimate
// (verl/trainer/ppo/ray_trainer.py:86-101), in one pass.
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void kl_reward_kernel(
    const float* __restrict__ scores, const float* __restrict__ logprob, const float* __restrict__ ref,
    const M* __restrict__ mask, int64_t rows, int64_t cols, int chunks, int kind, float beta, Work wk,
    float* __restrict__ rewards, float* __restrict__ current_kl) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float sc[kGroups][4], lp[kGroups][4], rf[kGroups][4], w[kGroups][4];
  load_groups<VEC>(scores, pos, sc);
  load_groups<VEC>(logprob, pos, lp);
  load_groups<VEC>(ref, pos, rf);
  load_mask_groups<VEC>(mask, pos, w);
  float s_kl = 0, s_m = 0;
  with_kl_kind(kind, [&](auto which) {
    constexpr int KIND = decltype(which)::value;
#pragma unroll
    for (int g = 0; g < kGroups; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float kld, dk;
        kl_point<KIND>(kind, false, lp[g][e], rf[g][e], kld, dk);
        const float we = w[g][e];
        const float km = kld * we;
        s_kl += (we == 0.f ? 0.f : km) * we;  // masked_sum: where(mask, v, 0) * mask; zeros past the end of the row
        s_m += we;
        sc[g][e] = sc[g][e] - beta * km;
      }
  });
  store_groups<VEC>(rewards, pos, sc);
  __shared__ double smem[2 * 4];
  double acc[2] = {s_kl, s_m};
  block_sum<2, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) {
    store_record<2>(wk.partials, row, chunk, rows, chunks, acc);
  }
  if (!last_block_arrives(wk.ticket)) return;
  double total = 0;
  for (int64_t r0 = threadIdx.x; r0 < rows; r0 += 4 * kRcThreads) {
    int64_t rr[4];
    bool have[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      rr[k] = r0 + (int64_t)k * kRcThreads;
      have[k] = rr[k] < rows;
    }
    double f[4][2];
    fold_row_records<2, 2, 4>(wk.partials, rr, have, rows, chunks, f);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (have[k]) total += (double)((float)f[k][0] / ((float)f[k][1] + 1e-8f));
  }
  double t[1] = {total};
  block_sum<1, kRcThreads>(t, smem);
  if (threadIdx.x == 0) current_kl[0] = (float)(t[0] / (double)rows);
  ticket_reset(wk.ticket);
}

// =============================================================================================
// GRPO
// =============================================================================================
constexpr int kGrpoLdsGroups = 2048;   // groups whose statistics fit one workgroup's LDS
constexpr int kGrpoInlineGroups = 512;  // ... and the LDS of every workgroup of the streaming pass

struct GrpoArgs {
  const int64_t* gid;
  int64_t rows, n_groups;
  float eps;
  int norm_by_std, std_mode;
  int estimator;            // VAMD_ADV_*
  float f_norm;             // GPG
  const double* row_moments;  // OPO: [rows][4] per-row masked moments, slot 0 = response length
  float* scores;   // [rows] scratch
  float* scalars;  // [rows] out: normalised scalar per response
  double* mean;    // [n_groups] (only used by the large-group-count path)
  double* stdv;
};

// Row sums of the rewards (the mask is NOT applied, core_algos.py:303); the last workgroup turns
// them into scores, per-group statistics and the per-response scalar of the chosen estimator:
//   GRPO             (s - mean) / (std + eps)  or  s - mean             core_algos.py:266-330
//   RLOO             s n/(n-1) - mean n/(n-1); a single-member group keeps s      :479-528
//   RLOO_VECTORIZED  the same, a single-member group gets 0                       :720-753
//   MEAN_BASELINE    s - mean (REINFORCE++ baseline before its whitening)         :421-474
//   OPO              s - sum(len s) / sum(len), len = response length             :531-579
//   GPG              alpha (s - mean) / f_norm, alpha = rows / max(#{s != 0}, 1)  :657-717
//   GRPO_PASSK       (max - second max) [/ (std + eps)] for the best response of a group, 0 for
//                    the others                                                   :360-418
// A single-member group has mean 0 (and std 1) in every estimator.
// std_mode 0: unbiased torch.std; 1: sqrt(clamp(var, min=eps)) of group_mean_std.  Singleton
// groups get mean 0, std 1 (core_algos.py:314-316, groupwise.py:215-221).
// Scores, per-group statistics and the per-response scalar from the (row, chunk) row-sum records; run by one
// workgroup of kRcThreads threads; g_cnt / g_sum / g_sq are LDS arrays of n_groups entries.
template <bool COHERENT, int HELD, int NT, int EST = -1>
__device__ __forceinline__ void grpo_scalars_from_records(const double* __restrict__ partials, int chunks,
                                                          const GrpoArgs& ga, int* __restrict__ g_cnt,
                                                          double* __restrict__ g_sum, double* __restrict__ g_sq) {
  for (int64_t g = threadIdx.x; g < ga.n_groups; g += NT) {
    g_cnt[g] = 0;
    g_sum[g] = 0.0;
    g_sq[g] = 0.0;
  }
  __syncthreads();
  const int estimator = EST >= 0 ? EST : ga.estimator;  // a compile-time estimator drops the other branches
  const bool opo = estimator == VAMD_ADV_OPO;
  double nnz_local = 0;
  // One workgroup runs this with nothing else to hide its latency, so a thread takes HELD rows per trip with
  // all their loads in flight, and when one trip covers the launch (rows <= HELD * NT) the rows' scores
  // and group ids stay in registers for the passes below instead of being read back.
  constexpr int64_t kTrip = (int64_t)HELD * NT;
  const bool resident = ga.rows <= kTrip;
  // Thread index -> row through a stride permutation: responses of one group usually sit next to each other,
  // and 64 lanes adding to a handful of LDS addresses are served one lane after the other.  A prime stride that
  // does not divide the row count is a bijection and sends neighbouring lanes to different groups.
  // Index i = threadIdx.x + m * NT maps to row (i * stride) mod rows, walked by adding (NT * stride) mod rows.
  const unsigned n_rows = (unsigned)ga.rows;
  // (a row count divisible by 61, 59 and 53 at once -- a multiple of 190747 -- walks the rows in order instead)
  const unsigned stride = n_rows % 61 ? 61 : (n_rows % 59 ? 59 : (n_rows % 53 ? 53 : 1));
  const unsigned first_row = (threadIdx.x * stride) % n_rows, row_step = ((unsigned)NT * stride) % n_rows;
  // rows of the HELD indices of a trip; `at` is the row of the trip's first index and moves on to the next trip
  auto trip_rows = [&](unsigned& at, int64_t (&rk)[HELD]) {
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      rk[k] = at;
      at += row_step;
      if (at >= n_rows) at -= n_rows;
    }
  };
  float sc[HELD];
  int gi[HELD];
  unsigned at = first_row;
  int64_t rk[HELD];
  for (int64_t base = threadIdx.x; base < ga.rows; base += kTrip) {
    double len[HELD];
    trip_rows(at, rk);
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      const int64_t i = base + (int64_t)k * NT;
      gi[k] = i < ga.rows ? (int)ga.gid[rk[k]] : 0;
      len[k] = (opo && i < ga.rows) ? ga.row_moments[rk[k] * 4] : 0.0;
    }
    constexpr int kSub = HELD < 4 ? HELD : 4;  // rows whose chunk records are in flight together
#pragma unroll
    for (int h = 0; h < HELD; h += kSub) {
      int64_t rr[kSub];
      bool have[kSub];
#pragma unroll
      for (int k = 0; k < kSub; ++k) {
        rr[k] = rk[h + k];
        have[k] = base + (int64_t)(h + k) * NT < ga.rows;
      }
      double row_sum[kSub][1];
      fold_row_records<1, 1, kSub, COHERENT>(partials, rr, have, ga.rows, chunks, row_sum);
#pragma unroll
      for (int k = 0; k < kSub; ++k) sc[h + k] = (float)row_sum[k][0];
    }
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      if (base + (int64_t)k * NT >= ga.rows) break;
      ga.scores[rk[k]] = sc[k];
      nnz_local += sc[k] != 0.f ? 1.0 : 0.0;
      atomicAdd(&g_cnt[gi[k]], 1);
      if (opo) {  // g_sum: sum(len * s), g_sq: sum(len)
        atomicAdd(&g_sum[gi[k]], len[k] * (double)sc[k]);
        atomicAdd(&g_sq[gi[k]], len[k]);
      } else {
        atomicAdd(&g_sum[gi[k]], (double)sc[k]);
      }
    }
  }
  __syncthreads();
  // scores and group ids of the trip starting at `base`: still in registers, or read back
  auto held_rows = [&](int64_t base) {
    if (resident) return;  // rk[] is then still the one trip's
    trip_rows(at, rk);
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      const int64_t i = base + (int64_t)k * NT;
      gi[k] = i < ga.rows ? (int)ga.gid[rk[k]] : 0;
      sc[k] = i < ga.rows ? ga.scores[rk[k]] : 0.f;
    }
  };
  if (estimator == VAMD_ADV_GRPO || estimator == VAMD_ADV_GRPO_PASSK) {
    at = first_row;
    for (int64_t base = threadIdx.x; base < ga.rows; base += kTrip) {
      held_rows(base);
#pragma unroll
      for (int k = 0; k < HELD; ++k) {
        if (base + (int64_t)k * NT >= ga.rows) break;
        const double d = (double)sc[k] - g_sum[gi[k]] / (double)g_cnt[gi[k]];
        atomicAdd(&g_sq[gi[k]], d * d);
      }
    }
    __syncthreads();
  }
  if (estimator == VAMD_ADV_GRPO_PASSK) {
    // one thread per group walks the responses in index order: best score (first index on ties,
    // where the advantage is 0 anyway), runner-up, unbiased std; the group's entry of `mean`
    // receives the advantage and the entry of `stdv` the index of the best response
    __syncthreads();
    for (int64_t g = threadIdx.x; g < ga.n_groups; g += NT) {
      float best = -INFINITY, second = -INFINITY;
      int64_t arg = -1;
      for (int64_t r = 0; r < ga.rows; ++r) {
        if (ga.gid[r] != g) continue;
        const float sc = ga.scores[r];
        if (sc > best) {
          second = best;
          best = sc;
          arg = r;
        } else if (sc > second) {
          second = sc;
        }
      }
      const int c = g_cnt[g];
      float a = best - second;
      if (ga.norm_by_std) a = a / ((float)sqrt(g_sq[g] / (double)(c - 1)) + ga.eps);
      g_sum[g] = (double)a;
      g_sq[g] = (double)arg;
    }
    __syncthreads();
  }
  float alpha = 1.f;
  if (estimator == VAMD_ADV_GPG) {
    __shared__ double nz_smem[NT / 64];
    __shared__ float alpha_bc;
    double acc1[1] = {nnz_local};
    block_sum<1, NT>(acc1, nz_smem);
    if (threadIdx.x == 0) alpha_bc = (float)ga.rows / fmaxf((float)acc1[0], 1.f);
    __syncthreads();
    alpha = alpha_bc;
  }
  at = first_row;
  for (int64_t base = threadIdx.x; base < ga.rows; base += kTrip) {
    held_rows(base);
#pragma unroll
    for (int k = 0; k < HELD; ++k) {
      if (base + (int64_t)k * NT >= ga.rows) break;
      const int64_t r = rk[k];
      const int g = gi[k];
      const int c = g_cnt[g];
      // The scores are fp32 like the reference's, everything after them is evaluated in double and rounded once:
      // rounding the group mean to fp32 before the subtraction would cost 1e-4 of the advantage in a group whose
      // scores nearly coincide.
      const double sck = (double)sc[k];
      const double mean = c > 1 ? g_sum[g] / (double)c : 0.0;
      double out;
      switch (estimator) {
        case VAMD_ADV_GRPO: {
          double sd = 1.0;
          if (c > 1) {
            const double var = g_sq[g] / (double)(c - 1);
            sd = ga.std_mode == 0 ? sqrt(var) : sqrt(fmax(var, (double)ga.eps));
          }
          const double cen = sck - mean;
          out = ga.norm_by_std ? cen / (sd + (double)ga.eps) : cen;
        } break;
        case VAMD_ADV_RLOO:
        case VAMD_ADV_RLOO_VECTORIZED: {
          if (c > 1) {
            const double n = (double)c, n1 = (double)(c - 1);
            out = sck * n / n1 - mean * n / n1;
          } else {
            out = estimator == VAMD_ADV_RLOO ? sck : 0.0;
          }
        } break;
        case VAMD_ADV_OPO:
          out = c > 1 ? sck - g_sum[g] / g_sq[g] : sck;
          break;
        case VAMD_ADV_GPG:
          out = (double)alpha * (sck - mean) / (double)ga.f_norm;
          break;
        case VAMD_ADV_GRPO_PASSK:
          out = (double)r == g_sq[g] ? g_sum[g] : 0.0;
          break;
        default:  // VAMD_ADV_MEAN_BASELINE
          out = sck - mean;
          break;
      }
      // COHERENT: workgroups of the same launch (on other XCDs, behind other L2s) may read the scalars next
      if constexpr (COHERENT) peer_store_f32(ga.scalars + r, (float)out);
      else ga.scalars[r] = (float)out;
    }
  }
}

// Small launches let the workgroup that arrives last run the statistics (TAIL); large ones leave them to a launch
// of their own, whose registers and LDS are then not charged to every wavefront of the streaming pass.
// `chunks` counts the records per row: a workgroup walks `span` consecutive 4096-column chunks (1 for small
// launches; for launches of thousands of rows the whole row, so that the records stay few enough for the statistics
// to run in the same launch).
template <bool VEC, bool TAIL>
__global__ __launch_bounds__(kRcThreads) void grpo_rowsum_kernel(const float* __restrict__ x, int64_t cols,
                                                                 int chunks, int span, Work wk, GrpoArgs ga) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const bool streaming = streams_past_caches(ga.rows * cols);
  double total = 0.0;
  for (int u = 0; u < span; ++u) {
    const ChunkPos pos(row, chunk * span + u, cols);
    float v[kGroups][4];
    load_groups<VEC>(x, pos, v, streaming);
    float s = 0;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) s += (v[g][0] + v[g][1]) + (v[g][2] + v[g][3]);
    total += (double)s;
  }
  __shared__ double smem[4];
  double acc[1] = {total};
  block_sum<1, kRcThreads>(acc, smem);
  if constexpr (TAIL) {
    if (threadIdx.x == 0) store_record<1>(wk.partials, row, chunk, ga.rows, chunks, acc);
    if (!last_block_arrives(wk.ticket)) return;
    __shared__ int g_cnt[kGrpoInlineGroups];
    __shared__ double g_sum[kGrpoInlineGroups], g_sq[kGrpoInlineGroups];
    grpo_scalars_from_records<true, 4, kRcThreads>(wk.partials, chunks, ga, g_cnt, g_sum, g_sq);
    ticket_reset(wk.ticket);
  } else {
    if (threadIdx.x == 0) wk.partials[record_at(0, row, chunk, ga.rows, chunks)] = acc[0];
  }
}

// GRPO proper, up to a few thousand responses, in one launch without a serial statistics step: workgroup b owns rows
// b, b + grid, ...  Pass 1 leaves every row's score (the unmasked row sum, fp32 like the reference's) in memory; in
// pass 2 each workgroup finds the other members of its rows' groups by comparing the group ids (a few KB,
// cache-resident), takes the group's mean and unbiased standard deviation from their scores in double, and streams
// scalar * mask.  Every workgroup repeats a little arithmetic, none waits for a single workgroup to do all of it.
// Between the passes a workgroup waits either at one meeting of the whole launch or, when it walks several rows,
// for the ready bytes of its groups' members only.  A workgroup that owns at most kGrpoHeldSlots chunks keeps its
// mask as bits in LDS between the passes and only stores afterwards.  The waits are bounded; a
// workgroup whose wait ran out (the launch's workgroups were not all running at once) sums the rows of its groups'
// members itself, so the launch finishes with the right result whatever the device lets run together.
constexpr int kGrpoHeldSlots = 32;  // chunks of one workgroup whose mask bits stay in LDS (16 KB)
struct GrpoRowsArgs {
  const float* rewards;
  const void* mask;
  const int64_t* gid;
  int64_t rows, cols;
  int chunks;
  float eps;
  int norm_by_std, std_mode;
  float* scores;   // [rows] scratch, written and read through the device-coherent path
  float* scalars;  // [rows] optional out
  float* out;
  unsigned* ticket;
  unsigned spin_limit;
};

constexpr int64_t kGrpoRowsLimit = 32 * kRcThreads;  // one membership bit per thread for every 256 responses
// One "score is in memory" byte per response (ready_byte).
static_assert(kGrpoRowsLimit <= kReadyBytes, "one ready byte per response");
__device__ __forceinline__ unsigned char* grpo_ready_byte(unsigned* ticket, int64_t row) { return ready_byte(ticket, row); }
// Bit k set: response k * 256 + threadIdx.x belongs to the group of `row` (no bits for a row past the end).
__device__ __forceinline__ unsigned grpo_member_bits(const int64_t* __restrict__ gid, int64_t rows, int64_t row) {
  unsigned bits = 0;
  if (row < rows) {
    const int64_t g = gid[row];
    for (int k = 0; (int64_t)k * kRcThreads + threadIdx.x < rows; ++k)
      bits |= (gid[(int64_t)k * kRcThreads + threadIdx.x] == g ? 1u : 0u) << k;
  }
  return bits;
}

// The unmasked sum of one row of rewards, valid in thread 0: the same chunk order and workgroup reduction whoever
// computes it, so that a workgroup that has to work out another row's score itself arrives at the same bits.
template <bool VEC>
__device__ __forceinline__ double grpo_row_sum(const float* __restrict__ rewards, int64_t row, int64_t cols, int chunks,
                                               bool streaming, double* smem) {
  double total = 0.0;
  for (int c = 0; c < chunks; ++c) {
    const ChunkPos pos(row, c, cols);
    float v[kGroups][4];
    load_groups<VEC>(rewards, pos, v, streaming);
    float s = 0;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) s += (v[g][0] + v[g][1]) + (v[g][2] + v[g][3]);
    total += (double)s;
  }
  double acc[1] = {total};
  block_sum<1, kRcThreads>(acc, smem);
  return acc[0];
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void grpo_rows_kernel(GrpoRowsArgs a) {
  const M* __restrict__ mask = static_cast<const M*>(a.mask);
  const bool streaming = streams_past_caches(a.rows * a.cols);
  // How a workgroup learns that the scores it needs are in memory.  A workgroup that walks several rows waits for its
  // groups' members only, so that early workgroups store while late ones still read (71 instead of 74 us at
  // 2048 x 16384); with one row each everybody finishes together and one launch-wide meeting is quicker (14.4
  // against 16.6 us at 512 x 4096).
  const bool by_group = gridDim.x < a.rows;
  // read before anything else: whoever arrives last does so after this workgroup has arrived, hence after this load
  const unsigned epoch_on_entry =
      by_group ? 0u : __hip_atomic_load(a.ticket + kEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // One bit per mask element this workgroup owns, kept in LDS across the meeting when they fit, so that pass 2 only
  // stores.  A thread that met a mask value other than 0 and 1 reads its mask again instead.
  static_assert(kGroups * 4 <= 16, "one 16-bit word per thread and chunk");
  __shared__ unsigned short held_bits[kGrpoHeldSlots * kRcThreads];
  const int64_t own_rows = (a.rows - blockIdx.x + gridDim.x - 1) / gridDim.x;
  const bool held = own_rows * a.chunks <= kGrpoHeldSlots;
  bool binary = true;
  int slot = 0;
  __shared__ double smem[6 * (kRcThreads / 64)];
  __shared__ double bc[2];
  float w[kGroups][4];
  for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
    double total = 0.0;
    for (int c = 0; c < a.chunks; ++c) {
      const ChunkPos pos(row, c, a.cols);
      float v[kGroups][4];
      load_groups<VEC>(a.rewards, pos, v, streaming);
      if (held) {
        load_mask_groups<VEC>(mask, pos, w, streaming);
        unsigned bits = 0;
#pragma unroll
        for (int g = 0; g < kGroups; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float m = w[g][e];
            bits |= (m != 0.f ? 1u : 0u) << (g * 4 + e);
            binary = binary && (m == 0.f || m == 1.f);
          }
        held_bits[slot * kRcThreads + threadIdx.x] = (unsigned short)bits;
        ++slot;
      }
      float s = 0;
#pragma unroll
      for (int g = 0; g < kGroups; ++g) s += (v[g][0] + v[g][1]) + (v[g][2] + v[g][3]);
      total += (double)s;
    }
    double acc[1] = {total};
    block_sum<1, kRcThreads>(acc, smem);
    if (threadIdx.x == 0) {  // the score, and once it has landed, the row's ready byte
      peer_store_f32(a.scores + row, (float)acc[0]);
      if (by_group) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __hip_atomic_store(grpo_ready_byte(a.ticket, row), (unsigned char)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  // Which responses share a group with this workgroup's first two rows does not depend on the scores: thread t notes
  // it for responses t, t + 256, ... (one bit each, kGrpoRowsLimit / 256 of them) while the others are still summing.
  unsigned member[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) member[r] = grpo_member_bits(a.gid, a.rows, (int64_t)blockIdx.x + (int64_t)r * gridDim.x);
  bool all_open = true;
  if (!by_group) {
    // One meeting of the whole launch, with nothing to fold and nobody to report to (a workgroup whose wait ran out helps itself),
    // so it needs no departure count: the gate is an epoch word that the last arrival advances after it has put the
    // arrival counters back to zero; the others wait for the word to differ from what they read on entry.
    const bool last = last_block_arrives(a.ticket);  // waits for this workgroup's stores first
    if (last) {
      ticket_reset(a.ticket);
      if (threadIdx.x == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __hip_atomic_store(a.ticket + kEpochWord, epoch_on_entry + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    } else {
      __shared__ unsigned moved;
      if (threadIdx.x == 0) {
        unsigned seen = epoch_on_entry;
        for (unsigned spins = 0;; ++spins) {
          seen = __hip_atomic_load(a.ticket + kEpochWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (seen != epoch_on_entry || spins >= a.spin_limit) break;
          __builtin_amdgcn_s_sleep(4);
        }
        moved = seen != epoch_on_entry ? 1u : 0u;
        if (!moved) note_gave_up(a.ticket);
      }
      __syncthreads();
      all_open = moved != 0u;
    }
  }
  slot = 0;
  unsigned polls = 0;
  // two rows at a time: their group statistics share one pass over the scores and one workgroup reduction
  for (int64_t base = blockIdx.x; base < a.rows; base += 2 * (int64_t)gridDim.x) {
    float scalar[2] = {0.f, 0.f};
    if (base != blockIdx.x)
#pragma unroll
      for (int r = 0; r < 2; ++r) member[r] = grpo_member_bits(a.gid, a.rows, base + (int64_t)r * gridDim.x);
    // wait for the scores of the groups' members only -- typically neighbouring rows that finish together -- not for
    // the whole launch; every thread polls the ready bytes of the members it noted, a bounded number of times
    bool ready = all_open;
#pragma unroll
    for (int r = 0; r < 2; ++r)
      for (unsigned bits = by_group ? member[r] : 0u; bits && ready; bits &= bits - 1) {
        const int64_t i = (int64_t)(__ffs(bits) - 1) * kRcThreads + threadIdx.x;
        const unsigned char* flag = grpo_ready_byte(a.ticket, i);
        while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
          if (polls++ >= a.spin_limit) {
            ready = false;
            break;
          }
          __builtin_amdgcn_s_sleep(4);
        }
      }
    const bool open = by_group ? __syncthreads_and(ready) != 0 : all_open;
    if (by_group && !open && threadIdx.x == 0) note_gave_up(a.ticket);
    // count, sum and sum of squares of (score - own score) over the group: differences of fp32 scores are exact
    // in double, and shifted by the row's own score the one-pass variance loses nothing to cancellation
    double own[2], cs[6];
    if (open) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int64_t row = base + (int64_t)r * gridDim.x;
        own[r] = row < a.rows ? (double)peer_load_f32(a.scores + row) : 0.0;
        cs[3 * r] = cs[3 * r + 1] = cs[3 * r + 2] = 0.0;
        for (unsigned bits = member[r]; bits; bits &= bits - 1) {
          const int64_t i = (int64_t)(__ffs(bits) - 1) * kRcThreads + threadIdx.x;
          const double d = (double)peer_load_f32(a.scores + i) - own[r];
          cs[3 * r] += 1.0;
          cs[3 * r + 1] += d;
          cs[3 * r + 2] += d * d;
        }
      }
      block_sum<6, kRcThreads>(cs, smem);
    } else {
      // The wait ran out (the launch's workgroups are not all running, say on a GPU that other work shares): this
      // workgroup sums the rows of its groups' members itself, to the same bits their owners arrive at, and depends
      // on nobody.  Every thread walks all responses; the sums of the members end up in thread 0.
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int64_t row = base + (int64_t)r * gridDim.x;
        cs[3 * r] = cs[3 * r + 1] = cs[3 * r + 2] = 0.0;
        own[r] = 0.0;
        if (row >= a.rows) continue;
        const int64_t g = a.gid[row];
        own[r] = (double)(float)grpo_row_sum<VEC>(a.rewards, row, a.cols, a.chunks, streaming, smem);
        for (int64_t i = 0; i < a.rows; ++i) {
          if (a.gid[i] != g) continue;
          const double d = (double)(float)grpo_row_sum<VEC>(a.rewards, i, a.cols, a.chunks, streaming, smem) - own[r];
          cs[3 * r] += 1.0;
          cs[3 * r + 1] += d;
          cs[3 * r + 2] += d * d;
        }
      }
    }
    {
      if (threadIdx.x == 0) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int64_t row = base + (int64_t)r * gridDim.x;
          if (row >= a.rows) continue;
          // scores are fp32 like the reference's; everything after them is evaluated in double and rounded once
          const double cnt = cs[3 * r], s1 = cs[3 * r + 1], s2 = cs[3 * r + 2];
          double cen = own[r], sd = 1.0;  // a group of one: mean 0, std 1
          if (cnt > 1.0) {
            cen = -s1 / cnt;
            const double var = fmax(s2 - s1 * s1 / cnt, 0.0) / (cnt - 1.0);
            sd = a.std_mode == 0 ? sqrt(var) : sqrt(fmax(var, (double)a.eps));
          }
          bc[r] = a.norm_by_std ? cen / (sd + (double)a.eps) : cen;
          if (a.scalars) a.scalars[row] = (float)bc[r];
        }
      }
      __syncthreads();
      scalar[0] = (float)bc[0];
      scalar[1] = (float)bc[1];
      __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int64_t row = base + (int64_t)r * gridDim.x;
      if (row >= a.rows) break;
      for (int c = 0; c < a.chunks; ++c) {
        const ChunkPos pos(row, c, a.cols);
        if (held && binary) {
          const unsigned bits = held_bits[slot * kRcThreads + threadIdx.x];
#pragma unroll
          for (int g = 0; g < kGroups; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e) w[g][e] = (bits >> (g * 4 + e)) & 1u ? 1.f : 0.f;
        } else {
          load_mask_groups<VEC>(mask, pos, w, streaming);
        }
        ++slot;
#pragma unroll
        for (int g = 0; g < kGroups; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) w[g][e] *= scalar[r];
        store_groups<VEC>(a.out, pos, w, streaming);
      }
    }
  }
  // by group: the last workgroup to leave clears the ready bytes with the counters, zero again for the next call
  if (by_group && gate_depart(a.ticket) != 0)
    for (int64_t w = threadIdx.x; w < (a.rows + 3) / 4; w += kRcThreads)  // four rows' bytes per word
      __hip_atomic_store(reinterpret_cast<unsigned*>(grpo_ready_byte(a.ticket, w * 4)), 0u, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
}

constexpr int kGrpoTailThreads = 1024;
template <int EST>
__global__ __launch_bounds__(kGrpoTailThreads) void grpo_scalars_kernel_lds(const double* __restrict__ partials, int chunks,
                                                                            GrpoArgs ga) {
  __shared__ int g_cnt[kGrpoLdsGroups];
  __shared__ double g_sum[kGrpoLdsGroups], g_sq[kGrpoLdsGroups];
  grpo_scalars_from_records<false, 2, kGrpoTailThreads, EST>(partials, chunks, ga, g_cnt, g_sum, g_sq);
}

// ---- path for more groups than fit in LDS (and for group_mean_std itself) ----
__global__ void rowsum_finalize_kernel(const double* __restrict__ partials, int64_t rows, int chunks,
                                       float* __restrict__ scores) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  double s = 0;
  for (int c = 0; c < chunks; ++c) s += partials[record_at(0, r, c, rows, chunks)];
  scores[r] = (float)s;
}

// One thread per group: count, mean, std over the group's members in index order; written as fp32 for
// group_mean_std itself and in double for the GRPO path, which subtracts and divides in double.
template <class T>
__global__ void group_stats_kernel(const float* __restrict__ scores, const int64_t* __restrict__ gid, int64_t n,
                                   int64_t n_groups, float eps, int std_mode, T* __restrict__ mean,
                                   T* __restrict__ stdv, float* __restrict__ count) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n_groups) return;
  double s = 0;
  int64_t c = 0;
  for (int64_t i = 0; i < n; ++i)
    if (gid[i] == g) {
      s += scores[i];
      ++c;
    }
  double mu = 0.0, sd = 1.0;
  if (c > 1) {
    const double m = s / (double)c;
    double q = 0;
    for (int64_t i = 0; i < n; ++i)
      if (gid[i] == g) {
        const double d = (double)scores[i] - m;
        q += d * d;
      }
    const double var = q / (double)(c - 1);
    mu = m;
    if (std_mode == 0) sd = sqrt(var);
    else sd = sizeof(T) == sizeof(double) ? sqrt(fmax(var, (double)eps)) : (double)sqrtf(fmaxf((float)var, eps));
  }
  mean[g] = (T)mu;
  stdv[g] = (T)sd;
  if (count) count[g] = (float)c;
}

__global__ void grpo_scalars_kernel(const float* __restrict__ scores, const int64_t* __restrict__ gid, int64_t n,
                                    const double* __restrict__ mean, const double* __restrict__ stdv, float eps,
                                    int norm_by_std, float* __restrict__ scalars) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t g = gid[i];
  const double c = (double)scores[i] - mean[g];
  scalars[i] = (float)(norm_by_std ? c / (stdv[g] + (double)eps) : c);
}

// adv[i][t] = scalars[i] * (float)mask[i][t]
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void broadcast_rows_kernel(const float* __restrict__ scalars,
                                                                    const M* __restrict__ mask, int64_t cols,
                                                                    int chunks, float* __restrict__ out) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float w[kGroups][4];
  load_mask_groups<VEC>(mask, pos, w);
  const float a = scalars[row];
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) w[g][e] *= a;
  store_groups<VEC>(out, pos, w);
}

// ---------------------------------------------------------------------------------------------
static int check_matrix(const char* what, int64_t rows, int64_t cols) {
  VAMD_REQUIRE(rows > 0 && cols > 0, "%s: empty input (%lld x %lld)", what, (long long)rows, (long long)cols);
  VAMD_REQUIRE(rows * chunks_of(cols) < (1ll << 31), "%s: too many workgroups", what);
  return VAMD_OK;
}

static AggParams make_agg(int mode, double dp, double bnt, double gbs, double lsf) {
  return make_agg_params(mode, dp, bnt, gbs, lsf);
}

static size_t reduce_workspace_bytes(int64_t rows, int64_t cols, int nv) {
  if (rows <= 0 || cols <= 0) return 0;
  return kTicketBytes + align_up(((size_t)rows * chunks_of(cols) + kShareSlots) * nv * sizeof(double), 256);
}

static Work carve_work(void* workspace) {
  Work w;
  w.ticket = static_cast<unsigned*>(workspace);
  w.partials = reinterpret_cast<double*>(static_cast<char*>(workspace) + kTicketBytes);
  w.totals = 0;
  return w;
}

}  // namespace vamd

using namespace vamd;

#define VAMD_VEC_DISPATCH(vec, V, ...) \
  if (vec) { constexpr bool V = true; __VA_ARGS__; } else { constexpr bool V = false; __VA_ARGS__; }

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_masked_moments_workspace_bytes(int64_t rows, int64_t cols) {
  return reduce_workspace_bytes(rows, cols, 4);
}

static int masked_moments_of_difference(const float* values, const float* minus, const void* mask, int mask_dtype,
                                        int64_t rows, int64_t cols, int per_row, MomentOuts out, void* workspace,
                                        size_t workspace_bytes, void* stream);

extern "C" int vamd_masked_moments(const float* values, const void* mask, int mask_dtype, int64_t rows,
                                   int64_t cols, int per_row, double* out, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  VAMD_REQUIRE(out, "masked_moments: null pointer");
  return masked_moments_of_difference(values, nullptr, mask, mask_dtype, rows, cols, per_row,
                                      MomentOuts{out, nullptr, nullptr, nullptr, nullptr, 1}, workspace,
                                      workspace_bytes, stream);
}

extern "C" int vamd_masked_reduce(const float* values, const void* mask, int mask_dtype, int64_t rows, int64_t cols,
                                  int per_row, double* moments, float* sum, float* mean, float* denom,
                                  float* whiten_stats, int shift_mean, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  VAMD_REQUIRE(moments || sum || mean || denom || whiten_stats, "masked_reduce: no output requested");
  VAMD_REQUIRE(!(per_row && whiten_stats), "masked_reduce: whitening statistics are taken over the whole input");
  return masked_moments_of_difference(values, nullptr, mask, mask_dtype, rows, cols, per_row,
                                      MomentOuts{moments, sum, mean, denom, whiten_stats, shift_mean}, workspace,
                                      workspace_bytes, stream);
}

static int masked_moments_of_difference(const float* values, const float* minus, const void* mask, int mask_dtype,
                                        int64_t rows, int64_t cols, int per_row, MomentOuts out, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  int st = check_matrix("masked_moments", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(values && mask, "masked_moments: null pointer");
  if (!workspace || workspace_bytes < vamd_masked_moments_workspace_bytes(rows, cols)) {
    set_error("masked_moments: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int all_chunks = (int)chunks_of(cols);
  const int span = record_span(rows, all_chunks);
  const int chunks = (all_chunks + span - 1) / span;  // records per row
  const Work wk = carve_work(workspace);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {values, minus}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((moments_kernel<V, M>), dim3((unsigned)(rows * chunks)),
                                                 dim3(kRcThreads), 0, s, values, minus, static_cast<const M*>(mask),
                                                 rows, cols, chunks, span, per_row, wk, out));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
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
  VAMD_REQUIRE(chunks_of(n) < (1ll << 31), "affine_by_stats: too many elements");
  const bool vec = (n % 4 == 0) && aligned_to(values, 16) && aligned_to(out, 16);
  const dim3 grid((unsigned)chunks_of(n));
  hipStream_t s = static_cast<hipStream_t>(stream);
  VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((affine_kernel<V>), grid, dim3(kRcThreads), 0, s, values, stats, n,
                                               out));
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_affine_by_stats_masked(const float* values, const float* stats, const void* mask, int mask_dtype,
                                           int64_t n, float* out, void* stream) {
  VAMD_REQUIRE(values && stats && mask && out && n > 0, "affine_by_stats_masked: bad argument");
  VAMD_REQUIRE(chunks_of(n) < (1ll << 31), "affine_by_stats_masked: too many elements");
  const dim3 grid((unsigned)chunks_of(n));
  hipStream_t s = static_cast<hipStream_t>(stream);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(n, {values, out}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((affine_masked_kernel<V, M>), grid, dim3(kRcThreads), 0, s, values,
                                                 stats, static_cast<const M*>(mask), n, out));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_agg_loss_workspace_bytes(int64_t rows, int64_t cols) {
  return reduce_workspace_bytes(rows, cols, 2);
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
  Work wk = carve_work(workspace);
  const AggParams ap = make_agg(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor);
  bool sep = rows * chunks > kInlineFoldRecords;  // fold the records in a launch of their own
  wk.totals = sep && totals_suffice(mode);        // ... unless the launch totals are all the mode needs
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {loss_mat}, mask, sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
    if (vec && sep)
      hipLaunchKernelGGL((agg_kernel<true, M, false>), grid, block, 0, s, loss_mat, mk, rows, cols, chunks, ap, wk,
                         out_loss, coef_out);
    else if (vec)
      hipLaunchKernelGGL((agg_kernel<true, M, true>), grid, block, 0, s, loss_mat, mk, rows, cols, chunks, ap, wk,
                         out_loss, coef_out);
    else
      hipLaunchKernelGGL((agg_kernel<false, M, true>), grid, block, 0, s, loss_mat, mk, rows, cols, chunks, ap, wk,
                         out_loss, coef_out);
    sep = sep && vec;
  });
  if (sep && !wk.totals)
    hipLaunchKernelGGL((fold_loss_kernel<2, kEpiAgg>), dim3(1), dim3(kFoldThreads), 0, s, wk.partials, rows, chunks,
                       cols, ap, coef_out, out_loss);
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
  return reduce_workspace_bytes(rows, cols, 5);
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
  if (!workspace || workspace_bytes < vamd_policy_loss_workspace_bytes(rows, cols)) {
    set_error("policy_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  // the vanilla loss never touches the per-row moments the general query reserves room for
  return vamd_policy_loss_variant_forward(VAMD_PL_VANILLA, old_log_prob, log_prob, advantages, mask, mask_dtype,
                                          is_weights, rows, cols, clip_low, clip_high, clip_c, 1.f, 1.f, mode,
                                          dp_size, batch_num_tokens, global_batch_size, loss_scale_factor, out,
                                          grad_unscaled, coef_out, workspace,
                                          vamd_policy_loss_variant_workspace_bytes(rows, cols), stream);
}

extern "C" size_t vamd_policy_loss_variant_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  // the reduction records, then per-row (GSPO) or per-(row, chunk) (GEO_MEAN) sums of the row pre-pass
  return reduce_workspace_bytes(rows, cols, 5) + align_up((size_t)rows * chunks_of(cols) * 4 * sizeof(double), 256);
}

extern "C" int vamd_policy_loss_variant_forward(int variant, const float* old_log_prob, const float* log_prob,
                                                const float* advantages, const void* mask, int mask_dtype,
                                                const float* is_weights, int64_t rows, int64_t cols, float clip_low,
                                                float clip_high, float clip_c, float tau_pos, float tau_neg, int mode,
                                                double dp_size, double batch_num_tokens, double global_batch_size,
                                                double loss_scale_factor, float* out, float* grad_unscaled,
                                                float* coef_out, void* workspace, size_t workspace_bytes,
                                                void* stream) {
  int st = check_matrix("policy_loss", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(old_log_prob && log_prob && advantages && mask && out, "policy_loss: null pointer");
  VAMD_REQUIRE(variant >= VAMD_PL_VANILLA && variant <= VAMD_PL_GEO_MEAN, "policy_loss: invalid variant %d", variant);
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "policy_loss: invalid mode %d", mode);
  VAMD_REQUIRE(variant != VAMD_PL_VANILLA || clip_c > 1.0f, "policy_loss: clip_ratio_c must be > 1.0, got %f",
               (double)clip_c);
  VAMD_REQUIRE(variant != VAMD_PL_SAPO || (tau_pos != 0.f && tau_neg != 0.f), "policy_loss: SAPO needs non-zero tau");
  VAMD_REQUIRE(!grad_unscaled || coef_out, "policy_loss: grad output needs coef_out");
  if (!workspace || workspace_bytes < vamd_policy_loss_variant_workspace_bytes(rows, cols)) {
    set_error("policy_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  Work wk = carve_work(workspace);
  PolicyParams pp;
  pp.ratio_lo = (float)(1.0 - (double)clip_low);
  pp.ratio_hi = (float)(1.0 + (double)clip_high);
  pp.clip_c = clip_c;
  pp.variant = variant;
  pp.tau_pos = tau_pos;
  pp.tau_neg = tau_neg;
  pp.row_moments = nullptr;
  pp.row_partials = nullptr;
  pp.spin_limit = 0;
  pp.nkl_lo = pp.nkl_hi = 0.f;
  const bool per_row = variant == VAMD_PL_GSPO || variant == VAMD_PL_GEO_MEAN;  // losses built on a per-sequence quantity
  double* const row_area =
      reinterpret_cast<double*>(static_cast<char*>(workspace) + reduce_workspace_bytes(rows, cols, 5));
  AggParams ap = make_agg(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor);
  const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
  const float* token_weights = is_weights;  // what the per-token pass multiplies by
  if (variant == VAMD_PL_GEO_MEAN) {
    // the loss is the plain mean of the per-sequence losses over all rows (:1706): every valid token carries its
    // row's loss / M, summed per row and divided by the number of rows
    ap = make_agg(VAMD_AGG_SEQ_MEAN_TOKEN_SUM, 1.0, -1.0, (double)rows, -1.0);
    pp.nkl_lo = -clip_low;
    pp.nkl_hi = clip_high;
  }
  // The loss kernel works the per-sequence quantity out itself (one pass over the inputs, 20 against 24.5 us at
  // 512 x 4096) when the whole launch is resident at once, so that a workgroup waiting for its row's other chunks
  // keeps nobody from starting, and the tensors qualify for 16-byte accesses; otherwise a pre-pass leaves it in the
  // workspace.  (With more workgroups than fit the device at once the waits add up: 305 against 190 us at 2048 x 16384.)
  bool rows_inline = false;
  if (per_row && waiting_kernels_allowed() && rows * chunks <= kInlineFoldRecords && rows * chunks <= kReadyBytes &&
      chunks <= kRowSyncChunks) {
    VAMD_MASK_DISPATCH(mask_dtype, M, {
      // occupancy of the instantiation that would be launched (mask type, gradient and weights change its registers)
      const void* k = grad_unscaled
          ? (is_weights ? (const void*)policy_kernel<true, M, true, true, true, -1, true>
                        : (const void*)policy_kernel<true, M, true, false, true, -1, true>)
          : (is_weights ? (const void*)policy_kernel<true, M, false, true, true, -1, true>
                        : (const void*)policy_kernel<true, M, false, false, true, -1, true>);
      rows_inline = rows * chunks <= resident_workgroups(k, kRcThreads) &&
                    can_vectorize(cols, {old_log_prob, log_prob, advantages, is_weights, grad_unscaled}, mask, sizeof(M));
    });
  }
  if (per_row && !rows_inline && chunks > 1 && chunks <= kWholeRowChunks) {
    // rows of two to four chunks: one 1024-thread workgroup per row, no pre-pass, then the fold
    bool whole_rows = false;
    VAMD_MASK_DISPATCH(mask_dtype, M, {
      whole_rows = can_vectorize(cols, {old_log_prob, log_prob, advantages, is_weights, grad_unscaled}, mask, sizeof(M));
    });
    if (whole_rows) {
      const float* tw = is_weights;  // GSPO: per token; GMPO: through the row sum of their logarithms
      const int tm = ap.mode == VAMD_AGG_TOKEN_MEAN;
#define VAMD_WR(G, W, K)                                                                                              \
  hipLaunchKernelGGL((policy_whole_row_kernel<M, G, W, K>), dim3((unsigned)rows), dim3(kWholeRowThreads), 0, s,      \
                     old_log_prob, log_prob, advantages, mk, tw, rows, cols, pp, tm, wk.partials, grad_unscaled)
#define VAMD_WR_K(G, W) \
  if (variant == VAMD_PL_GSPO) VAMD_WR(G, W, VAMD_PL_GSPO); else VAMD_WR(G, W, VAMD_PL_GEO_MEAN)
      VAMD_MASK_DISPATCH(mask_dtype, M, {
        const M* mk = static_cast<const M*>(mask);
        if (grad_unscaled) { if (tw) { VAMD_WR_K(true, true); } else { VAMD_WR_K(true, false); } }
        else { if (tw) { VAMD_WR_K(false, true); } else { VAMD_WR_K(false, false); } }
      });
#undef VAMD_WR_K
#undef VAMD_WR
      hipLaunchKernelGGL((fold_loss_kernel<5, kEpiPolicy>), dim3(1), dim3(kFoldThreads), 0, s, wk.partials, rows, 1,
                         cols, ap, coef_out, out);
      VAMD_LAUNCH_CHECK();
      return VAMD_OK;
    }
  }
  if (rows_inline) {
    pp.row_partials = row_area;
    pp.spin_limit = gate_spin_limit(kRowWaitSpins);
  } else if (variant == VAMD_PL_GSPO) {  // sequence-level log-ratio: per-row masked moments of log_prob - old_log_prob
    st = masked_moments_of_difference(log_prob, old_log_prob, mask, mask_dtype, rows, cols, 1,
                                      MomentOuts{row_area, nullptr, nullptr, nullptr, nullptr, 1}, workspace,
                                      reduce_workspace_bytes(rows, cols, 5), stream);
    if (st != VAMD_OK) return st;
    pp.row_moments = row_area;
  } else if (variant == VAMD_PL_GEO_MEAN) {
    pp.row_moments = row_area;
#define VAMD_GEO(V, W)                                                                                            \
  hipLaunchKernelGGL((geo_rows_kernel<V, M, W>), grid, block, 0, s, old_log_prob, log_prob, advantages, mk,       \
                     is_weights, cols, chunks, pp.nkl_lo, pp.nkl_hi, row_area)
    VAMD_MASK_DISPATCH(mask_dtype, M, {
      const bool vec = can_vectorize(cols, {old_log_prob, log_prob, advantages, is_weights}, mask, sizeof(M));
      const M* mk = static_cast<const M*>(mask);
      if (vec) { if (is_weights) VAMD_GEO(true, true); else VAMD_GEO(true, false); }
      else { if (is_weights) VAMD_GEO(false, true); else VAMD_GEO(false, false); }
    });
#undef VAMD_GEO
    token_weights = nullptr;  // already folded into the sequence loss
  }
  bool sep = rows * chunks > kInlineFoldRecords;  // fold the records in a launch of their own
  wk.totals = sep && totals_suffice(ap.mode);     // ... unless the launch totals are all the mode needs
  // the clipped PPO loss gets kernels of its own, the other variants share one with a per-token switch
#define VAMD_PL_LAUNCH(V, G, W, F, K, R)                                                                              \
  hipLaunchKernelGGL((policy_kernel<V, M, G, W, F, K, (R) && (V) && (F)>), grid, block, 0, s, old_log_prob, log_prob, advantages, mk, \
                     token_weights, rows, cols, chunks, pp, ap, wk, out, grad_unscaled, coef_out)
#define VAMD_PL(V, G, W, F)                                                           \
  if (variant == VAMD_PL_VANILLA) VAMD_PL_LAUNCH(V, G, W, F, VAMD_PL_VANILLA, false); \
  else if (rows_inline) VAMD_PL_LAUNCH(V, G, W, F, -1, true); /* rows_inline implies 16-byte accesses */ \
  else VAMD_PL_LAUNCH(V, G, W, F, -1, false)
#define VAMD_PL_GW(V, F)                                                                             \
  if (grad_unscaled) { if (token_weights) { VAMD_PL(V, true, true, F); } else { VAMD_PL(V, true, false, F); } } \
  else { if (token_weights) { VAMD_PL(V, false, true, F); } else { VAMD_PL(V, false, false, F); } }
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {old_log_prob, log_prob, advantages, token_weights, grad_unscaled}, mask,
                                   sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    sep = sep && vec;
    if (sep) { VAMD_PL_GW(true, false) }
    else if (vec) { VAMD_PL_GW(true, true) }
    else { VAMD_PL_GW(false, true) }
  });
  if (sep && !wk.totals)
    hipLaunchKernelGGL((fold_loss_kernel<5, kEpiPolicy>), dim3(1), dim3(kFoldThreads), 0, s, wk.partials, rows,
                       chunks, cols, ap, coef_out, out);
#undef VAMD_PL_GW
#undef VAMD_PL
#undef VAMD_PL_LAUNCH
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_value_loss_workspace_bytes(int64_t rows, int64_t cols) {
  return reduce_workspace_bytes(rows, cols, 3);
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
  Work wk = carve_work(workspace);
  const AggParams ap = make_agg(mode, 1.0, -1.0, -1.0, -1.0);
  const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
  bool sep = rows * chunks > kInlineFoldRecords;
  wk.totals = sep && totals_suffice(mode);
#define VAMD_VL(V, G, F)                                                                                     \
  hipLaunchKernelGGL((value_kernel<V, M, G, F>), grid, block, 0, s, vpreds, returns, values, mk, rows, cols, \
                     chunks, cliprange_value, ap, wk, out, grad_unscaled, coef_out)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {vpreds, returns, values, grad_unscaled}, mask, sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    sep = sep && vec;
    if (sep) { if (grad_unscaled) VAMD_VL(true, true, false); else VAMD_VL(true, false, false); }
    else if (vec) { if (grad_unscaled) VAMD_VL(true, true, true); else VAMD_VL(true, false, true); }
    else { if (grad_unscaled) VAMD_VL(false, true, true); else VAMD_VL(false, false, true); }
  });
  if (sep && !wk.totals)
    hipLaunchKernelGGL((fold_loss_kernel<3, kEpiValue>), dim3(1), dim3(kFoldThreads), 0, s, wk.partials, rows, chunks,
                       cols, ap, coef_out, out);
#undef VAMD_VL
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" int vamd_kl_penalty(const float* logprob, const float* ref_logprob, int64_t n, int kind,
                               int straight_through, float* kld, float* grad, void* stream) {
  VAMD_REQUIRE(n >= 0 && n < (1ll << 40), "kl_penalty: bad element count");
  VAMD_REQUIRE(kind >= VAMD_KL_K1 && kind <= VAMD_KL_K3, "kl_penalty: invalid estimator %d", kind);
  if (n == 0) return VAMD_OK;
  VAMD_REQUIRE(logprob && ref_logprob && (kld || grad), "kl_penalty: null pointer");
  hipLaunchKernelGGL(kl_elementwise_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), logprob, ref_logprob, n, kind, straight_through, kld, grad);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" size_t vamd_kl_loss_workspace_bytes(int64_t rows, int64_t cols) {
  return reduce_workspace_bytes(rows, cols, 2);
}

extern "C" int vamd_kl_loss_forward(const float* logprob, const float* ref_logprob, const void* mask, int mask_dtype,
                                    int64_t rows, int64_t cols, int kind, int straight_through, int mode,
                                    double dp_size, double batch_num_tokens, double global_batch_size,
                                    double loss_scale_factor, float* out, float* grad_unscaled, float* coef_out,
                                    void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_matrix("kl_loss", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(logprob && ref_logprob && mask && out, "kl_loss: null pointer");
  VAMD_REQUIRE(kind >= VAMD_KL_K1 && kind <= VAMD_KL_K3, "kl_loss: invalid estimator %d", kind);
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "kl_loss: invalid mode %d", mode);
  VAMD_REQUIRE(!grad_unscaled || coef_out, "kl_loss: grad output needs coef_out");
  if (!workspace || workspace_bytes < vamd_kl_loss_workspace_bytes(rows, cols)) {
    set_error("kl_loss: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  Work wk = carve_work(workspace);
  const AggParams ap = make_agg(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor);
  const dim3 grid((unsigned)(rows * chunks)), block(kRcThreads);
  bool sep = rows * chunks > kInlineFoldRecords;
  wk.totals = sep && totals_suffice(mode);
#define VAMD_KL(V, G, F)                                                                                       \
  hipLaunchKernelGGL((kl_loss_kernel<V, M, G, F>), grid, block, 0, s, logprob, ref_logprob, mk, rows, cols, chunks, \
                     kind, straight_through, ap, wk, out, grad_unscaled, coef_out)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {logprob, ref_logprob, grad_unscaled}, mask, sizeof(M));
    const M* mk = static_cast<const M*>(mask);
    sep = sep && vec;
    if (sep) { if (grad_unscaled) VAMD_KL(true, true, false); else VAMD_KL(true, false, false); }
    else if (vec) { if (grad_unscaled) VAMD_KL(true, true, true); else VAMD_KL(true, false, true); }
    else { if (grad_unscaled) VAMD_KL(false, true, true); else VAMD_KL(false, false, true); }
  });
  if (sep && !wk.totals)
    hipLaunchKernelGGL((fold_loss_kernel<2, kEpiKl>), dim3(1), dim3(kFoldThreads), 0, s, wk.partials, rows, chunks,
                       cols, ap, coef_out, out);
#undef VAMD_KL
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" size_t vamd_apply_kl_penalty_workspace_bytes(int64_t rows, int64_t cols) {
  return reduce_workspace_bytes(rows, cols, 2);
}

extern "C" int vamd_apply_kl_penalty(const float* scores, const float* logprob, const float* ref_logprob,
                                     const void* mask, int mask_dtype, int64_t rows, int64_t cols, int kind,
                                     float beta, float* token_level_rewards, float* current_kl, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  int st = check_matrix("apply_kl_penalty", rows, cols);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(scores && logprob && ref_logprob && mask && token_level_rewards && current_kl,
               "apply_kl_penalty: null pointer");
  VAMD_REQUIRE(kind >= VAMD_KL_K1 && kind <= VAMD_KL_K3, "apply_kl_penalty: invalid estimator %d", kind);
  if (!workspace || workspace_bytes < vamd_apply_kl_penalty_workspace_bytes(rows, cols)) {
    set_error("apply_kl_penalty: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(cols);
  const Work wk = carve_work(workspace);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(cols, {scores, logprob, ref_logprob, token_level_rewards}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((kl_reward_kernel<V, M>), dim3((unsigned)(rows * chunks)),
                                                 dim3(kRcThreads), 0, s, scores, logprob, ref_logprob,
                                                 static_cast<const M*>(mask), rows, cols, chunks, kind, beta, wk,
                                                 token_level_rewards, current_kl));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// ---------------------------------------------------------------------------------------------
extern "C" size_t vamd_grpo_workspace_bytes(int64_t batch, int64_t length, int64_t n_groups) {
  if (batch <= 0 || length <= 0 || n_groups <= 0) return 0;
  size_t b = reduce_workspace_bytes(batch, length, 1);
  b += 2 * align_up((size_t)batch * sizeof(float), 256);     // scores, scalars
  b += 2 * align_up((size_t)n_groups * sizeof(double), 256);  // mean, std (large-group-count path)
  return b;
}

extern "C" int vamd_group_mean_std(const float* scores, const int64_t* group_ids, int64_t n, int64_t n_groups,
                                   float eps, float* mean, float* std, float* count, void* stream) {
  VAMD_REQUIRE(scores && group_ids && mean && std && n > 0 && n_groups > 0, "group_mean_std: bad argument");
  hipLaunchKernelGGL(group_stats_kernel<float>, dim3((unsigned)((n_groups + 63) / 64)), dim3(64), 0,
                     static_cast<hipStream_t>(stream), scores, group_ids, n, n_groups, eps, 1, mean, std, count);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" size_t vamd_group_outcome_advantage_workspace_bytes(int64_t batch, int64_t length, int64_t n_groups) {
  if (batch <= 0 || length <= 0 || n_groups <= 0) return 0;
  // sized for the estimator that needs most: OPO runs a per-row moments pass (4 doubles per workgroup) first
  return vamd_grpo_workspace_bytes(batch, length, n_groups) - reduce_workspace_bytes(batch, length, 1) +
         reduce_workspace_bytes(batch, length, 4) + align_up((size_t)batch * 4 * sizeof(double), 256);
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
  // GRPO uses neither the wider partial records nor the per-row moments the general query reserves room for
  return vamd_group_outcome_advantage(rewards, mask, mask_dtype, group_ids, batch, length, n_groups, VAMD_ADV_GRPO,
                                      epsilon, norm_by_std, std_mode, 1.f, advantages, scores_out, workspace,
                                      vamd_group_outcome_advantage_workspace_bytes(batch, length, n_groups), stream);
}

extern "C" int vamd_group_outcome_advantage(const float* rewards, const void* mask, int mask_dtype,
                                            const int64_t* group_ids, int64_t batch, int64_t length,
                                            int64_t n_groups, int estimator, float epsilon, int norm_by_std,
                                            int std_mode, float f_norm, float* advantages, float* scores_out,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_matrix("group_outcome_advantage", batch, length);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(rewards && mask && group_ids && advantages && n_groups > 0, "group_outcome_advantage: bad argument");
  VAMD_REQUIRE(estimator >= VAMD_ADV_GRPO && estimator <= VAMD_ADV_GRPO_PASSK, "group_outcome_advantage: invalid estimator %d",
               estimator);
  VAMD_REQUIRE(estimator == VAMD_ADV_GRPO || n_groups <= kGrpoLdsGroups,
               "group_outcome_advantage: estimators other than GRPO support at most %d groups", kGrpoLdsGroups);
  VAMD_REQUIRE(estimator != VAMD_ADV_GPG || f_norm != 0.f, "group_outcome_advantage: f_norm must not be 0");
  if (!workspace || workspace_bytes < vamd_group_outcome_advantage_workspace_bytes(batch, length, n_groups)) {
    set_error("group_outcome_advantage: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (int)chunks_of(length);
  const Work wk = carve_work(workspace);
  const bool opo = estimator == VAMD_ADV_OPO;
  Carver carve(static_cast<char*>(workspace) + reduce_workspace_bytes(batch, length, opo ? 4 : 1));
  GrpoArgs ga;
  ga.gid = group_ids;
  ga.rows = batch;
  ga.n_groups = n_groups;
  ga.eps = epsilon;
  ga.norm_by_std = norm_by_std;
  ga.std_mode = std_mode;
  ga.estimator = estimator;
  ga.f_norm = f_norm;
  ga.scores = carve.take<float>((size_t)batch);
  float* scalars = carve.take<float>((size_t)batch);
  ga.scalars = scores_out ? scores_out : scalars;
  ga.mean = carve.take<double>((size_t)n_groups);
  ga.stdv = carve.take<double>((size_t)n_groups);
  ga.row_moments = nullptr;
  if (opo) {  // response lengths: per-row masked moments of the rewards, slot 0 = sum(mask)
    double* row_moments = carve.take<double>((size_t)batch * 4);
    ga.row_moments = row_moments;
    st = vamd_masked_moments(rewards, mask, mask_dtype, batch, length, 1, row_moments, workspace,
                             reduce_workspace_bytes(batch, length, 4), stream);
    if (st != VAMD_OK) return st;
  }
  const bool may_wait = waiting_kernels_allowed();
  if (may_wait && estimator == VAMD_ADV_GRPO && batch <= kGrpoRowsLimit) {
    GrpoRowsArgs ra;
    ra.rewards = rewards;
    ra.mask = mask;
    ra.gid = group_ids;
    ra.rows = batch;
    ra.cols = length;
    ra.chunks = chunks;
    ra.eps = epsilon;
    ra.norm_by_std = norm_by_std;
    ra.std_mode = std_mode;
    ra.scores = ga.scores;
    ra.scalars = scores_out;
    ra.out = advantages;
    ra.ticket = wk.ticket;
    ra.spin_limit = gate_spin_limit(kGateSpinLimit);
    VAMD_MASK_DISPATCH(mask_dtype, M, {
      const bool vec = can_vectorize(length, {rewards, advantages}, mask, sizeof(M));
      auto go = [&](auto kernel) {
        const int64_t grid = balanced_waiting_grid(batch, resident_workgroups(reinterpret_cast<const void*>(kernel), kRcThreads));
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kRcThreads), 0, s, ra);
      };
      if (vec) go(grpo_rows_kernel<true, M>);
      else go(grpo_rows_kernel<false, M>);
    });
    VAMD_LAUNCH_CHECK();
    return VAMD_OK;
  }
  // records per row of the row-sum pass: one per chunk, or one per row once there are enough rows to fill the device
  const int span = (batch >= 1024 && chunks > 1) ? chunks : 1;
  const int rec_chunks = (chunks + span - 1) / span;
  {
    const bool vec = can_vectorize(length, {rewards}, nullptr, 0);
    const bool lds_stats = n_groups <= kGrpoLdsGroups;
    const dim3 grid((unsigned)(batch * rec_chunks));
    if (n_groups <= kGrpoInlineGroups && batch * rec_chunks <= kInlineFoldRecords) {
      VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((grpo_rowsum_kernel<V, true>), grid, dim3(kRcThreads), 0, s,
                                                   rewards, length, rec_chunks, span, wk, ga));
    } else {
      VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((grpo_rowsum_kernel<V, false>), grid, dim3(kRcThreads), 0, s,
                                                   rewards, length, rec_chunks, span, wk, ga));
      if (lds_stats) {
        VAMD_LAUNCH_CHECK();
        if (estimator == VAMD_ADV_GRPO)
          hipLaunchKernelGGL(grpo_scalars_kernel_lds<VAMD_ADV_GRPO>, dim3(1), dim3(kGrpoTailThreads), 0, s,
                             wk.partials, rec_chunks, ga);
        else
          hipLaunchKernelGGL(grpo_scalars_kernel_lds<-1>, dim3(1), dim3(kGrpoTailThreads), 0, s, wk.partials,
                             rec_chunks, ga);
      }
    }
    VAMD_LAUNCH_CHECK();
  }
  if (n_groups > kGrpoLdsGroups) {
    hipLaunchKernelGGL(rowsum_finalize_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, wk.partials,
                       batch, rec_chunks, ga.scores);
    VAMD_LAUNCH_CHECK();
    hipLaunchKernelGGL(group_stats_kernel<double>, dim3((unsigned)((n_groups + 63) / 64)), dim3(64), 0, s, ga.scores,
                       group_ids, batch, n_groups, epsilon, std_mode, ga.mean, ga.stdv, (float*)nullptr);
    VAMD_LAUNCH_CHECK();
    hipLaunchKernelGGL(grpo_scalars_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, ga.scores,
                       group_ids, batch, ga.mean, ga.stdv, epsilon, norm_by_std, ga.scalars);
    VAMD_LAUNCH_CHECK();
  }
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(length, {advantages}, mask, sizeof(M));
    VAMD_VEC_DISPATCH(vec, V, hipLaunchKernelGGL((broadcast_rows_kernel<V, M>), dim3((unsigned)(batch * chunks)),
                                                 dim3(kRcThreads), 0, s, ga.scalars, static_cast<const M*>(mask),
                                                 length, chunks, advantages));
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
