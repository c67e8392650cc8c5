// Rollout-correction importance weights and off-policy diagnostics in one pass.
//
// compute_rollout_correction_weights + compute_is_metrics + compute_offpolicy_metrics
// (verl/trainer/ppo/rollout_corr_helper.py:481-712, 835-937) evaluate about thirty masked reductions
// over old_log_prob, rollout_log_prob and the response mask, each followed by .item().  Here every
// (row, 4096-column chunk) workgroup reads the three tensors once, writes the truncated token-level
// weights if those are asked for, and leaves a record of partial sums; a single-workgroup launch then
// folds the records into per-sequence quantities and the metric vector (a launch of its own, so that
// the fold's registers are not charged to every wavefront of the streaming kernel).  Sequence-level
// weights (one per row, known only after the fold) are broadcast by a further small launch, as is the
// batch normalisation of token-level weights.  The response mask is taken as binary.
#include "rowchunk.h"

namespace vamd {

constexpr float kSafetyBound = 20.f;  // rollout_corr_helper.py:75

enum {
  kRcM = 0,    // sum of the mask
  kRcOld,      // sum old_log_prob m
  kRcRoll,     // sum rollout_log_prob m
  kRcD,        // sum (old - rollout) m
  kRcK3,       // sum (exp(d) - d - 1) m
  kRcRho2,     // sum exp(clamp(d))^2 m
  kRcW,        // token level: sum w m,  w = exp(clamp(d))
  kRcC,        // sum clamp(w, 1/thr, thr) m
  kRcC2,       // sum clamp(w, 1/thr, thr)^2 m
  kRcTrunc,    // sum min(w, thr) m
  kRcHigh,     // number of valid tokens with w > thr
  kRcLow,      // number of valid tokens with w < 1/thr
  kRcWMax,     // max w over the valid tokens
  kRcWMinNeg,  // -(min w over the valid tokens)
  kRcRec
};
constexpr int kRcSums = kRcWMax;

struct RcArgs {
  const float *old_lp, *roll_lp;  // roll_lp may be null: only the training perplexity is produced
  int64_t rows, cols;
  int chunks;          // records per row: spans of `span` 4096-column chunks
  int span;
  int level;  // VAMD_IS_*
  float thr, lower;
  int normalize;
  float* weights;      // [rows][cols] or null
  double* records;     // kRcRec slots per (row, chunk) workgroup, slot-major
  float* row_weight;   // [rows]: sequence-level weight, truncated (the broadcast divides by `factor`)
  double* shares;      // per workgroup of the fold launch: its 26 sums and 9 maxima
  unsigned* fold_counter;  // arrivals of the fold launch's workgroups; the streaming pass clears it
  float* factor;       // [1]: batch-normalisation divisor for the token-level weights (1 when not applied)
  double* out;         // [VAMD_RC_COUNT]
};

template <int NV, int NT>
__device__ __forceinline__ void block_max_f64(double (&v)[NV], double* smem) {
  block_reduce<NV, NT>(v, smem, MaxOp());
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void rollout_stats_kernel(RcArgs a, const M* __restrict__ mask) {
  const int64_t row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  if (blockIdx.x == 0 && threadIdx.x == 0) a.fold_counter[0] = 0u;
  // A workgroup walks a.span consecutive 4096-column chunks of its row and leaves one record (a.chunks counts
  // those spans): the workgroup reduction of a record this wide costs more vector-ALU time than streaming one chunk.
  double acc[kRcSums];
#pragma unroll
  for (int i = 0; i < kRcSums; ++i) acc[i] = 0.0;
  float wmax = -__builtin_inff(), wmin = __builtin_inff();
  for (int u = 0; u < a.span; ++u) {
    const ChunkPos pos(row, chunk * a.span + u, a.cols);
    float s[kRcSums];  // per-thread partials over 16 elements in fp32, widened after every chunk
#pragma unroll
    for (int i = 0; i < kRcSums; ++i) s[i] = 0.f;
    float o[kGroups][4], r[kGroups][4], m[kGroups][4];
    const bool streaming = streams_past_caches(a.rows * a.cols);  // the grid counts spans of chunks, not chunks
    load_groups<VEC>(a.old_lp, pos, o, streaming);
    if (a.roll_lp) load_groups<VEC>(a.roll_lp, pos, r, streaming);
    load_mask_groups<VEC>(mask, pos, m, streaming);
#pragma unroll
    for (int k = 0; k < kGroups; ++k) {
      float wt[4];  // the group's weights leave as soon as they exist: 16 registers fewer than holding the chunk's
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wt[e] = 0.f;
        if (e >= pos.valid[k] || m[k][e] == 0.f) continue;
        s[kRcM] += 1.f;
        s[kRcOld] += o[k][e];
        if (!a.roll_lp) continue;
        const float d = o[k][e] - r[k][e];
        const float dc = fminf(fmaxf(d, -kSafetyBound), kSafetyBound);
        const float w = expf(dc);
        const float ed = d == dc ? w : expf(d);  // one exponential per token unless the clamp acted
        s[kRcRoll] += r[k][e];
        s[kRcD] += d;
        s[kRcK3] += ed - d - 1.f;
        s[kRcRho2] += w * w;
        if (a.level == VAMD_IS_TOKEN) {
          const float c = fminf(fmaxf(w, a.lower), a.thr);
          const float t = fminf(w, a.thr);
          s[kRcW] += w;
          s[kRcC] += c;
          s[kRcC2] += c * c;
          s[kRcTrunc] += t;
          s[kRcHigh] += w > a.thr ? 1.f : 0.f;
          s[kRcLow] += w < a.lower ? 1.f : 0.f;
          wmax = fmaxf(wmax, w);
          wmin = fminf(wmin, w);
          wt[e] = t;
        }
      }
      if (a.level == VAMD_IS_TOKEN && a.weights && pos.valid[k] > 0)
        st4<VEC>(a.weights, pos.idx[k], pos.valid[k], wt, streaming);
    }
#pragma unroll
    for (int i = 0; i < kRcSums; ++i) acc[i] += (double)s[i];
  }
  __shared__ double smem[24 * 4];
  block_sum<kRcSums, kRcThreads>(acc, smem);
  double ext[2] = {wmax, -(double)wmin};
  block_max_f64<2, kRcThreads>(ext, smem);
  if (threadIdx.x == 0) {
    double rec[kRcRec];
#pragma unroll
    for (int i = 0; i < kRcSums; ++i) rec[i] = acc[i];
    rec[kRcWMax] = ext[0];
    rec[kRcWMinNeg] = ext[1];
    store_record<kRcRec>(a.records, row, chunk, a.rows, a.chunks, rec);
  }
}

constexpr int kFoldRows = 4;          // rows per thread and trip of the fold launch
constexpr int kRcFoldThreads = 128;   // a workgroup of the fold launch takes up to kFoldRows * kRcFoldThreads rows

// records -> per-sequence quantities -> the metric vector (and the per-row weights): one row per thread, the
// workgroups' totals combined by the last of them to finish.
template <int NT>
__global__ __launch_bounds__(NT) void rollout_fold_kernel(RcArgs a) {
  const double inf = __longlong_as_double(0x7ff0000000000000ll);
  __shared__ double stage[(NT / 64) * 26 * kWidePitch];
  enum {
    tM = 0, tD, tK3, tRho2, tW, tC, tC2, tTrunc, tHigh, tLow,         // token totals
    tTrainPpl, tTrainLog, tRollPpl, tRollLog, tGap, tGapAbs, tRatio, tChiSeq,  // sums over rows
    tSeq, tSeq2, tSeqHigh, tSeqLow,                                   // per-sequence mean weight
    tLogHigh, tLogLow,                                                // sequence level: thresholds in log space
    tAlive, tSeqTrunc,                                                // rows with tokens; their truncated weights
    tN
  };
  enum { xGap = 0, xGapMinNeg, xW, xWMinNeg, xSeq, xSeqMinNeg, xDev, xLog, xLogMinNeg, xN };
  double t[tN], x[xN];
#pragma unroll
  for (int i = 0; i < tN; ++i) t[i] = 0;
#pragma unroll
  for (int i = 0; i < xN; ++i) x[i] = -inf;
  const float log_hi = logf(a.thr), log_lo = logf(a.lower);
  const bool seq_level = a.level == VAMD_IS_SEQUENCE;
  // kFoldRows rows per thread and trip, their records in flight together: few wavefronts keep the workgroup
  // reductions below short, and the loads of a trip are one round trip to memory whatever their number
  for (int64_t r0 = (int64_t)blockIdx.x * NT * kFoldRows + threadIdx.x; r0 < a.rows;
       r0 += (int64_t)gridDim.x * NT * kFoldRows) {
    int64_t rr[kFoldRows];
    bool have[kFoldRows];
#pragma unroll
    for (int k = 0; k < kFoldRows; ++k) {
      rr[k] = r0 + (int64_t)k * NT;
      have[k] = rr[k] < a.rows;
    }
    double rec[kFoldRows][kRcRec];
    fold_row_records<kRcRec, kRcSums, kFoldRows, false, 1>(a.records, rr, have, a.rows, a.chunks, rec);
#pragma unroll
    for (int k = 0; k < kFoldRows; ++k) {
      if (!have[k]) break;
      const int64_t r = rr[k];
      const double* f = rec[k];
      x[xW] = fmax(x[xW], rec[k][kRcWMax]);
      x[xWMinNeg] = fmax(x[xWMinNeg], rec[k][kRcWMinNeg]);
      const float Mi = (float)f[kRcM];
      const float train = (float)f[kRcOld] / (Mi + 1e-8f);  // masked_mean(., axis=-1)
      t[tM] += f[kRcM]; t[tD] += f[kRcD]; t[tK3] += f[kRcK3]; t[tRho2] += f[kRcRho2];
      t[tTrainPpl] += (double)expf(-train);
      t[tTrainLog] += (double)(-train);
      if (Mi > 0.f) t[tAlive] += 1.0;
      if (!a.roll_lp) continue;
      const float roll = (float)f[kRcRoll] / (Mi + 1e-8f);
      const float gap = roll - train;
      const float dsum = (float)f[kRcD];
      const float dsafe = fminf(fmaxf(dsum, -kSafetyBound), kSafetyBound);
      t[tRollPpl] += (double)expf(-roll);
      t[tRollLog] += (double)(-roll);
      t[tGap] += (double)gap;
      t[tGapAbs] += (double)fabsf(gap);
      t[tRatio] += (double)expf(gap);
      t[tChiSeq] += (double)expf(2.f * dsafe);
      x[xGap] = fmax(x[xGap], (double)gap);
      x[xGapMinNeg] = fmax(x[xGapMinNeg], -(double)gap);
      float seq = 0.f;  // masked_mean(weights, axis=-1) of the untruncated weights
      if (a.level == VAMD_IS_TOKEN) {
        t[tW] += f[kRcW]; t[tC] += f[kRcC]; t[tC2] += f[kRcC2]; t[tTrunc] += f[kRcTrunc];
        t[tHigh] += f[kRcHigh]; t[tLow] += f[kRcLow];
        seq = (float)f[kRcW] / (Mi + 1e-8f);
      } else if (seq_level) {
        const float w = expf(dsafe);
        const float c = fminf(fmaxf(w, a.lower), a.thr);
        const float tr = fminf(w, a.thr);
        t[tW] += (double)w * f[kRcM]; t[tC] += (double)c * f[kRcM]; t[tC2] += (double)c * (double)c * f[kRcM];
        t[tLogHigh] += dsum > log_hi ? 1.0 : 0.0;
        t[tLogLow] += dsum < log_lo ? 1.0 : 0.0;
        x[xLog] = fmax(x[xLog], (double)dsum);
        x[xLogMinNeg] = fmax(x[xLogMinNeg], -(double)dsum);
        seq = w * Mi / (Mi + 1e-8f);
        if (Mi > 0.f) t[tSeqTrunc] += (double)(tr * Mi / (Mi + 1e-8f));
        a.row_weight[r] = tr;
      }
      if (a.level != VAMD_IS_NONE) {
        t[tSeq] += (double)seq;
        t[tSeq2] += (double)seq * (double)seq;
        t[tSeqHigh] += seq > a.thr ? 1.0 : 0.0;
        t[tSeqLow] += seq < a.lower ? 1.0 : 0.0;
        x[xSeq] = fmax(x[xSeq], (double)seq);
        x[xSeqMinNeg] = fmax(x[xSeqMinNeg], -(double)seq);
        x[xDev] = fmax(x[xDev], (double)fabsf(seq - 1.f));
      }
    }
  }
  static_assert(tN <= 26 && xN <= 26, "the staging area is sized for 26 values");
  block_reduce_wide<tN, NT>(t, stage, SumOp());
  block_reduce_wide<xN, NT>(x, stage, MaxOp());
  if (!fold_across_workgroups<tN, xN, NT>(t, x, a.shares, a.fold_counter, stage)) return;
  if (threadIdx.x == 0) {
    double* o = a.out;
    const double B = (double)a.rows, Mt = t[tM];
    const double den = (double)((float)Mt + 1e-8f);  // masked_mean over everything
    o[VAMD_RC_VALID_TOKENS] = Mt;
    o[VAMD_RC_TRAINING_PPL] = t[tTrainPpl] / B;
    o[VAMD_RC_TRAINING_LOG_PPL] = t[tTrainLog] / B;
    o[VAMD_RC_KL] = -t[tD] / den;
    o[VAMD_RC_K3_KL] = t[tK3] / den;
    o[VAMD_RC_ROLLOUT_PPL] = t[tRollPpl] / B;
    o[VAMD_RC_ROLLOUT_LOG_PPL] = t[tRollLog] / B;
    o[VAMD_RC_LOG_PPL_DIFF] = t[tGap] / B;
    o[VAMD_RC_LOG_PPL_ABS_DIFF] = t[tGapAbs] / B;
    o[VAMD_RC_LOG_PPL_DIFF_MAX] = x[xGap];
    o[VAMD_RC_LOG_PPL_DIFF_MIN] = -x[xGapMinNeg];
    o[VAMD_RC_PPL_RATIO] = t[tRatio] / B;
    o[VAMD_RC_CHI2_TOKEN] = t[tRho2] / den - 1.0;
    o[VAMD_RC_CHI2_SEQ] = t[tChiSeq] / B - 1.0;
    float divisor = 1.f;
    if (a.level != VAMD_IS_NONE) {
      const double mean_c = t[tC] / den, mean_c2 = t[tC2] / den;
      o[VAMD_RC_IS_MEAN] = t[tW] / den;
      if (seq_level) {
        o[VAMD_RC_IS_MAX] = (double)expf(fminf((float)x[xLog], kSafetyBound));
        o[VAMD_RC_IS_MIN] = (double)expf((float)(-x[xLogMinNeg]));
        o[VAMD_RC_IS_FRACTION_HIGH] = t[tLogHigh] / B;
        o[VAMD_RC_IS_FRACTION_LOW] = t[tLogLow] / B;
      } else {
        o[VAMD_RC_IS_MAX] = x[xW];
        o[VAMD_RC_IS_MIN] = -x[xWMinNeg];
        o[VAMD_RC_IS_FRACTION_HIGH] = t[tHigh] / den;
        o[VAMD_RC_IS_FRACTION_LOW] = t[tLow] / den;
      }
      o[VAMD_RC_IS_STD] = Mt > 1.0 ? sqrt(fmax(mean_c2 - mean_c * mean_c, 0.0)) : 0.0;
      o[VAMD_RC_IS_ESS] = (mean_c + 1e-8) * (mean_c + 1e-8) / mean_c2;
      o[VAMD_RC_IS_SEQ_MEAN] = t[tSeq] / B;
      o[VAMD_RC_IS_SEQ_STD] = B > 1.0 ? sqrt(fmax((t[tSeq2] - t[tSeq] * t[tSeq] / B) / (B - 1.0), 0.0)) : 0.0;
      o[VAMD_RC_IS_SEQ_MAX] = x[xSeq];
      o[VAMD_RC_IS_SEQ_MIN] = -x[xSeqMinNeg];
      o[VAMD_RC_IS_SEQ_MAX_DEVIATION] = x[xDev];
      o[VAMD_RC_IS_SEQ_FRACTION_HIGH] = t[tSeqHigh] / B;
      o[VAMD_RC_IS_SEQ_FRACTION_LOW] = t[tSeqLow] / B;
      o[VAMD_RC_IS_BATCH_NORM_FACTOR] = 1.0;
      if (a.normalize) {
        const double mean = seq_level ? t[tSeqTrunc] / fmax(t[tAlive], 1e-8) : t[tTrunc] / den;
        if (mean > 1e-8) {
          divisor = (float)mean;
          o[VAMD_RC_IS_BATCH_NORM_FACTOR] = mean;
        }
      }
    }
    a.factor[0] = divisor;
  }
}

// weights[i][t] = row_weight[i] / factor * mask[i][t]  (the division is skipped when the factor is 1)
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void rollout_broadcast_kernel(const float* __restrict__ row_weight,
                                                                       const float* __restrict__ factor,
                                                                       const M* __restrict__ mask, int64_t cols,
                                                                       int chunks, float* __restrict__ weights) {
  const int64_t row = blockIdx.x / chunks;
  const ChunkPos pos(row, blockIdx.x % chunks, cols);
  float m[kGroups][4];
  load_mask_groups<VEC>(mask, pos, m);
  const float f = factor[0];
  const float w = f != 1.f ? row_weight[row] / f : row_weight[row];
#pragma unroll
  for (int k = 0; k < kGroups; ++k)
#pragma unroll
    for (int e = 0; e < 4; ++e) m[k][e] = m[k][e] != 0.f ? w : 0.f;
  store_groups<VEC>(weights, pos, m);
}

// weights /= factor[0] (skipped when the factor is 1)
__global__ __launch_bounds__(256) void rollout_divide_kernel(float* __restrict__ weights, int64_t n,
                                                             const float* __restrict__ factor) {
  const float f = factor[0];
  if (f == 1.f) return;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (i + e < n) weights[i + e] = weights[i + e] / f;
}

}  // namespace vamd

using namespace vamd;

// workgroups of the fold launch (at most 256), each leaving 26 sums and 9 maxima
constexpr size_t kRcShareSlots = 26 + 9;
static unsigned rc_fold_workgroups(int64_t batch) {
  const int64_t per = (int64_t)kFoldRows * kRcFoldThreads;
  const int64_t n = (batch + per - 1) / per;
  return (unsigned)(n < 1 ? 1 : (n > 256 ? 256 : n));
}

extern "C" size_t vamd_rollout_correction_workspace_bytes(int64_t batch, int64_t length) {
  if (batch <= 0 || length <= 0) return 0;
  return align_up((size_t)batch * chunks_of(length) * kRcRec * sizeof(double), 256) +
         align_up((size_t)batch * sizeof(float), 256) + 256 +
         align_up((size_t)rc_fold_workgroups(batch) * kRcShareSlots * sizeof(double), 256) + 256;
}

extern "C" int vamd_rollout_correction(const float* old_log_prob, const float* rollout_log_prob, const void* mask,
                                       int mask_dtype, int64_t batch, int64_t length, int level, float threshold,
                                       int batch_normalize, float* weights, double* metrics, void* workspace,
                                       size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "rollout_correction: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31), "rollout_correction: too many workgroups");
  VAMD_REQUIRE(old_log_prob && mask && metrics, "rollout_correction: null pointer");
  VAMD_REQUIRE(level >= VAMD_IS_NONE && level <= VAMD_IS_SEQUENCE, "rollout_correction: invalid level %d", level);
  VAMD_REQUIRE(level == VAMD_IS_NONE || (rollout_log_prob && weights),
               "rollout_correction: importance weights need rollout_log_prob and an output buffer");
  VAMD_REQUIRE(level == VAMD_IS_NONE || threshold > 0.f, "rollout_correction: threshold must be positive");
  if (!workspace || workspace_bytes < vamd_rollout_correction_workspace_bytes(batch, length)) {
    set_error("rollout_correction: workspace too small");
    return VAMD_EWORKSPACE;
  }
  RcArgs a;
  a.old_lp = old_log_prob; a.roll_lp = rollout_log_prob;
  a.rows = batch; a.cols = length;
  a.span = record_span(batch, (int)chunks_of(length));
  a.chunks = ((int)chunks_of(length) + a.span - 1) / a.span;
  a.level = level; a.thr = threshold; a.lower = level == VAMD_IS_NONE ? 0.f : 1.0f / threshold;
  a.normalize = batch_normalize;
  a.weights = weights;
  Carver carve(workspace);
  a.records = carve.take<double>((size_t)batch * a.chunks * kRcRec);
  a.row_weight = carve.take<float>((size_t)batch);
  a.factor = carve.take<float>(1);
  a.shares = carve.take<double>((size_t)rc_fold_workgroups(batch) * kRcShareSlots);
  a.fold_counter = carve.take<unsigned>(1);
  a.out = metrics;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(batch * a.chunks)), block(kRcThreads);
  const int col_chunks = (int)chunks_of(length);  // the broadcast takes one 4096-column chunk per workgroup
  const dim3 cols_grid((unsigned)(batch * col_chunks));
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    const bool vec = can_vectorize(length, {old_log_prob, rollout_log_prob, weights}, mask, sizeof(M));
    if (vec)
      hipLaunchKernelGGL((rollout_stats_kernel<true, M>), grid, block, 0, s, a, mk);
    else
      hipLaunchKernelGGL((rollout_stats_kernel<false, M>), grid, block, 0, s, a, mk);
    hipLaunchKernelGGL(rollout_fold_kernel<kRcFoldThreads>, dim3(rc_fold_workgroups(batch)), dim3(kRcFoldThreads), 0,
                       s, a);
    if (level == VAMD_IS_SEQUENCE) {
      if (vec)
        hipLaunchKernelGGL((rollout_broadcast_kernel<true, M>), cols_grid, block, 0, s, a.row_weight, a.factor, mk,
                           length, col_chunks, weights);
      else
        hipLaunchKernelGGL((rollout_broadcast_kernel<false, M>), cols_grid, block, 0, s, a.row_weight, a.factor, mk,
                           length, col_chunks, weights);
    }
  });
  if (level == VAMD_IS_TOKEN && batch_normalize) {
    const int64_t n = batch * length;
    hipLaunchKernelGGL(rollout_divide_kernel, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, s, weights, n,
                       a.factor);
  }
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

// =============================================================================================================
// Rejection sampling (compute_rollout_rejection_mask, rollout_corr_helper.py:163-357).
//
// Two streaming passes with the decisions that need a whole sequence taken between them on the host, from a
// [batch]-sized table: the first pass leaves, per (row, chunk), the sums and maxima of the three divergence
// estimates k1 = -r, k2 = r^2 / 2, k3 = exp(r) - 1 - r (r = the log ratio clamped to +-20); the host folds the
// chunks, evaluates the sequence-level options (sum / mean / max against their bounds) and hands back one keep flag
// per row; the second pass applies the token-level options and that flag, writes the new mask in the element
// type of the old one and leaves the per-(row, chunk) counts the token-level metrics are made of.
// =============================================================================================================
namespace vamd {

enum { kRsCount = 0, kRsK1, kRsK2, kRsK3, kRsK2Max, kRsK3Max, kRsRowSlots };
enum { kRsSum = 0, kRsMax, kRsMinNeg, kRsHigh, kRsLow, kRsClamp, kRsClamp2, kRsRejected, kRsOptionSlots };
constexpr int kRsMaxTokenOptions = 3;

__device__ __forceinline__ void rs_estimates(float old_lp, float roll_lp, float (&k)[3]) {
  const float r = fminf(fmaxf(old_lp - roll_lp, -kSafetyBound), kSafetyBound);
  k[0] = -r;
  k[1] = 0.5f * r * r;
  k[2] = expf(r) - 1.f - r;
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void rs_rows_kernel(const float* __restrict__ old_lp,
                                                             const float* __restrict__ roll_lp,
                                                             const M* __restrict__ mask, int64_t rows, int64_t cols,
                                                             int chunks, double* __restrict__ records) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float o[kGroups][4], r[kGroups][4], m[kGroups][4];
  load_groups<VEC>(old_lp, pos, o);
  load_groups<VEC>(roll_lp, pos, r);
  load_mask_groups<VEC>(mask, pos, m);
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  float top[2] = {-__builtin_inff(), -__builtin_inff()};
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= pos.valid[g] || m[g][e] == 0.f) continue;
      float k[3];
      rs_estimates(o[g][e], r[g][e], k);
      s[0] += 1.f;
      s[1] += k[0]; s[2] += k[1]; s[3] += k[2];
      top[0] = fmaxf(top[0], k[1]);
      top[1] = fmaxf(top[1], k[2]);
    }
  __shared__ double smem[4 * 4];
  double acc[4] = {s[0], s[1], s[2], s[3]};
  block_sum<4, kRcThreads>(acc, smem);
  double ext[2] = {top[0], top[1]};
  block_max_f64<2, kRcThreads>(ext, smem);
  if (threadIdx.x == 0) {
    const double rec[kRsRowSlots] = {acc[0], acc[1], acc[2], acc[3], ext[0], ext[1]};
#pragma unroll
    for (int i = 0; i < kRsRowSlots; ++i) records[record_at(i, row, chunk, rows, chunks)] = rec[i];
  }
}

struct RsOptions {
  int n;                                  // token-level options, 0..3
  int estimator[kRsMaxTokenOptions];      // 0 k1, 1 k2, 2 k3
  float lower[kRsMaxTokenOptions];        // keep rule and metric thresholds (k1: logs of the ratio bounds)
  float upper[kRsMaxTokenOptions];
  int two_sided[kRsMaxTokenOptions];      // k1: keep inside [lower, upper]; others: keep below upper
};

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void rs_apply_kernel(const float* __restrict__ old_lp,
                                                              const float* __restrict__ roll_lp,
                                                              const M* __restrict__ mask,
                                                              const uint8_t* __restrict__ row_keep, int64_t rows,
                                                              int64_t cols, int chunks, RsOptions opt,
                                                              M* __restrict__ new_mask, double* __restrict__ records) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float o[kGroups][4], r[kGroups][4], m[kGroups][4];
  load_groups<VEC>(old_lp, pos, o);
  load_groups<VEC>(roll_lp, pos, r);
  load_mask_groups<VEC>(mask, pos, m);
  const bool row_ok = row_keep[row] != 0;
  float s[kRsMaxTokenOptions][kRsOptionSlots];
#pragma unroll
  for (int j = 0; j < kRsMaxTokenOptions; ++j)
#pragma unroll
    for (int i = 0; i < kRsOptionSlots; ++i) s[j][i] = (i == kRsMax || i == kRsMinNeg) ? -__builtin_inff() : 0.f;
  float rejected = 0.f;
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    M out[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float k[3];
      rs_estimates(o[g][e], r[g][e], k);
      bool keep = row_ok;
      const bool in = e < pos.valid[g] && m[g][e] != 0.f;
#pragma unroll
      for (int j = 0; j < kRsMaxTokenOptions; ++j) {
        if (j >= opt.n) break;
        const float v = opt.estimator[j] == 0 ? k[0] : (opt.estimator[j] == 1 ? k[1] : k[2]);
        const bool ok = opt.two_sided[j] ? (v >= opt.lower[j] && v <= opt.upper[j]) : (v <= opt.upper[j]);
        keep = keep && ok;
        if (in) {
          const float c = fminf(fmaxf(v, opt.two_sided[j] ? opt.lower[j] : 0.f), opt.upper[j]);
          s[j][kRsSum] += v;
          s[j][kRsMax] = fmaxf(s[j][kRsMax], v);
          s[j][kRsMinNeg] = fmaxf(s[j][kRsMinNeg], -v);
          s[j][kRsHigh] += v > opt.upper[j] ? 1.f : 0.f;
          s[j][kRsLow] += (opt.two_sided[j] && v < opt.lower[j]) ? 1.f : 0.f;
          s[j][kRsClamp] += c;
          s[j][kRsClamp2] += c * c;
          s[j][kRsRejected] += ok ? 0.f : 1.f;
        }
      }
      if (in && !keep) rejected += 1.f;
      // response_mask * combined keep, in the mask's own element type; masked-out positions keep their 0
      out[e] = keep ? static_cast<M>(m[g][e]) : static_cast<M>(0);
    }
    if (pos.valid[g] > 0) {
      if constexpr (VEC) {
        struct alignas(sizeof(M) * 4) Pack { M v[4]; };
        Pack p;
#pragma unroll
        for (int e = 0; e < 4; ++e) p.v[e] = out[e];
        *reinterpret_cast<Pack*>(new_mask + pos.idx[g]) = p;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (e < pos.valid[g]) new_mask[pos.idx[g] + e] = out[e];
      }
    }
  }
  __shared__ double smem[8 * 4];
  double rej[1] = {rejected};
  block_sum<1, kRcThreads>(rej, smem);
  if (threadIdx.x == 0) records[record_at(0, row, chunk, rows, chunks)] = rej[0];
#pragma unroll
  for (int j = 0; j < kRsMaxTokenOptions; ++j) {
    if (j >= opt.n) break;
    double sums[6] = {s[j][kRsSum], s[j][kRsHigh], s[j][kRsLow], s[j][kRsClamp], s[j][kRsClamp2], s[j][kRsRejected]};
    block_sum<6, kRcThreads>(sums, smem);
    double ext[2] = {s[j][kRsMax], s[j][kRsMinNeg]};
    block_max_f64<2, kRcThreads>(ext, smem);
    if (threadIdx.x == 0) {
      const double rec[kRsOptionSlots] = {sums[0], ext[0], ext[1], sums[1], sums[2], sums[3], sums[4], sums[5]};
#pragma unroll
      for (int i = 0; i < kRsOptionSlots; ++i)
        records[record_at(1 + j * kRsOptionSlots + i, row, chunk, rows, chunks)] = rec[i];
    }
  }
}

}  // namespace vamd

extern "C" int64_t vamd_rollout_rs_chunks(int64_t length) { return chunks_of(length); }

extern "C" int vamd_rollout_rs_row_stats(const float* old_log_prob, const float* rollout_log_prob, const void* mask,
                                         int mask_dtype, int64_t batch, int64_t length, double* records,
                                         void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "rollout_rs_row_stats: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31), "rollout_rs_row_stats: too many workgroups");
  VAMD_REQUIRE(old_log_prob && rollout_log_prob && mask && records, "rollout_rs_row_stats: null pointer");
  const int chunks = (int)chunks_of(length);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(batch * chunks)), block(kRcThreads);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    if (can_vectorize(length, {old_log_prob, rollout_log_prob}, mask, sizeof(M)))
      hipLaunchKernelGGL((rs_rows_kernel<true, M>), grid, block, 0, s, old_log_prob, rollout_log_prob, mk, batch,
                         length, chunks, records);
    else
      hipLaunchKernelGGL((rs_rows_kernel<false, M>), grid, block, 0, s, old_log_prob, rollout_log_prob, mk, batch,
                         length, chunks, records);
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_rollout_rs_apply(const float* old_log_prob, const float* rollout_log_prob, const void* mask,
                                     int mask_dtype, int64_t batch, int64_t length, const uint8_t* row_keep,
                                     int n_token_options, const int* estimators, const float* lower,
                                     const float* upper, void* new_mask, double* records, void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "rollout_rs_apply: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31), "rollout_rs_apply: too many workgroups");
  VAMD_REQUIRE(old_log_prob && rollout_log_prob && mask && row_keep && new_mask && records,
               "rollout_rs_apply: null pointer");
  VAMD_REQUIRE(n_token_options >= 0 && n_token_options <= kRsMaxTokenOptions,
               "rollout_rs_apply: at most %d token-level options", kRsMaxTokenOptions);
  VAMD_REQUIRE(n_token_options == 0 || (estimators && lower && upper), "rollout_rs_apply: null option tables");
  RsOptions opt;
  opt.n = n_token_options;
  for (int j = 0; j < kRsMaxTokenOptions; ++j) {
    const bool have = j < n_token_options;
    opt.estimator[j] = have ? estimators[j] : 0;
    VAMD_REQUIRE(opt.estimator[j] >= 0 && opt.estimator[j] <= 2, "rollout_rs_apply: invalid estimator %d",
                 opt.estimator[j]);
    opt.lower[j] = have ? lower[j] : 0.f;
    opt.upper[j] = have ? upper[j] : 0.f;
    opt.two_sided[j] = opt.estimator[j] == 0;
  }
  const int chunks = (int)chunks_of(length);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(batch * chunks)), block(kRcThreads);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    M* out = static_cast<M*>(new_mask);
    if (can_vectorize(length, {old_log_prob, rollout_log_prob}, mask, sizeof(M)) && aligned_to(new_mask, sizeof(M) * 4))
      hipLaunchKernelGGL((rs_apply_kernel<true, M>), grid, block, 0, s, old_log_prob, rollout_log_prob, mk, row_keep,
                         batch, length, chunks, opt, out, records);
    else
      hipLaunchKernelGGL((rs_apply_kernel<false, M>), grid, block, 0, s, old_log_prob, rollout_log_prob, mk, row_keep,
                         batch, length, chunks, opt, out, records);
  });
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
