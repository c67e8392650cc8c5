// Per-step batch statistics of the trainer in one pass over the [batch, length] tensors.
//
// compute_data_metrics (verl/trainer/ppo/metric_utils.py:81-225) derives about thirty scalars from
// six tensors with one masked_select / reduction / .item() each.  Here one launch reads every
// tensor once: each (row, 4096-column chunk) workgroup leaves a record of partial sums and
// extrema.  A second, single-workgroup launch folds the records into per-row quantities (sequence
// score and reward, prompt and response length) and then into the output vector, so the host
// reads the whole set with a single copy.  The fold is a launch of its own because its registers
// (a 17-slot record per row in flight, 32 running statistics) would otherwise be charged to every
// wavefront of the streaming kernel.
#include "rowchunk.h"

namespace vamd {

// record slots
enum {
  kDmScore = 0,   // sum of token_level_scores over the row chunk (unmasked, :105)
  kDmReward,      // sum of token_level_rewards (unmasked, :106)
  kDmRespLen,     // sum of attention_mask over the response columns (:69-70)
  kDmPromptLen,   // sum of attention_mask over the prompt columns (chunk 0 only)
  kDmValid,       // number of response_mask != 0 elements
  kDmAdv, kDmRet, kDmRet2, kDmVal, kDmDiff, kDmDiff2,  // sums over the valid elements
  kDmAdvMax, kDmAdvMinNeg, kDmRetMax, kDmRetMinNeg, kDmValMax, kDmValMinNeg,  // minima are stored negated
  kDmRec
};
constexpr int kDmSums = kDmAdvMax;  // slots [0, kDmSums) add, the rest are extrema

// Maximum of NV doubles per thread over the workgroup; result valid in thread 0.
template <int NV, int NT>
__device__ __forceinline__ void block_max(double (&v)[NV], double* smem /* NV * NT/64 doubles */) {
  block_reduce<NV, NT>(v, smem, MaxOp());
}

struct DmArgs {
  const float *scores, *rewards, *adv, *ret, *val;  // val may be null
  int64_t rows, cols, prompt;                       // attention_mask is [rows][prompt + cols]
  int chunks;       // records per row: spans of `span` 4096-column chunks
  int span;
  double* records;  // kDmRec slots per (row, span) workgroup, slot-major
  double* shares;   // per workgroup of the fold launch: its 16 sums and 16 maxima
  unsigned* fold_counter;  // arrivals of the fold launch's workgroups; the streaming pass clears it
  double* out;      // [VAMD_DM_COUNT]
};

// WIDE: the 17-value workgroup reduction through an LDS staging area (block_reduce_wide), which shortens the tail
// of a launch of one round of workgroups; its 23 KB per workgroup would cost a larger launch its occupancy.
template <bool VEC, class M, class A, bool WIDE>
__global__ __launch_bounds__(kRcThreads) void data_metrics_kernel(DmArgs a, const M* __restrict__ mask,
                                                                  const A* __restrict__ attention) {
  const int64_t row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  if (blockIdx.x == 0 && threadIdx.x == 0) a.fold_counter[0] = 0u;
  // A workgroup walks a.span consecutive 4096-column chunks of its row and leaves one record (a.chunks counts
  // those spans): the workgroup reduction of a record this wide costs more vector-ALU time than streaming one chunk.
  double acc[kDmSums];
#pragma unroll
  for (int i = 0; i < kDmSums; ++i) acc[i] = 0.0;
  float hi[3] = {-__builtin_inff(), -__builtin_inff(), -__builtin_inff()};  // adv, ret, val
  float lo[3] = {__builtin_inff(), __builtin_inff(), __builtin_inff()};
  const int64_t att_row = row * (a.prompt + a.cols) + a.prompt;
  const bool streaming = streams_past_caches(a.rows * a.cols);  // the grid counts spans of chunks, not chunks
  for (int u = 0; u < a.span; ++u) {
    const ChunkPos pos(row, chunk * a.span + u, a.cols);
    // per-thread partials over its 16 elements in fp32 (exact counts, 1e-7 relative on the sums), widened per chunk
    float s[kDmSums];
#pragma unroll
    for (int i = 0; i < kDmSums; ++i) s[i] = 0.f;
#pragma unroll 2
    for (int k = 0; k < kGroups; ++k) {
      if (pos.valid[k] <= 0) continue;
      float sc[4], rw[4], ad[4], rt[4], vl[4] = {0.f, 0.f, 0.f, 0.f}, m[4], at[4];
      ld4<VEC>(a.scores, pos.idx[k], pos.valid[k], sc, streaming);
      ld4<VEC>(a.rewards, pos.idx[k], pos.valid[k], rw, streaming);
      ld4<VEC>(a.adv, pos.idx[k], pos.valid[k], ad, streaming);
      ld4<VEC>(a.ret, pos.idx[k], pos.valid[k], rt, streaming);
      if (a.val) ld4<VEC>(a.val, pos.idx[k], pos.valid[k], vl, streaming);
      ldmask4<VEC>(mask, pos.idx[k], pos.valid[k], m, streaming);
      ldmask4<VEC>(attention, att_row + (pos.idx[k] - row * a.cols), pos.valid[k], at, streaming);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (e >= pos.valid[k]) continue;
        s[kDmScore] += sc[e];
        s[kDmReward] += rw[e];
        s[kDmRespLen] += at[e];
        if (m[e] != 0.f) {
          s[kDmValid] += 1.f;
          s[kDmAdv] += ad[e];
          s[kDmRet] += rt[e];
          s[kDmRet2] += rt[e] * rt[e];
          hi[0] = fmaxf(hi[0], ad[e]); lo[0] = fminf(lo[0], ad[e]);
          hi[1] = fmaxf(hi[1], rt[e]); lo[1] = fminf(lo[1], rt[e]);
          if (a.val) {
            const float d = rt[e] - vl[e];  // the fp32 difference the reference forms (:143)
            s[kDmVal] += vl[e];
            s[kDmDiff] += d;
            s[kDmDiff2] += d * d;
            hi[2] = fmaxf(hi[2], vl[e]); lo[2] = fminf(lo[2], vl[e]);
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kDmSums; ++i) acc[i] += (double)s[i];
  }
  if (chunk == 0) {
    const int64_t p0 = row * (a.prompt + a.cols);
    float prompt_len = 0.f;
    for (int64_t c = threadIdx.x; c < a.prompt; c += kRcThreads) prompt_len += (float)attention[p0 + c];
    acc[kDmPromptLen] += (double)prompt_len;
  }
  __shared__ double stage[WIDE ? 4 * kDmSums * kWidePitch : kDmSums * 4];
  double ext[6] = {hi[0], -(double)lo[0], hi[1], -(double)lo[1], hi[2], -(double)lo[2]};
  if constexpr (WIDE) {
    block_reduce_wide<kDmSums, kRcThreads>(acc, stage, SumOp());
    block_reduce_wide<6, kRcThreads>(ext, stage, MaxOp());
  } else {
    block_sum<kDmSums, kRcThreads>(acc, stage);
    block_max<6, kRcThreads>(ext, stage);
  }
  if (threadIdx.x == 0) {
    double rec[kDmRec];
#pragma unroll
    for (int i = 0; i < kDmSums; ++i) rec[i] = acc[i];
#pragma unroll
    for (int i = 0; i < 6; ++i) rec[kDmSums + i] = ext[i];  // maxima, and minima negated
    store_record<kDmRec>(a.records, row, chunk, a.rows, a.chunks, rec);  // read by the next launch
  }
}

constexpr int kFoldRows = 4;          // rows per thread and trip of the fold launch
constexpr int kDmFoldThreads = 128;   // a workgroup of the fold launch takes up to kFoldRows * kDmFoldThreads rows

// records -> per-row quantities -> the output vector: one row per thread, the workgroups' totals combined by the
// last of them to finish.
template <int NT>
__global__ __launch_bounds__(NT) void data_metrics_fold_kernel(DmArgs a) {
  const double inf = __longlong_as_double(0x7ff0000000000000ll);
  __shared__ double stage[(NT / 64) * 16 * kWidePitch];
  // ---- fold: thread-strided over rows -------------------------------------------------------------
  // sums: 0 n_non_aborted 1 score 2 reward 3 resp_len 4 resp_len==cols 5 resp_len (non-aborted)
  //       6 resp_len==cols (non-aborted) 7 prompt_len 8 prompt_len==prompt
  //       9.. the valid-element sums kDmValid .. kDmDiff2
  constexpr int kElem = kDmSums - kDmValid;  // 7
  double t[9 + kElem];
#pragma unroll
  for (int i = 0; i < 9 + kElem; ++i) t[i] = 0;
  // maxima (minima negated): 0/1 score, 2/3 reward, 4/5 resp_len, 6/7 resp_len non-aborted, 8/9 prompt_len,
  //                          10..15 adv, ret, val
  double x[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) x[i] = -inf;
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
    double rec[kFoldRows][kDmRec];
    fold_row_records<kDmRec, kDmSums, kFoldRows, false, 1>(a.records, rr, have, a.rows, a.chunks, rec);
#pragma unroll
    for (int k = 0; k < kFoldRows; ++k) {
      if (!have[k]) break;
      const double* row_s = rec[k];
#pragma unroll
      for (int i = 0; i < kElem; ++i) t[9 + i] += rec[k][kDmValid + i];
#pragma unroll
      for (int i = 0; i < 6; ++i) x[10 + i] = fmax(x[10 + i], rec[k][kDmSums + i]);
      const double score = (double)(float)row_s[kDmScore], reward = (double)(float)row_s[kDmReward];
      const double rl = row_s[kDmRespLen], pl = row_s[kDmPromptLen];
      t[3] += rl;
      t[4] += rl == (double)a.cols ? 1.0 : 0.0;
      x[4] = fmax(x[4], rl); x[5] = fmax(x[5], -rl);
      t[7] += pl;
      t[8] += pl == (double)a.prompt ? 1.0 : 0.0;
      x[8] = fmax(x[8], pl); x[9] = fmax(x[9], -pl);
      if (rl != 0.0) {  // not aborted (:119-120)
        t[0] += 1.0;
        t[1] += score;
        t[2] += reward;
        x[0] = fmax(x[0], score); x[1] = fmax(x[1], -score);
        x[2] = fmax(x[2], reward); x[3] = fmax(x[3], -reward);
        t[5] += rl;
        t[6] += rl == (double)a.cols ? 1.0 : 0.0;
        x[6] = fmax(x[6], rl); x[7] = fmax(x[7], -rl);
      }
    }
  }
  block_reduce_wide<9 + kElem, NT>(t, stage, SumOp());
  block_reduce_wide<16, NT>(x, stage, MaxOp());
  if (!fold_across_workgroups<9 + kElem, 16, NT>(t, x, a.shares, a.fold_counter, stage)) return;
  if (threadIdx.x == 0) {
    double* o = a.out;
    const double B = (double)a.rows, na = t[0];
    const double n = t[9 + 0], s_adv = t[9 + 1], s_ret = t[9 + 2], s_ret2 = t[9 + 3], s_val = t[9 + 4],
                 s_d = t[9 + 5], s_d2 = t[9 + 6];
    o[VAMD_DM_SCORE_MEAN] = t[1] / na;  o[VAMD_DM_SCORE_MAX] = x[0];  o[VAMD_DM_SCORE_MIN] = -x[1];
    o[VAMD_DM_REWARD_MEAN] = t[2] / na; o[VAMD_DM_REWARD_MAX] = x[2]; o[VAMD_DM_REWARD_MIN] = -x[3];
    o[VAMD_DM_ADV_MEAN] = s_adv / n;    o[VAMD_DM_ADV_MAX] = x[10];   o[VAMD_DM_ADV_MIN] = -x[11];
    o[VAMD_DM_RET_MEAN] = s_ret / n;    o[VAMD_DM_RET_MAX] = x[12];   o[VAMD_DM_RET_MIN] = -x[13];
    o[VAMD_DM_VAL_MEAN] = s_val / n;    o[VAMD_DM_VAL_MAX] = x[14];   o[VAMD_DM_VAL_MIN] = -x[15];
    // torch.var: unbiased, NaN for a single element
    const double var_d = (s_d2 - s_d * s_d / n) / (n - 1.0);
    const double var_r = (s_ret2 - s_ret * s_ret / n) / (n - 1.0);
    o[VAMD_DM_VF_EXPLAINED_VAR] = 1.0 - var_d / (var_r + 1e-5);
    o[VAMD_DM_RESP_LEN_MEAN] = t[3] / B; o[VAMD_DM_RESP_LEN_MAX] = x[4]; o[VAMD_DM_RESP_LEN_MIN] = -x[5];
    o[VAMD_DM_RESP_LEN_CLIP] = t[4] / B;
    o[VAMD_DM_RESP_LEN_NA_MEAN] = t[5] / na; o[VAMD_DM_RESP_LEN_NA_MAX] = x[6]; o[VAMD_DM_RESP_LEN_NA_MIN] = -x[7];
    o[VAMD_DM_RESP_LEN_NA_CLIP] = t[6] / na;
    o[VAMD_DM_ABORTED_RATIO] = (B - na) / B;
    o[VAMD_DM_PROMPT_LEN_MEAN] = t[7] / B; o[VAMD_DM_PROMPT_LEN_MAX] = x[8]; o[VAMD_DM_PROMPT_LEN_MIN] = -x[9];
    o[VAMD_DM_PROMPT_LEN_CLIP] = t[8] / B;
    o[VAMD_DM_VALID_TOKENS] = n;
    o[VAMD_DM_NON_ABORTED] = na;
  }
}

// Per-row sums behind compute_variance_proxy_metrics (verl/trainer/ppo/metric_utils.py:306-412):
// slot 0 number of valid tokens, 1 sum of advantages, 2 sum of w = 1 - 2 exp(old_log_prob) + sum_pi_squared
// (times is_weight^2 when importance weights are given), 3 sum of the importance weights,
// 4 sum of w / max(is_weight^2, 1e-10), each over the valid tokens.  The [batch]-sized rest is host arithmetic.
enum { kVpCount = 0, kVpAdv, kVpW, kVpIsw, kVpWOriginal, kVpSlots };

template <bool VEC, class M, bool ISW>
__global__ __launch_bounds__(kRcThreads) void variance_proxy_rows_kernel(const float* __restrict__ adv,
                                                                         const float* __restrict__ old_lp,
                                                                         const float* __restrict__ pi2,
                                                                         const float* __restrict__ isw,
                                                                         const M* __restrict__ mask, int64_t rows,
                                                                         int64_t cols, int chunks,
                                                                         double* __restrict__ records) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float a[kGroups][4], lp[kGroups][4], q[kGroups][4], iw[kGroups][4], m[kGroups][4];
  load_groups<VEC>(adv, pos, a);
  load_groups<VEC>(old_lp, pos, lp);
  load_groups<VEC>(pi2, pos, q);
  if (ISW) load_groups<VEC>(isw, pos, iw);
  load_mask_groups<VEC>(mask, pos, m);
  float s[kVpSlots] = {0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= pos.valid[g] || m[g][e] == 0.f) continue;
      float w = 1.f - 2.f * expf(lp[g][e]) + q[g][e];
      s[kVpCount] += 1.f;
      s[kVpAdv] += a[g][e];
      if (ISW) {
        const float r2 = iw[g][e] * iw[g][e];
        w = w * r2;
        s[kVpIsw] += iw[g][e];
        s[kVpWOriginal] += w / fmaxf(r2, 1e-10f);
      }
      s[kVpW] += w;
    }
  __shared__ double smem[kVpSlots * 4];
  double acc[kVpSlots];
#pragma unroll
  for (int i = 0; i < kVpSlots; ++i) acc[i] = s[i];
  block_sum<kVpSlots, kRcThreads>(acc, smem);
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < kVpSlots; ++i) records[record_at(i, row, chunk, rows, chunks)] = acc[i];
}

}  // namespace vamd

using namespace vamd;

// workgroups of the fold launch (at most 256)
static unsigned dm_fold_workgroups(int64_t batch) {
  const int64_t per = (int64_t)kFoldRows * kDmFoldThreads;
  const int64_t n = (batch + per - 1) / per;
  return (unsigned)(n < 1 ? 1 : (n > 256 ? 256 : n));
}

extern "C" int vamd_variance_proxy_rows(const float* advantages, const float* old_log_probs,
                                        const float* sum_pi_squared, const float* is_weights, const void* mask,
                                        int mask_dtype, int64_t batch, int64_t length, double* records,
                                        void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "variance_proxy_rows: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31), "variance_proxy_rows: too many workgroups");
  VAMD_REQUIRE(advantages && old_log_probs && sum_pi_squared && mask && records, "variance_proxy_rows: null pointer");
  const int chunks = (int)chunks_of(length);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(batch * chunks)), block(kRcThreads);
#define VAMD_VP(V, W)                                                                                            \
  hipLaunchKernelGGL((variance_proxy_rows_kernel<V, M, W>), grid, block, 0, s, advantages, old_log_probs,        \
                     sum_pi_squared, is_weights, mk, batch, length, chunks, records)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    const bool vec = can_vectorize(length, {advantages, old_log_probs, sum_pi_squared, is_weights}, mask, sizeof(M));
    if (vec) { if (is_weights) VAMD_VP(true, true); else VAMD_VP(true, false); }
    else { if (is_weights) VAMD_VP(false, true); else VAMD_VP(false, false); }
  });
#undef VAMD_VP
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}


extern "C" size_t vamd_data_metrics_workspace_bytes(int64_t batch, int64_t response_length) {
  if (batch <= 0 || response_length <= 0) return 0;
  return align_up((size_t)batch * chunks_of(response_length) * kDmRec * sizeof(double), 256) +
         align_up((size_t)dm_fold_workgroups(batch) * 32 * sizeof(double), 256) + 256;
}

extern "C" int vamd_data_metrics(const float* token_level_scores, const float* token_level_rewards,
                                 const float* advantages, const float* returns, const float* values,
                                 const void* response_mask, int mask_dtype, const void* attention_mask,
                                 int attention_dtype, int64_t batch, int64_t prompt_length, int64_t response_length,
                                 double* out, void* workspace, size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(batch > 0 && response_length > 0 && prompt_length >= 0, "data_metrics: empty input");
  VAMD_REQUIRE(batch * chunks_of(response_length) < (1ll << 31), "data_metrics: too many workgroups");
  VAMD_REQUIRE(token_level_scores && token_level_rewards && advantages && returns && response_mask &&
                   attention_mask && out,
               "data_metrics: null pointer");
  if (!workspace || workspace_bytes < vamd_data_metrics_workspace_bytes(batch, response_length)) {
    set_error("data_metrics: workspace too small");
    return VAMD_EWORKSPACE;
  }
  DmArgs a;
  a.scores = token_level_scores; a.rewards = token_level_rewards; a.adv = advantages; a.ret = returns; a.val = values;
  a.rows = batch; a.cols = response_length; a.prompt = prompt_length;
  a.span = record_span(batch, (int)chunks_of(response_length));
  a.chunks = ((int)chunks_of(response_length) + a.span - 1) / a.span;
  Carver carve(workspace);
  a.records = carve.take<double>((size_t)batch * a.chunks * kDmRec);
  a.shares = carve.take<double>((size_t)dm_fold_workgroups(batch) * 32);
  a.fold_counter = carve.take<unsigned>(1);
  a.out = out;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(batch * a.chunks)), block(kRcThreads);
  const bool wide = batch * a.chunks <= 1024;  // one round of workgroups at six per CU
#define VAMD_DM(A)                                                                                            \
  VAMD_MASK_DISPATCH(mask_dtype, M, {                                                                          \
    const bool vec = can_vectorize(response_length, {token_level_scores, token_level_rewards, advantages,      \
                                                     returns, values}, response_mask, sizeof(M)) &&            \
                     prompt_length % 4 == 0 && aligned_to(attention_mask, 4 * sizeof(A));                      \
    if (vec && wide)                                                                                           \
      hipLaunchKernelGGL((data_metrics_kernel<true, M, A, true>), grid, block, 0, s, a,                        \
                         static_cast<const M*>(response_mask), static_cast<const A*>(attention_mask));         \
    else if (vec)                                                                                              \
      hipLaunchKernelGGL((data_metrics_kernel<true, M, A, false>), grid, block, 0, s, a,                       \
                         static_cast<const M*>(response_mask), static_cast<const A*>(attention_mask));         \
    else                                                                                                       \
      hipLaunchKernelGGL((data_metrics_kernel<false, M, A, false>), grid, block, 0, s, a,                      \
                         static_cast<const M*>(response_mask), static_cast<const A*>(attention_mask));         \
  })
  switch (attention_dtype) {
    case VAMD_MASK_F32: VAMD_DM(float); break;
    case VAMD_MASK_I64: VAMD_DM(int64_t); break;
    case VAMD_MASK_U8: VAMD_DM(uint8_t); break;
    case VAMD_MASK_I32: VAMD_DM(int32_t); break;
    default: set_error("unknown mask dtype code %d", attention_dtype); return VAMD_EINVAL;
  }
#undef VAMD_DM
  hipLaunchKernelGGL(data_metrics_fold_kernel<kDmFoldThreads>, dim3(dm_fold_workgroups(batch)), dim3(kDmFoldThreads),
                     0, s, a);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
