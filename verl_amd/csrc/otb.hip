// Optimal-token-baseline advantages (compute_optimal_token_baseline_advantage,
// verl/trainer/ppo/core_algos.py:756-875):
//
//   returns_t = sum_{s >= t} r_s m_s                                   (reward to go)
//   w_t       = 1 - 2 exp(old_log_prob_t) + sum_pi_squared_t  [* is_weight_t^2]
//   W_t       = sum_{s <= t} w_s m_s                                   (cumulative path-variance proxy)
//   B_t(g)    = sum_{i in g} returns W m / (sum_{i in g} W m + eps)    per prompt group and column,
//               0 for a group of one
//   adv       = (returns - B) m
//
// Two launches.  The first walks every row twice inside one workgroup -- right to left for the
// returns, left to right for W -- as plain prefix sums carried in double (1024-column segments,
// 4 columns per thread, wavefront scan by lane exchanges plus the four wavefront totals through LDS).  The
// second gives each (group, 1024-column segment) to one workgroup, which adds up the group's rows
// column by column in index order, forms the baseline and writes the advantages of those rows.
// Nothing is reduced across workgroups, so neither launch needs arrival counters.
//
// The multi-turn variant (compute_multi_turn_optimal_token_baseline_advantage, :876-1004) packs each
// row's valid tokens to the left before the group reduction, so that the k-th valid token of every
// trajectory shares baseline column k.  Here the first launch also counts the valid tokens in front
// of each column (a third running sum), writes returns and W of the valid tokens at that rank into
// packed copies of the rows, and a third launch gathers the packed advantages back by rank.
#include "rowchunk.h"

namespace vamd {

constexpr int kOtbSeg = 1024;

// Running sum along one row in walk order (REVERSE: last column first).  load(col0, valid, v[4])
// fills the 4 values at col0 .. col0 + 3 (0 beyond `valid`); store(col0, valid, out[4]) receives
// the inclusive sums at those columns.
template <bool REVERSE, class Load, class Store>
__device__ __forceinline__ double row_running_sum(int64_t cols, double (*wave_tot)[4], Load load, Store store) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = REVERSE ? kRcThreads - 1 - tid : tid;  // thread order = walk order
  const int nseg = (int)((cols + kOtbSeg - 1) / kOtbSeg);
  double carry = 0.0;
  int par = 0;
  for (int k = 0; k < nseg; ++k) {
    const int seg = REVERSE ? nseg - 1 - k : k;
    const int64_t col0 = (int64_t)seg * kOtbSeg + slot * 4;
    const int64_t left = cols - col0;
    const int valid = left >= 4 ? 4 : (left > 0 ? (int)left : 0);
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (valid > 0) load(col0, valid, v);
    double inc[4];
    double run = 0.0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = REVERSE ? 3 - j : j;
      run += (double)v[e];
      inc[e] = run;
    }
    const double scan = wave_running_sum(run);  // inclusive scan of the thread totals over the wavefront
    if (lane == 63) wave_tot[par][wave] = scan;
    __syncthreads();
    double before = carry + (scan - run);
    double all = 0.0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const double t = wave_tot[par][w];
      if (w < wave) before += t;
      all += t;
    }
    carry += all;
    if (valid > 0) {
      float out[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] = (float)(before + inc[e]);
      store(col0, valid, out);
    }
    par ^= 1;
  }
  return carry;
}

struct OtbPacked {  // multi-turn variant only
  int* rank;          // [rows][cols] valid tokens in front of a column
  int64_t* row_len;   // [rows] valid tokens of the row
  float* g;           // [rows][cols] returns of the valid tokens, packed to the left
  float* w;           // [rows][cols] W of the valid tokens, packed to the left
};

template <bool VEC, class M, bool ISW, bool PACK>
__global__ __launch_bounds__(kRcThreads) void otb_scan_kernel(const float* __restrict__ rewards,
                                                              const M* __restrict__ mask,
                                                              const float* __restrict__ old_lp,
                                                              const float* __restrict__ pi2,
                                                              const float* __restrict__ isw, int64_t cols,
                                                              float* returns, float* __restrict__ w_cum,
                                                              OtbPacked pk) {
  const int64_t base = (int64_t)blockIdx.x * cols;
  // one workgroup per row: the launch is past the caches when rows x cols is (the inputs are read once; returns and
  // W are read again by the baseline launch, but two tensors of that size do not survive in the caches either)
  const bool streaming = streams_past_caches((int64_t)gridDim.x * cols);
  __shared__ double wave_tot[2][4];
  row_running_sum<true>(
      cols, wave_tot,
      [&](int64_t c, int valid, float (&v)[4]) {
        float m[4];
        ld4<VEC>(rewards, base + c, valid, v, streaming);
        ldmask4<VEC>(mask, base + c, valid, m, false);  // read again by the forward walk
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = e < valid ? v[e] * m[e] : 0.f;
      },
      [&](int64_t c, int valid, const float (&o)[4]) { st4<VEC>(returns, base + c, valid, o, streaming && !PACK); });
  __syncthreads();  // the forward walks below own other columns than the walk above did
  if constexpr (PACK) {
    const double n = row_running_sum<false>(
        cols, wave_tot,
        [&](int64_t c, int valid, float (&v)[4]) {
          float m[4];
          ldmask4<VEC>(mask, base + c, valid, m, false);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = (e < valid && m[e] != 0.f) ? 1.f : 0.f;
        },
        [&](int64_t c, int valid, const float (&o)[4]) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (e < valid) pk.rank[base + c + e] = (int)o[e] - 1;  // exact: counts stay below 2^24
        });
    if (threadIdx.x == 0) pk.row_len[blockIdx.x] = (int64_t)n;
    __syncthreads();
  }
  float keep_m[4], keep_g[4];
  int keep_rank[4];
  row_running_sum<false>(
      cols, wave_tot,
      [&](int64_t c, int valid, float (&v)[4]) {
        float lp[4], q[4], iw[4];
        ld4<VEC>(old_lp, base + c, valid, lp, streaming);
        ld4<VEC>(pi2, base + c, valid, q, streaming);
        ldmask4<VEC>(mask, base + c, valid, keep_m, false);
        if (ISW) ld4<VEC>(isw, base + c, valid, iw, streaming);
        if constexpr (PACK) {
          ld4<VEC>(returns, base + c, valid, keep_g, false);
#pragma unroll
          for (int e = 0; e < 4; ++e) keep_rank[e] = e < valid ? pk.rank[base + c + e] : 0;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float w = 1.f - 2.f * expf(lp[e]) + q[e];
          if (ISW) w = w * (iw[e] * iw[e]);
          v[e] = e < valid ? w * keep_m[e] : 0.f;
        }
      },
      [&](int64_t c, int valid, const float (&o)[4]) {
        if constexpr (PACK) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (e < valid && keep_m[e] != 0.f) {
              pk.w[base + keep_rank[e]] = o[e];
              pk.g[base + keep_rank[e]] = keep_g[e];
            }
        } else {
          st4<VEC>(w_cum, base + c, valid, o, streaming);
        }
      });
}

struct OtbGroups {
  const int64_t* rows_by_group;  // row indices, the rows of group 0 first, each group in index order
  const int64_t* group_offsets;  // [n_groups + 1]
  const int64_t* tail_start;     // optional [batch]: the baseline of a row is 0 from this column on
  const int64_t* row_len;        // packed rows: columns below row_len[row] are valid and the mask is not read
};

// Mask of the 4 columns at `col` of `row`: read, or implied by the row's packed length.
template <bool VEC, class M>
__device__ __forceinline__ void otb_mask4(const M* __restrict__ mask, const OtbGroups& gr, int64_t row, int64_t cols,
                                          int64_t col, int valid, float (&m)[4]) {
  if (gr.row_len) {
    const int64_t n = gr.row_len[row];
#pragma unroll
    for (int e = 0; e < 4; ++e) m[e] = (e < valid && col + e < n) ? 1.f : 0.f;
  } else {
    ldmask4<VEC>(mask, row * cols + col, valid, m, false);
  }
}

constexpr int kOtbRows = 4;  // rows of a larger group whose loads are in flight together
constexpr int kOtbHeld = 8;  // a group of up to this many rows is held in registers between its loads and its stores

// One workgroup per (group, 1024-column segment), a thread per 4 columns: the group's rows are added up in index
// order, kOtbRows of them in flight at a time (a group is a handful of rows, so the launch needs narrow segments to
// fill the device, and a thread walking the rows one load at a time would wait out every trip to memory).
// `adv` may be `returns` itself (each thread overwrites only what it has just read).
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void otb_baseline_kernel(const float* returns,
                                                                  const float* __restrict__ w_cum,
                                                                  const M* __restrict__ mask, OtbGroups gr,
                                                                  int64_t cols, int segs, float eps, float* adv,
                                                                  int streaming_launch) {
  const bool streaming = streaming_launch != 0;
  const int64_t g = blockIdx.x / segs;
  const int64_t col = (int64_t)(blockIdx.x % segs) * kOtbSeg + threadIdx.x * 4;
  const int64_t left = cols - col;
  const int valid = left >= 4 ? 4 : (left > 0 ? (int)left : 0);
  if (valid == 0) return;
  const int64_t first = gr.group_offsets[g], last = gr.group_offsets[g + 1];
  float num[4] = {0.f, 0.f, 0.f, 0.f}, den[4] = {0.f, 0.f, 0.f, 0.f};
  if (last - first > 1 && last - first <= kOtbHeld) {
    // A group of up to kOtbHeld rows stays in registers from its one round of loads to its stores: nothing is read a
    // second time and the workgroup makes one trip to memory instead of four.  Same additions in the same order as
    // the general path below.
    float R[kOtbHeld][4], W[kOtbHeld][4], m[kOtbHeld][4];
    int64_t row[kOtbHeld];
#pragma unroll
    for (int k = 0; k < kOtbHeld; ++k) {
#pragma unroll
      for (int e = 0; e < 4; ++e) R[k][e] = W[k][e] = m[k][e] = 0.f;
      row[k] = first + k < last ? gr.rows_by_group[first + k] : -1;
      if (row[k] >= 0) {
        ld4<VEC>(returns, row[k] * cols + col, valid, R[k], streaming);
        ld4<VEC>(w_cum, row[k] * cols + col, valid, W[k], streaming);
        otb_mask4<VEC>(mask, gr, row[k], cols, col, valid, m[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < kOtbHeld; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (m[k][e] != 0.f) {
          num[e] += R[k][e] * W[k][e] * m[k][e];
          den[e] += W[k][e] * m[k][e];
        }
#pragma unroll
    for (int e = 0; e < 4; ++e) num[e] = num[e] / (den[e] + eps);
#pragma unroll
    for (int k = 0; k < kOtbHeld; ++k) {
      if (row[k] < 0) continue;
      const int64_t cut = gr.tail_start ? gr.tail_start[row[k]] : cols;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float b = col + e < cut ? num[e] : 0.f;
        R[k][e] = m[k][e] != 0.f ? (R[k][e] - b) * m[k][e] : 0.f;
      }
      st4<VEC>(adv, row[k] * cols + col, valid, R[k], streaming);
    }
    return;
  }
  if (last - first > 1) {
    for (int64_t i0 = first; i0 < last; i0 += kOtbRows) {
      float R[kOtbRows][4], W[kOtbRows][4], m[kOtbRows][4];
#pragma unroll
      for (int k = 0; k < kOtbRows; ++k) {
#pragma unroll
        for (int e = 0; e < 4; ++e) R[k][e] = W[k][e] = m[k][e] = 0.f;
        if (i0 + k < last) {
          const int64_t row = gr.rows_by_group[i0 + k];
          ld4<VEC>(returns, row * cols + col, valid, R[k], false);  // read again below
          ld4<VEC>(w_cum, row * cols + col, valid, W[k], streaming);
          otb_mask4<VEC>(mask, gr, row, cols, col, valid, m[k]);
        }
      }
#pragma unroll
      for (int k = 0; k < kOtbRows; ++k)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (m[k][e] != 0.f) {  // packed rows hold no defined value beyond their length
            num[e] += R[k][e] * W[k][e] * m[k][e];
            den[e] += W[k][e] * m[k][e];
          }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) num[e] = num[e] / (den[e] + eps);  // the baseline
  }
  for (int64_t i0 = first; i0 < last; i0 += kOtbRows) {
    float R[kOtbRows][4], m[kOtbRows][4];
    int64_t row[kOtbRows], cut[kOtbRows];
#pragma unroll
    for (int k = 0; k < kOtbRows; ++k) {
#pragma unroll
      for (int e = 0; e < 4; ++e) R[k][e] = m[k][e] = 0.f;
      row[k] = -1;
      cut[k] = 0;
      if (i0 + k < last) {
        row[k] = gr.rows_by_group[i0 + k];
        cut[k] = gr.tail_start ? gr.tail_start[row[k]] : cols;
        ld4<VEC>(returns, row[k] * cols + col, valid, R[k], false);
        otb_mask4<VEC>(mask, gr, row[k], cols, col, valid, m[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < kOtbRows; ++k) {
      if (row[k] < 0) break;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float b = col + e < cut[k] ? num[e] : 0.f;
        R[k][e] = m[k][e] != 0.f ? (R[k][e] - b) * m[k][e] : 0.f;
      }
      st4<VEC>(adv, row[k] * cols + col, valid, R[k], streaming);
    }
  }
}

// advantages[i][t] = packed[i][rank[i][t]] * mask[i][t]
template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void otb_unpack_kernel(const float* __restrict__ packed,
                                                                const int* __restrict__ rank,
                                                                const M* __restrict__ mask, int64_t cols, int chunks,
                                                                float* __restrict__ adv) {
  const int64_t row = blockIdx.x / chunks;
  const ChunkPos pos(row, blockIdx.x % chunks, cols);
  float m[kGroups][4], out[kGroups][4];
  load_mask_groups<VEC>(mask, pos, m);
#pragma unroll
  for (int k = 0; k < kGroups; ++k)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[k][e] = 0.f;
      if (e < pos.valid[k] && m[k][e] != 0.f) out[k][e] = packed[row * cols + rank[pos.idx[k] + e]] * m[k][e];
    }
  store_groups<VEC>(adv, pos, out);
}

}  // namespace vamd

using namespace vamd;

extern "C" size_t vamd_otb_advantage_workspace_bytes(int64_t batch, int64_t length, int packed) {
  if (batch <= 0 || length <= 0) return 0;
  const size_t plane = align_up((size_t)batch * length * 4, 256);
  if (!packed) return plane;                                                  // W
  return 3 * plane + align_up((size_t)batch * sizeof(int64_t), 256);          // packed W, packed returns, rank, lengths
}

extern "C" int vamd_otb_advantage(const float* rewards, const void* mask, int mask_dtype, const float* old_log_probs,
                                  const float* sum_pi_squared, const float* is_weights, const int64_t* rows_by_group,
                                  const int64_t* group_offsets, const int64_t* tail_start, int64_t batch,
                                  int64_t length, int64_t n_groups, int packed, float epsilon, float* advantages,
                                  float* returns, void* workspace, size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0 && n_groups >= 0, "otb_advantage: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31) && n_groups * ((length + kOtbSeg - 1) / kOtbSeg) < (1ll << 31),
               "otb_advantage: too many workgroups");
  VAMD_REQUIRE(length < (1ll << 24), "otb_advantage: rows longer than 2^24 - 1 columns are not supported");
  VAMD_REQUIRE(rewards && mask && old_log_probs && sum_pi_squared && advantages && returns,
               "otb_advantage: null pointer");
  VAMD_REQUIRE(n_groups == 0 || (rows_by_group && group_offsets), "otb_advantage: null group tables");
  VAMD_REQUIRE(n_groups > 0 || packed, "otb_advantage: no groups");
  if (!workspace || workspace_bytes < vamd_otb_advantage_workspace_bytes(batch, length, packed)) {
    set_error("otb_advantage: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  Carver carve(workspace);
  const size_t plane = (size_t)batch * length;
  float* w_cum = carve.take<float>(plane);
  OtbPacked pk{nullptr, nullptr, nullptr, nullptr};
  if (packed) {
    pk.w = w_cum;
    pk.g = carve.take<float>(plane);
    pk.rank = carve.take<int>(plane);
    pk.row_len = carve.take<int64_t>((size_t)batch);
  }
  const int chunks = (int)chunks_of(length);
  const OtbGroups gr{rows_by_group, group_offsets, tail_start, pk.row_len};
  const int segs = (int)((length + kOtbSeg - 1) / kOtbSeg);  // 1024-column segments of the baseline pass
  const dim3 threads(kRcThreads), per_row((unsigned)batch), per_group((unsigned)(n_groups * segs)),
      per_chunk((unsigned)(batch * chunks));
  const int past_caches = batch * length >= (int64_t)kStreamingGrid * 4096 ? 1 : 0;
#define VAMD_OTB(V, W)                                                                                              \
  do {                                                                                                              \
    if (packed) {                                                                                                   \
      hipLaunchKernelGGL((otb_scan_kernel<V, M, W, true>), per_row, threads, 0, s, rewards, mk, old_log_probs,       \
                         sum_pi_squared, is_weights, length, returns, w_cum, pk);                                   \
      if (n_groups > 0)                                                                                             \
        hipLaunchKernelGGL((otb_baseline_kernel<V, M>), per_group, threads, 0, s, pk.g, pk.w, mk, gr, length,        \
                           segs, epsilon, pk.g, 0);                                                                 \
      hipLaunchKernelGGL((otb_unpack_kernel<V, M>), per_chunk, threads, 0, s, pk.g, pk.rank, mk, length, chunks,     \
                         advantages);                                                                               \
    } else {                                                                                                        \
      hipLaunchKernelGGL((otb_scan_kernel<V, M, W, false>), per_row, threads, 0, s, rewards, mk, old_log_probs,      \
                         sum_pi_squared, is_weights, length, returns, w_cum, pk);                                   \
      hipLaunchKernelGGL((otb_baseline_kernel<V, M>), per_group, threads, 0, s, returns, w_cum, mk, gr, length,      \
                         segs, epsilon, advantages, past_caches);                                                   \
    }                                                                                                               \
  } while (0)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    const bool vec = can_vectorize(length, {rewards, old_log_probs, sum_pi_squared, is_weights, advantages, returns},
                                   mask, sizeof(M));
    if (vec) {
      if (is_weights) VAMD_OTB(true, true); else VAMD_OTB(true, false);
    } else {
      if (is_weights) VAMD_OTB(false, true); else VAMD_OTB(false, false);
    }
  });
#undef VAMD_OTB
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
