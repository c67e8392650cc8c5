// The two covariance-based policy losses: KL-Cov and Clip-Cov
// (verl/trainer/ppo/core_algos.py:1555-1632 and :1450-1552).
//
// Both treat a small set of tokens differently from the rest and choose that set by a global rule over the
// valid tokens of the batch: KL-Cov takes the k tokens with the largest covariance
// (A - mean A)(log_prob - mean log_prob), Clip-Cov draws clip_num tokens uniformly at random from those whose
// covariance lies in a band.  The reference does the first with a CPU top-k and the second with randperm.
// Here both are "the k largest of a 32-bit key": the key is the covariance mapped to an order-preserving
// unsigned integer (KL-Cov) or a hash of (seed, token index) (Clip-Cov: the k largest hashes of the candidates
// are a uniform draw without replacement), 0 marks a token that is not a candidate, and the k-th largest key
// is found by a radix select, 8 bits per pass over the keys, without leaving the device.  Tokens whose key
// equals the threshold share the remaining places first come, first served (exact ties only).
//
// Launch sequence: per-(row, chunk) sums -> means, k and the select state (1 workgroup) -> keys + histogram of the
// top byte -> [pick a bin (1 workgroup) -> histogram of the next byte] x 3 -> pick -> loss pass -> record fold.
#include "rowchunk.h"

namespace vamd {

enum { kCovKl = 0, kCovClip = 1 };

struct CovState {
  float mean_a, mean_lp;
  unsigned k;            // tokens to select
  unsigned n_cand;       // candidates (key != 0): the total of the first histogram
  unsigned prefix;       // the digits of the threshold key found so far
  unsigned k_rem;        // places left for keys equal to the prefix
  unsigned take_all;     // every candidate is selected
  unsigned tie_counter;  // tickets for keys equal to the threshold
  // kHistCopies copies of the 256-bin histogram, workgroup b adding to copy b % kHistCopies: the keys of a
  // launch fall into a handful of bins, and adds to one address are served one after the other
  unsigned hist[64][256];
};
constexpr int kHistCopies = 64;

struct CovArgs {
  const float *old_lp, *lp, *adv, *isw;
  int64_t rows, cols;
  int chunks;
  int kind;
  float ratio_lo, ratio_hi;  // Clip-Cov: 1 - clip_low, 1 + clip_high
  float cov_lb, cov_ub;      // Clip-Cov: the covariance band
  double select_ratio;       // kl_cov_ratio / clip_cov_ratio
  float kl_coef;             // KL-Cov: ppo_kl_coef
  unsigned long long seed;
  CovState* state;
  double* stats;    // 4 slots per (row, chunk): sum of the mask, valid tokens, sum A, sum log_prob over the valid tokens
  unsigned* keys;   // [rows * cols]
  double* records;  // 5 slots per (row, chunk) for the loss fold
};

// Order-preserving map from float to unsigned; never 0 for a finite value or an infinity.
__device__ __forceinline__ unsigned sortable_key(float x) {
  const unsigned u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ unsigned random_key(unsigned long long seed, unsigned long long index) {
  unsigned long long z = seed + 0x9E3779B97F4A7C15ull * (index + 1);  // splitmix64
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (unsigned)(z >> 32) | 1u;
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void cov_stats_kernel(CovArgs a, const M* __restrict__ mask) {
  const int64_t row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  const ChunkPos pos(row, chunk, a.cols);
  float A[kGroups][4], lp[kGroups][4], m[kGroups][4];
  load_groups<VEC>(a.adv, pos, A);
  load_groups<VEC>(a.lp, pos, lp);
  load_mask_groups<VEC>(mask, pos, m);
  float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= pos.valid[g]) continue;
      s[0] += m[g][e];
      if (m[g][e] > 0.f) {
        s[1] += 1.f;
        s[2] += A[g][e];
        s[3] += lp[g][e];
      }
    }
  __shared__ double smem[4 * 4];
  double acc[4] = {s[0], s[1], s[2], s[3]};
  block_sum<4, kRcThreads>(acc, smem);
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) a.stats[record_at(i, row, chunk, a.rows, a.chunks)] = acc[i];
}

// One workgroup: totals -> means and k; the select state starts empty.
__global__ __launch_bounds__(256) void cov_prepare_kernel(CovArgs a) {
  __shared__ double smem[4 * 4];
  double t[4] = {0, 0, 0, 0};
  const int64_t n = a.rows * a.chunks;
  for (int64_t k = threadIdx.x; k < n; k += 256)
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] += a.stats[(int64_t)i * n + k];
  block_sum<4, 256>(t, smem);
  CovState* st = a.state;
  for (int c = 0; c < kHistCopies; ++c) st->hist[c][threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    const double msum = t[0], count = t[1];
    if (a.kind == kCovKl) {  // plain means over the valid tokens (:1604); k = max(1, int(n ratio)) (:1605)
      st->mean_a = (float)t[2] / (float)count;
      st->mean_lp = (float)t[3] / (float)count;
      const double k = floor(count * a.select_ratio);
      st->k = count > 0 ? (unsigned)(k < 1.0 ? 1.0 : k) : 0u;
    } else {  // masked_mean (:1507-1509); clip_num = max(int(ratio M), 1) (:1513)
      st->mean_a = (float)t[2] / ((float)msum + 1e-8f);
      st->mean_lp = (float)t[3] / ((float)msum + 1e-8f);
      const double k = floor(a.select_ratio * msum);
      st->k = (unsigned)(k < 1.0 ? 1.0 : k);
    }
    st->n_cand = 0;
    st->prefix = 0;
    st->k_rem = 0;
    st->take_all = 0;
    st->tie_counter = 0;
  }
}

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void cov_keys_kernel(CovArgs a, const M* __restrict__ mask) {
  const int64_t row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  const ChunkPos pos(row, chunk, a.cols);
  __shared__ unsigned hist[256];
  hist[threadIdx.x] = 0;
  __syncthreads();
  float o[kGroups][4], lp[kGroups][4], A[kGroups][4], m[kGroups][4];
  load_groups<VEC>(a.lp, pos, lp);
  load_groups<VEC>(a.adv, pos, A);
  load_mask_groups<VEC>(mask, pos, m);
  if (a.kind == kCovClip) load_groups<VEC>(a.old_lp, pos, o);
  const float mean_a = a.state->mean_a, mean_lp = a.state->mean_lp;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (e >= pos.valid[g]) continue;
      unsigned key = 0;
      if (m[g][e] > 0.f) {
        const float cov = (A[g][e] - mean_a) * (lp[g][e] - mean_lp);
        if (a.kind == kCovKl) {
          key = sortable_key(cov);
        } else {
          const float r = expf(lp[g][e] - o[g][e]);
          const float l1 = -A[g][e] * r;
          const float l2 = -A[g][e] * fminf(fmaxf(r, a.ratio_lo), a.ratio_hi);
          if (!(l2 > l1) && cov < a.cov_ub && cov > a.cov_lb) key = random_key(a.seed, (unsigned long long)(pos.idx[g] + e));
        }
      }
      a.keys[pos.idx[g] + e] = key;
      if (key != 0) atomicAdd(&hist[key >> 24], 1u);
    }
  __syncthreads();
  if (hist[threadIdx.x]) atomicAdd(&a.state->hist[blockIdx.x % kHistCopies][threadIdx.x], hist[threadIdx.x]);
}

// Histogram of the byte at `shift` over the keys whose higher bytes equal the prefix.
__global__ __launch_bounds__(256) void cov_hist_kernel(const unsigned* __restrict__ keys, int64_t n, int shift,
                                                       CovState* __restrict__ st) {
  __shared__ unsigned hist[256];
  hist[threadIdx.x] = 0;
  __syncthreads();
  if (st->take_all || st->k == 0) return;
  const unsigned prefix = st->prefix >> (shift + 8);
  auto count = [&](unsigned key) {
    if (key != 0 && (key >> (shift + 8)) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
  };
  // eight 16-byte loads per thread, all issued before the first key is looked at (the key plane is 256-byte aligned)
  const uint4* __restrict__ keys4 = reinterpret_cast<const uint4*>(keys);
  const int64_t n4 = n / 4;
  const int64_t first = (int64_t)blockIdx.x * 256 * 8 + threadIdx.x;
  uint4 v[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int64_t i = first + (int64_t)u * 256;
    v[u] = i < n4 ? keys4[i] : make_uint4(0u, 0u, 0u, 0u);
  }
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    count(v[u].x);
    count(v[u].y);
    count(v[u].z);
    count(v[u].w);
  }
  if (blockIdx.x == 0 && n4 * 4 + threadIdx.x < n) count(keys[n4 * 4 + threadIdx.x]);  // the last n % 4 keys
  __syncthreads();
  if (hist[threadIdx.x]) atomicAdd(&st->hist[blockIdx.x % kHistCopies][threadIdx.x], hist[threadIdx.x]);
}

// One workgroup: the bin that holds the k_rem-th largest key of this pass becomes the next digit of the threshold,
// i.e. the largest bin b >= 1 with at least k_rem keys in bins b .. 255 (bin 0 when there is none).  The counts
// from each bin upwards come from a 256-wide suffix scan in LDS rather than one thread walking the bins.
__global__ __launch_bounds__(256) void cov_pick_kernel(CovState* __restrict__ st, int shift) {
  __shared__ unsigned S[2][256];
  __shared__ unsigned bin;
  const unsigned t = threadIdx.x;
  unsigned sum = 0;
  for (int c = 0; c < kHistCopies; ++c) {
    sum += st->hist[c][t];
    st->hist[c][t] = 0;
  }
  S[0][t] = sum;
  if (t == 0) bin = 0;
  __syncthreads();
  int p = 0;
  for (unsigned d = 1; d < 256; d <<= 1, p ^= 1) {
    S[p ^ 1][t] = S[p][t] + (t + d < 256 ? S[p][t + d] : 0u);
    __syncthreads();
  }
  const unsigned* from = S[p];  // from[b]: keys in bins b .. 255
  unsigned k_rem = st->k_rem;
  if (shift == 24) {  // first pass: fix how many there are to take
    if (st->k >= from[0]) {
      if (t == 0) {
        st->n_cand = from[0];
        st->take_all = 1;  // fewer candidates than places (none selected when there are no candidates)
      }
      return;
    }
    k_rem = st->k;
  }
  if (st->take_all || st->k == 0) return;
  if (t >= 1 && from[t] >= k_rem && (t == 255 || from[t + 1] < k_rem)) bin = t;
  __syncthreads();
  if (t == 0) {
    const unsigned b = bin;
    if (shift == 24) st->n_cand = from[0];
    st->prefix |= b << shift;
    st->k_rem = k_rem - (b == 255 ? 0u : from[b + 1]);
  }
}

template <bool VEC, class M, bool GRAD, bool ISW>
__global__ __launch_bounds__(kRcThreads) void cov_loss_kernel(CovArgs a, const M* __restrict__ mask, AggParams ap,
                                                              float* __restrict__ grad,
                                                              uint8_t* __restrict__ selected_out) {
  const int64_t row = blockIdx.x / a.chunks;
  const int chunk = blockIdx.x % a.chunks;
  const ChunkPos pos(row, chunk, a.cols);
  float o[kGroups][4], n[kGroups][4], A[kGroups][4], w[kGroups][4], iw[kGroups][4], gr[kGroups][4];
  load_groups<VEC>(a.old_lp, pos, o);
  load_groups<VEC>(a.lp, pos, n);
  load_groups<VEC>(a.adv, pos, A);
  load_mask_groups<VEC>(mask, pos, w);
  if (ISW) load_groups<VEC>(a.isw, pos, iw);
  const unsigned T = a.state->prefix, k_rem = a.state->k_rem;
  const bool take_all = a.state->take_all != 0, none = a.state->k == 0;
  const bool token_mean = ap.mode == VAMD_AGG_TOKEN_MEAN;
  float s_loss = 0, s_m = 0, s_kl = 0, s_cf = 0;
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      gr[g][e] = 0.f;
      if (e >= pos.valid[g]) continue;
      const unsigned key = a.keys[pos.idx[g] + e];
      bool sel = false;
      if (key != 0 && !none) {
        if (take_all || key > T) sel = true;
        else if (key == T) sel = atomicAdd(&a.state->tie_counter, 1u) < k_rem;
      }
      if (selected_out) selected_out[pos.idx[g] + e] = sel ? 1 : 0;
      const float d = n[g][e] - o[g][e];
      const float r = expf(d);
      float loss, dloss, kl, cf = 0.f;
      if (a.kind == kCovKl) {
        loss = -A[g][e] * r;
        dloss = loss;
        kl = fabsf(d);
        if (sel) {
          loss += a.kl_coef * kl;
          dloss += a.kl_coef * (d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f));
        }
      } else {
        const float l1 = -A[g][e] * r;
        const float rc = fminf(fmaxf(r, a.ratio_lo), a.ratio_hi);
        const float l2 = -A[g][e] * rc;
        const float in_clip = (r >= a.ratio_lo && r <= a.ratio_hi) ? 1.f : 0.f;
        const float g1 = l1 > l2 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
        const float g2 = l2 > l1 ? 1.f : (l1 == l2 ? 0.5f : 0.f);
        loss = sel ? 0.f : fmaxf(l1, l2);
        dloss = sel ? 0.f : (g1 + g2 * in_clip) * l1;
        kl = -d;
        cf = sel ? 1.f : 0.f;
      }
      if (ISW) {
        loss *= iw[g][e];
        dloss *= iw[g][e];
      }
      const float we = w[g][e];
      const bool in = we != 0.f;
      s_loss += ((token_mean && !in) ? 0.f : loss) * we;
      s_m += we;
      s_kl += in ? kl * we : 0.f;
      s_cf += in ? cf * we : 0.f;
      gr[g][e] = dloss * we;
    }
  if (GRAD) store_groups<VEC>(grad, pos, gr);
  __shared__ double smem[5 * 4];
  double acc[5] = {s_loss, s_m, s_kl, s_cf, 0.0};
  block_sum<5, kRcThreads>(acc, smem);
  if (threadIdx.x == 0) store_record<5>(a.records, row, chunk, a.rows, a.chunks, acc);
}

}  // namespace vamd

using namespace vamd;

static size_t cov_plane(int64_t rows, int64_t cols, int slots) {
  return align_up((size_t)rows * chunks_of(cols) * slots * sizeof(double), 256);
}

extern "C" size_t vamd_policy_loss_cov_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return align_up(sizeof(CovState), 256) + cov_plane(rows, cols, 4) + cov_plane(rows, cols, 5) +
         align_up((size_t)rows * cols * sizeof(unsigned), 256);
}

extern "C" int vamd_policy_loss_cov_forward(int kind, const float* old_log_prob, const float* log_prob,
                                            const float* advantages, const void* mask, int mask_dtype,
                                            const float* is_weights, int64_t rows, int64_t cols, float clip_low,
                                            float clip_high, float cov_lb, float cov_ub, double select_ratio,
                                            float ppo_kl_coef, uint64_t seed, int mode, double dp_size,
                                            double batch_num_tokens, double global_batch_size,
                                            double loss_scale_factor, float* out, float* grad_unscaled,
                                            float* coef_out, uint8_t* selected_out, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(rows > 0 && cols > 0, "policy_loss_cov: empty input");
  VAMD_REQUIRE(rows * chunks_of(cols) < (1ll << 31) && rows * cols < (1ll << 32), "policy_loss_cov: too many tokens");
  VAMD_REQUIRE(old_log_prob && log_prob && advantages && mask && out, "policy_loss_cov: null pointer");
  VAMD_REQUIRE(kind == kCovKl || kind == kCovClip, "policy_loss_cov: invalid kind %d", kind);
  VAMD_REQUIRE(mode >= 0 && mode <= 3, "policy_loss_cov: invalid mode %d", mode);
  VAMD_REQUIRE(select_ratio > 0.0, "policy_loss_cov: the selection ratio must be positive");
  VAMD_REQUIRE(!grad_unscaled || coef_out, "policy_loss_cov: grad output needs coef_out");
  if (!workspace || workspace_bytes < vamd_policy_loss_cov_workspace_bytes(rows, cols)) {
    set_error("policy_loss_cov: workspace too small");
    return VAMD_EWORKSPACE;
  }
  VAMD_REQUIRE(aligned_to(workspace, 16), "policy_loss_cov: the workspace must be 16-byte aligned");
  CovArgs a;
  a.old_lp = old_log_prob; a.lp = log_prob; a.adv = advantages; a.isw = is_weights;
  a.rows = rows; a.cols = cols; a.chunks = (int)chunks_of(cols);
  a.kind = kind;
  a.ratio_lo = (float)(1.0 - (double)clip_low);
  a.ratio_hi = (float)(1.0 + (double)clip_high);
  a.cov_lb = cov_lb; a.cov_ub = cov_ub;
  a.select_ratio = select_ratio;
  a.kl_coef = ppo_kl_coef;
  a.seed = seed;
  Carver carve(workspace);
  a.state = carve.take<CovState>(1);
  a.stats = carve.take<double>((size_t)rows * a.chunks * 4);
  a.records = carve.take<double>((size_t)rows * a.chunks * 5);
  a.keys = carve.take<unsigned>((size_t)rows * cols);
  const AggParams ap = make_agg_params(mode, dp_size, batch_num_tokens, global_batch_size, loss_scale_factor);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(rows * a.chunks)), block(kRcThreads);
  const int64_t n = rows * cols;
  const unsigned hist_blocks = (unsigned)((n + 256 * 4 * 8 - 1) / (256 * 4 * 8));  // 8 strides per workgroup
#define VAMD_COV_LOSS(V, G, W)                                                                                      \
  hipLaunchKernelGGL((cov_loss_kernel<V, M, G, W>), grid, block, 0, s, a, mk, ap, grad_unscaled, selected_out)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    const bool vec = can_vectorize(cols, {old_log_prob, log_prob, advantages, is_weights, grad_unscaled}, mask,
                                   sizeof(M));
    if (vec) hipLaunchKernelGGL((cov_stats_kernel<true, M>), grid, block, 0, s, a, mk);
    else hipLaunchKernelGGL((cov_stats_kernel<false, M>), grid, block, 0, s, a, mk);
    hipLaunchKernelGGL(cov_prepare_kernel, dim3(1), dim3(256), 0, s, a);
    if (vec) hipLaunchKernelGGL((cov_keys_kernel<true, M>), grid, block, 0, s, a, mk);
    else hipLaunchKernelGGL((cov_keys_kernel<false, M>), grid, block, 0, s, a, mk);
    for (int shift = 24; shift >= 0; shift -= 8) {
      if (shift != 24) hipLaunchKernelGGL(cov_hist_kernel, dim3(hist_blocks), dim3(256), 0, s, a.keys, n, shift, a.state);
      hipLaunchKernelGGL(cov_pick_kernel, dim3(1), dim3(256), 0, s, a.state, shift);
    }
    if (vec) {
      if (grad_unscaled) { if (is_weights) VAMD_COV_LOSS(true, true, true); else VAMD_COV_LOSS(true, true, false); }
      else { if (is_weights) VAMD_COV_LOSS(true, false, true); else VAMD_COV_LOSS(true, false, false); }
    } else {
      if (grad_unscaled) { if (is_weights) VAMD_COV_LOSS(false, true, true); else VAMD_COV_LOSS(false, true, false); }
      else { if (is_weights) VAMD_COV_LOSS(false, false, true); else VAMD_COV_LOSS(false, false, false); }
    }
  });
#undef VAMD_COV_LOSS
  hipLaunchKernelGGL((fold_loss_kernel<5, kEpiPolicy>), dim3(1), dim3(kFoldThreads), 0, s, a.records, rows, a.chunks,
                     cols, ap, coef_out, out);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
