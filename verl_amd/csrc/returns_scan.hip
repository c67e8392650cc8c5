// Token-level return estimators that are one-variable reverse recurrences over a response:
//
//   ReMax        returns_t = sum_{s >= t} r_s m_s ;  adv = returns - baseline_i * m
//                (compute_remax_outcome_advantage, verl/trainer/ppo/core_algos.py:621-654)
//   REINFORCE++  walking t = L-1 .. 0:  R_t = r_t + gamma * c ;  c <- R_t * m_t  (reset after EOS);
//                adv = masked_whiten(R, m) * m
//                (compute_reinforce_plus_plus_outcome_advantage, core_algos.py:582-618)
//
// Both carry one value y leftwards through the affine step y' = a_t y + b_t
// (ReMax: a = 1, b = r m, output y';  REINFORCE++: a = gamma m, b = r m, output r + gamma y), and
// affine steps compose associatively, so a row is scanned like the GAE kernel scans its pairs:
// 1024-column segments right to left, 4 columns per thread, a wavefront scan by lane exchanges plus an LDS
// pass over the 4 wavefront totals, loads of four segments issued together.  The workgroup that
// finishes last folds the per-row masked moments of the returns into whitening statistics; a second
// streaming kernel forms the advantages.
#include "rowchunk.h"

namespace vamd {

enum : int { kReturnsRemax = 0, kReturnsReinforcePP = 1 };

struct Step {
  float a, b;
};

// later o earlier : apply `earlier` first
__device__ __forceinline__ Step compose(const Step& later, const Step& earlier) {
  return Step{later.a * earlier.a, fmaf(later.a, earlier.b, later.b)};
}

constexpr int kRsSeg = 1024;
constexpr int kRsBatch = 4;

struct ReturnsWork {
  unsigned* ticket;  // workspace head: zero on entry, zero on exit
  double* partials;  // per row sum(m), sum(R m), sum(R^2 m) with R zeroed outside the mask; slot-major
};

template <bool VEC, class M, int MODE>
__global__ __launch_bounds__(kRcThreads) void returns_scan_kernel(const float* __restrict__ rewards,
                                                                  const M* __restrict__ mask, int64_t rows,
                                                                  int64_t cols, float gamma,
                                                                  float* __restrict__ ret, ReturnsWork wk,
                                                                  double* __restrict__ moments,
                                                                  float* __restrict__ stats) {
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int slot = kRcThreads - 1 - tid;  // thread 0 owns the right-most 4 columns of a segment
  __shared__ Step wave_tot[2][4];
  __shared__ float carry[2];
  if (tid == 0) carry[0] = 0.f;
  float m0 = 0, m1 = 0, m2 = 0;
  const int nseg = (int)((cols + kRsSeg - 1) / kRsSeg);
  int par = 0;
  __syncthreads();
  for (int top = nseg - 1; top >= 0; top -= kRsBatch) {
    float r[kRsBatch][4], w[kRsBatch][4];
    int valid[kRsBatch];
#pragma unroll
    for (int b = 0; b < kRsBatch; ++b) {
      const int seg = top - b;
      const int64_t c = (int64_t)seg * kRsSeg + slot * 4;
      const int64_t left = cols - c;
      valid[b] = seg < 0 ? 0 : (left >= 4 ? 4 : (left > 0 ? (int)left : 0));
#pragma unroll
      for (int e = 0; e < 4; ++e) r[b][e] = w[b][e] = 0.f;
      if (valid[b] > 0) {
        const int64_t i = row * cols + c;
        ld4<VEC>(rewards, i, valid[b], r[b]);
        ldmask4<VEC>(mask, i, valid[b], w[b]);
      }
    }
#pragma unroll
    for (int b = 0; b < kRsBatch; ++b) {
      const int seg = top - b;
      if (seg < 0) break;
      // this thread's 4 columns as one step (right to left: e = 3 .. 0); columns past the row end
      // are the identity
      Step f{1.f, 0.f};
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        if (e < valid[b]) {
          const Step s{MODE == kReturnsRemax ? 1.f : gamma * w[b][e], r[b][e] * w[b][e]};
          f = compose(s, f);
        }
      }
      Step inc = f;  // inclusive scan over the wavefront; a lane without a source composes with the identity
      inc = compose(inc, Step{dpp_f32<0x111>(inc.a, 1.f), dpp_f32<0x111>(inc.b, 0.f)});
      inc = compose(inc, Step{dpp_f32<0x112>(inc.a, 1.f), dpp_f32<0x112>(inc.b, 0.f)});
      inc = compose(inc, Step{dpp_f32<0x114>(inc.a, 1.f), dpp_f32<0x114>(inc.b, 0.f)});
      inc = compose(inc, Step{dpp_f32<0x118>(inc.a, 1.f), dpp_f32<0x118>(inc.b, 0.f)});
      inc = compose(inc, Step{dpp_f32<0x142, 0xA>(inc.a, 1.f), dpp_f32<0x142, 0xA>(inc.b, 0.f)});
      inc = compose(inc, Step{dpp_f32<0x143, 0xC>(inc.a, 1.f), dpp_f32<0x143, 0xC>(inc.b, 0.f)});
      if (lane == 63) wave_tot[par][wave] = inc;
      const Step exc{dpp_f32<0x138>(inc.a, 1.f), dpp_f32<0x138>(inc.b, 0.f)};  // the lane before; identity into lane 0
      __syncthreads();
      float y = carry[par];
      for (int k = 0; k < wave; ++k) y = fmaf(wave_tot[par][k].a, y, wave_tot[par][k].b);
      y = fmaf(exc.a, y, exc.b);
      float out[4];
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        out[e] = 0.f;
        if (e < valid[b]) {
          float R;
          if (MODE == kReturnsRemax) {
            y = fmaf(r[b][e], w[b][e], y);
            R = y;
          } else {
            R = fmaf(gamma, y, r[b][e]);
            y = R * w[b][e];
          }
          out[e] = R;
          const float we = w[b][e];
          const float Rm = we != 0.f ? R : 0.f;  // where(mask.bool(), values, 0)
          m0 += we;
          m1 += Rm * we;
          m2 += Rm * Rm * we;
        }
      }
      if (tid == kRcThreads - 1) carry[par ^ 1] = y;
      if (valid[b] > 0) st4<VEC>(ret, row * cols + (int64_t)seg * kRsSeg + slot * 4, valid[b], out);
      __syncthreads();
      par ^= 1;
    }
  }
  __shared__ double smem[12];
  double acc[3] = {m0, m1, m2};
  block_sum<3, kRcThreads>(acc, smem);
  if (tid == 0) {
    store_record<3>(wk.partials, row, 0, rows, 1, acc);
  }
  if (!last_block_arrives(wk.ticket)) return;
  double a[3] = {0, 0, 0};
  sum_records_strided<3>(wk.partials, rows, a);
  block_sum<3, kRcThreads>(a, smem);
  if (tid == 0) {
#pragma unroll
    for (int i = 0; i < 3; ++i) moments[i] = a[i];
    whiten_stats_from_moments(a[0], a[1], a[2], 1, stats);
  }
  ticket_reset(wk.ticket);
}

// ReMax: adv = R - baseline[row] * m ;  REINFORCE++: adv = (R - mean) * rstd * m
template <bool VEC, class M, int MODE>
__global__ __launch_bounds__(kRcThreads) void returns_finish_kernel(const float* __restrict__ ret,
                                                                    const M* __restrict__ mask,
                                                                    const float* __restrict__ baseline,
                                                                    const float* __restrict__ stats, int64_t cols,
                                                                    int chunks, float* __restrict__ adv) {
  const int64_t row = blockIdx.x / chunks;
  const int chunk = blockIdx.x % chunks;
  const ChunkPos pos(row, chunk, cols);
  float x[kGroups][4], w[kGroups][4];
  load_groups<VEC>(ret, pos, x);
  load_mask_groups<VEC>(mask, pos, w);
  const float p0 = MODE == kReturnsRemax ? baseline[row] : stats[0];
  const float p1 = MODE == kReturnsRemax ? 0.f : stats[1];
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e)
      x[g][e] = MODE == kReturnsRemax ? x[g][e] - p0 * w[g][e] : ((x[g][e] - p0) * p1) * w[g][e];
  store_groups<VEC>(adv, pos, x);
}

}  // namespace vamd

using namespace vamd;

extern "C" size_t vamd_returns_advantage_workspace_bytes(int64_t batch, int64_t length) {
  if (batch <= 0 || length <= 0) return 0;
  return kTicketBytes + align_up((size_t)batch * 3 * sizeof(double), 256) + 256 /* moments */ + 256 /* stats */;
}

extern "C" int vamd_returns_advantage(const float* rewards, const void* mask, int mask_dtype,
                                      const float* row_baseline, int64_t batch, int64_t length, float gamma,
                                      int mode, float* advantages, float* returns, double* moments_out,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "returns_advantage: empty input");
  VAMD_REQUIRE(batch * chunks_of(length) < (1ll << 31), "returns_advantage: too many workgroups");
  VAMD_REQUIRE(rewards && mask && advantages && returns, "returns_advantage: null pointer");
  VAMD_REQUIRE(mode == kReturnsRemax || mode == kReturnsReinforcePP, "returns_advantage: invalid mode %d", mode);
  VAMD_REQUIRE(mode != kReturnsRemax || row_baseline, "returns_advantage: ReMax needs the per-response baselines");
  if (!workspace || workspace_bytes < vamd_returns_advantage_workspace_bytes(batch, length)) {
    set_error("returns_advantage: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  ReturnsWork wk;
  wk.ticket = static_cast<unsigned*>(workspace);
  Carver carve(static_cast<char*>(workspace) + kTicketBytes);
  wk.partials = carve.take<double>((size_t)batch * 3);
  double* moments = carve.take<double>(4);
  float* stats = carve.take<float>(4);
  double* mom = moments_out ? moments_out : moments;
  const int chunks = (int)chunks_of(length);
  const dim3 fin_grid((unsigned)(batch * chunks));
#define VAMD_RS(V, MODE)                                                                                         \
  do {                                                                                                           \
    hipLaunchKernelGGL((returns_scan_kernel<V, M, MODE>), dim3((unsigned)batch), dim3(kRcThreads), 0, s, rewards, \
                       mk, batch, length, gamma, returns, wk, mom, stats);                                       \
    hipLaunchKernelGGL((returns_finish_kernel<V, M, MODE>), fin_grid, dim3(kRcThreads), 0, s, returns, mk,        \
                       row_baseline, stats, length, chunks, advantages);                                         \
  } while (0)
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const M* mk = static_cast<const M*>(mask);
    const bool vec = can_vectorize(length, {rewards, advantages, returns}, mask, sizeof(M));
    if (mode == kReturnsRemax) {
      if (vec) VAMD_RS(true, kReturnsRemax); else VAMD_RS(false, kReturnsRemax);
    } else {
      if (vec) VAMD_RS(true, kReturnsReinforcePP); else VAMD_RS(false, kReturnsReinforcePP);
    }
  });
#undef VAMD_RS
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
