// Generalised Advantage Estimation as a chunked associative scan (one workgroup per sequence).
//
// Reference: compute_gae_advantage_return, verl/trainer/ppo/core_algos.py:214-262.  Walking a
// row from its last column to its first, a valid step maps the carried state (nv, g) to
//     nv' = v_t ,   g' = (r_t - v_t) + gamma * nv + gamma*lam * g ,
// and a masked step leaves it unchanged.  Every step is therefore an affine map
//     nv' = a nv + b ,  g' = P nv + Q g + R           (a in {0,1})
// and maps compose associatively, so the recurrence is a prefix "sum" over maps.  A row is cut
// into segments of 1024 columns walked right to left; inside a segment each of the 256 threads
// composes its 4 columns, a wavefront scan (lane exchanges) plus an LDS pass over the wavefront totals
// yields every thread's incoming state, and the thread then replays its 4 columns to emit the
// advantages.  Loads and stores are float4 and contiguous across the wavefront; four segments are
// loaded and scanned together, so memory latency, the exchange chain and the workgroup barrier
// are paid once per 4096 columns.  The workgroup that
// finishes last folds the per-row masked moments and writes the whitening statistics, so the
// whole estimator is two launches (scan, then the elementwise whitening).
#include "rowchunk.h"

namespace vamd {

struct Affine {
  float a, b, P, Q, R;
};

__device__ __forceinline__ Affine affine_identity() { return Affine{1.f, 0.f, 0.f, 1.f, 0.f}; }

// later o earlier : apply `earlier` first
__device__ __forceinline__ Affine compose(const Affine& later, const Affine& earlier) {
  Affine o;
  o.a = later.a * earlier.a;
  o.b = fmaf(later.a, earlier.b, later.b);
  o.P = fmaf(later.P, earlier.a, later.Q * earlier.P);
  o.Q = later.Q * earlier.Q;
  o.R = fmaf(later.P, earlier.b, fmaf(later.Q, earlier.R, later.R));
  return o;
}

// The map of the lane the pattern names, the identity where there is none (composing with it changes nothing,
// so the scan needs no lane test).
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ Affine dpp_affine(const Affine& x) {
  Affine o;
  o.a = dpp_f32<CTRL, ROW_MASK>(x.a, 1.f);
  o.b = dpp_f32<CTRL, ROW_MASK>(x.b, 0.f);
  o.P = dpp_f32<CTRL, ROW_MASK>(x.P, 0.f);
  o.Q = dpp_f32<CTRL, ROW_MASK>(x.Q, 1.f);
  o.R = dpp_f32<CTRL, ROW_MASK>(x.R, 0.f);
  return o;
}
// Inclusive scan of the maps over the wavefront (lane 0 first): shifts by 1, 2, 4, 8 inside each row of 16 lanes,
// then the last lane of row 0 / 2 into rows 1 / 3, then lane 31 into rows 2 and 3.
__device__ __forceinline__ void wave_scan_step(Affine& x, int step) {
  switch (step) {
    case 0: x = compose(x, dpp_affine<0x111>(x)); break;       // row_shr:1
    case 1: x = compose(x, dpp_affine<0x112>(x)); break;       // row_shr:2
    case 2: x = compose(x, dpp_affine<0x114>(x)); break;       // row_shr:4
    case 3: x = compose(x, dpp_affine<0x118>(x)); break;       // row_shr:8
    case 4: x = compose(x, dpp_affine<0x142, 0xA>(x)); break;  // row_bcast:15 into rows 1 and 3
    default: x = compose(x, dpp_affine<0x143, 0xC>(x)); break; // row_bcast:31 into rows 2 and 3
  }
}

constexpr int kSeg = 1024;  // columns per segment = 256 threads x 4
constexpr int kSegBatch = 4;  // segments whose loads are issued together (48 KiB in flight per workgroup)

struct GaeWork {
  unsigned* ticket;   // workspace head: zero on entry, zero on exit
  double* partials;   // per row the 4 masked moments of the raw advantages; slot-major
};

template <bool VEC, class M>
__global__ __launch_bounds__(kRcThreads) void gae_scan_kernel(const float* __restrict__ rewards,
                                                              const float* __restrict__ values,
                                                              const M* __restrict__ mask, int64_t rows, int64_t cols,
                                                              float gamma, float gl, float* __restrict__ adv,
                                                              float* __restrict__ ret, GaeWork wk,
                                                              double* __restrict__ moments, float* __restrict__ stats) {
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int slot = kRcThreads - 1 - tid;  // thread 0 owns the right-most 4 columns of a segment
  __shared__ Affine wave_tot[2][kSegBatch][4];
  __shared__ float carry[2][2];
  if (tid == 0) {
    carry[0][0] = 0.f;  // nv
    carry[0][1] = 0.f;  // g
  }
  float m0 = 0, m1 = 0, m2 = 0, mc = 0;  // masked moments of the raw advantages
  const int nseg = (int)((cols + kSeg - 1) / kSeg);
  int par = 0;
  __syncthreads();
  for (int top = nseg - 1; top >= 0; top -= kSegBatch) {
    // issue every load of up to kSegBatch segments before touching any of them
    float r[kSegBatch][4], v[kSegBatch][4], w[kSegBatch][4];
    int valid[kSegBatch];
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
      const int seg = top - b;
      const int64_t c = (int64_t)seg * kSeg + slot * 4;
      const int64_t left = cols - c;
      valid[b] = seg < 0 ? 0 : (left >= 4 ? 4 : (left > 0 ? (int)left : 0));
#pragma unroll
      for (int e = 0; e < 4; ++e) r[b][e] = v[b][e] = w[b][e] = 0.f;
      if (valid[b] > 0) {
        const int64_t i = row * cols + c;
        ld4<VEC>(rewards, i, valid[b], r[b]);
        ld4<VEC>(values, i, valid[b], v[b]);
        ldmask4<VEC>(mask, i, valid[b], w[b]);
      }
    }
    // The segments of the batch are scanned together: their wavefront scans are independent (the
    // exchanges of the four interleave), and one pass over the 16 wavefront totals in walk order
    // then gives every thread the state entering its 4 columns of each segment.
    Affine inc[kSegBatch], exc[kSegBatch];
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
      // this thread's 4 columns as one map (right to left: e = 3 .. 0); segments past the row start
      // (seg < 0) hold zero masks and stay the identity
      Affine f = affine_identity();
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        if (w[b][e] != 0.f) {
          Affine n;
          n.a = 0.f;
          n.b = v[b][e];
          n.P = fmaf(gl, f.P, gamma * f.a);
          n.Q = gl * f.Q;
          n.R = fmaf(gamma, f.b, fmaf(gl, f.R, r[b][e] - v[b][e]));
          f = n;
        }
      }
      inc[b] = f;
    }
#pragma unroll
    for (int step = 0; step < 6; ++step) {
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) wave_scan_step(inc[b], step);
    }
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
      if (lane == 63) wave_tot[par][b][wave] = inc[b];
      exc[b] = dpp_affine<0x138>(inc[b]);  // wave_shr:1, the identity into lane 0
    }
    __syncthreads();
    // walk the wavefront totals in order; remember the state where this thread's wavefront starts
    float nv = carry[par][0], g = carry[par][1];
    float nv_in[kSegBatch], g_in[kSegBatch];
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (k == wave) {
          nv_in[b] = nv;
          g_in[b] = g;
        }
        const Affine t = wave_tot[par][b][k];
        const float nv2 = fmaf(t.a, nv, t.b);
        g = fmaf(t.P, nv, fmaf(t.Q, g, t.R));
        nv = nv2;
      }
    }
    if (tid == 0) {
      carry[par ^ 1][0] = nv;
      carry[par ^ 1][1] = g;
    }
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
      const int seg = top - b;
      if (seg < 0) break;
      nv = fmaf(exc[b].a, nv_in[b], exc[b].b);
      g = fmaf(exc[b].P, nv_in[b], fmaf(exc[b].Q, g_in[b], exc[b].R));
      // replay the 4 columns
      float a_out[4], r_out[4];
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        if (w[b][e] != 0.f) {
          const float delta = r[b][e] + gamma * nv - v[b][e];
          g = fmaf(gl, g, delta);
          nv = v[b][e];
          m1 += g * w[b][e];
          m2 += g * g * w[b][e];
          mc += 1.f;
        }
        m0 += w[b][e];
        a_out[e] = g;
        r_out[e] = g + v[b][e];
      }
      if (valid[b] > 0) {
        const int64_t i = row * cols + (int64_t)seg * kSeg + slot * 4;
        st4<VEC>(adv, i, valid[b], a_out);
        st4<VEC>(ret, i, valid[b], r_out);
      }
    }
    par ^= 1;
  }
  __shared__ double smem[16];
  double acc[4] = {m0, m1, m2, mc};
  block_sum<4, kRcThreads>(acc, smem);
  if (tid == 0) {
    store_record<4>(wk.partials, row, 0, rows, 1, acc);
  }
  if (!last_block_arrives(wk.ticket)) return;
  // the last row to finish folds the per-row moments and derives the whitening statistics
  double a[4] = {0, 0, 0, 0};
  sum_records_strided<4>(wk.partials, rows, a);
  block_sum<4, kRcThreads>(a, smem);
  if (tid == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) moments[i] = a[i];
    whiten_stats_from_moments(a[0], a[1], a[2], 1, stats);
  }
  ticket_reset(wk.ticket);
}

}  // namespace vamd

using namespace vamd;

extern "C" size_t vamd_gae_workspace_bytes(int64_t batch, int64_t length) {
  if (batch <= 0 || length <= 0) return 0;
  return kTicketBytes + align_up((size_t)batch * 4 * sizeof(double), 256) + 256 /* moments */ + 256 /* stats */;
}

extern "C" int vamd_gae(const float* rewards, const float* values, const void* mask, int mask_dtype, int64_t batch,
                        int64_t length, float gamma, float lam, int whiten, float* advantages, float* returns,
                        double* moments_out, void* workspace, size_t workspace_bytes, void* stream) {
  VAMD_REQUIRE(batch > 0 && length > 0, "gae: empty input");
  VAMD_REQUIRE(batch < (1ll << 31), "gae: batch too large");
  VAMD_REQUIRE(rewards && values && mask && advantages && returns, "gae: null pointer");
  if (!workspace || workspace_bytes < vamd_gae_workspace_bytes(batch, length)) {
    set_error("gae: workspace too small");
    return VAMD_EWORKSPACE;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  GaeWork wk;
  wk.ticket = static_cast<unsigned*>(workspace);
  Carver carve(static_cast<char*>(workspace) + kTicketBytes);
  wk.partials = carve.take<double>((size_t)batch * 4);
  double* moments = carve.take<double>(4);
  float* stats = carve.take<float>(4);
  double* mom = moments_out ? moments_out : moments;
  const float gl = (float)((double)gamma * (double)lam);
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(length, {rewards, values, advantages, returns}, mask, sizeof(M));
    if (vec)
      hipLaunchKernelGGL((gae_scan_kernel<true, M>), dim3((unsigned)batch), dim3(kRcThreads), 0, s, rewards, values,
                         static_cast<const M*>(mask), batch, length, gamma, gl, advantages, returns, wk, mom, stats);
    else
      hipLaunchKernelGGL((gae_scan_kernel<false, M>), dim3((unsigned)batch), dim3(kRcThreads), 0, s, rewards, values,
                         static_cast<const M*>(mask), batch, length, gamma, gl, advantages, returns, wk, mom, stats);
  });
  VAMD_LAUNCH_CHECK();
  if (whiten) return vamd_affine_by_stats(advantages, stats, batch * length, advantages, stream);
  return VAMD_OK;
}
