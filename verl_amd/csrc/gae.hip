// Generalised Advantage Estimation as a chunked associative scan.
//
// Reference: compute_gae_advantage_return, verl/trainer/ppo/core_algos.py:214-262.  Walking a row from its last
// column to its first, a valid step maps the carried state (nv, g) to
//     nv' = v_t ,   g' = (r_t - v_t + gamma nv) + gamma*lam g ,
// and a masked step leaves it unchanged.  The two halves of the state are scanned one after the other, which keeps
// what the lanes exchange small:
//   1. nv entering a column is the value at the nearest valid column to its right: a "most recent flagged value"
//      scan.  Inside a wavefront it is one ballot, one count-leading-zeros and one lane read; across the 16
//      (segment, wavefront) pieces of a batch the first 16 lanes of wavefront 0 do the same once.
//   2. with nv known, delta_t = r_t - v_t + gamma nv_t is data, and g' = gamma*lam g + delta_t (valid) / g (masked)
//      is a one-variable affine map (Q, R): composing two of them is a multiply and a fused multiply-add.  A
//      wavefront scans its 64 lane maps with six lane-exchange steps; wavefront 0 scans the 16 piece totals.
// A row is cut into segments of 1024 columns (256 threads x 4) walked right to left, four segments per batch
// with all their loads issued together; every thread then replays its 4 columns per segment to emit the advantages.
//
// With whitening the whole estimator is ONE launch: every workgroup keeps a record of the masked moments of its
// rows, the workgroup that arrives last folds them into (mean, rstd) and opens the gate the others wait at, and
// each workgroup then whitens what it produced.  The last three batches a workgroup walked wait on chip (one in
// registers, two in LDS) and are written once, whitened; earlier batches were stored raw and are read back.
#include "rowchunk.h"

namespace vamd {

constexpr int kSeg = 1024;       // columns per segment = 256 threads x 4
constexpr int kSegBatch = 4;     // segments whose loads are issued together (48 KiB in flight per workgroup)
constexpr int kPieces = kSegBatch * (kRcThreads / 64);  // (segment, wavefront) pieces of a batch, in walk order
static_assert(kPieces == 16, "wavefront 0 scans the piece totals inside one row of 16 lanes");

constexpr int kGaeLdsHeld = 2;   // batches of a workgroup that wait in LDS across the rendezvous (32 KiB)

struct GaeWork {
  unsigned* ticket;   // workspace head: zero on entry, zero on exit
  double* partials;   // per workgroup the 4 masked moments of the raw advantages; slot-major
};

// g -> Q g + R
struct Lin {
  float Q, R;
};
// later o earlier : apply `earlier` first
__device__ __forceinline__ Lin lin_after(const Lin& later, const Lin& earlier) {
  return Lin{later.Q * earlier.Q, fmaf(later.Q, earlier.R, later.R)};
}
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ Lin dpp_lin(const Lin& x) {  // the identity where the pattern names no lane
  return Lin{dpp_f32<CTRL, ROW_MASK>(x.Q, 1.f), dpp_f32<CTRL, ROW_MASK>(x.R, 0.f)};
}
__device__ __forceinline__ void row_scan_lin(Lin& x) {  // inclusive, inside each row of 16 lanes
  x = lin_after(x, dpp_lin<0x111>(x));  // row_shr:1
  x = lin_after(x, dpp_lin<0x112>(x));  // row_shr:2
  x = lin_after(x, dpp_lin<0x114>(x));  // row_shr:4
  x = lin_after(x, dpp_lin<0x118>(x));  // row_shr:8
}
__device__ __forceinline__ void wave_scan_lin_tail(Lin& x) {  // rows -> whole wavefront
  x = lin_after(x, dpp_lin<0x142, 0xA>(x));  // row_bcast:15 into rows 1 and 3
  x = lin_after(x, dpp_lin<0x143, 0xC>(x));  // row_bcast:31 into rows 2 and 3
}

// Among the lanes below `lane` whose bit is set in `flags`, the highest; -1 if none.
__device__ __forceinline__ int nearest_flagged_below(unsigned long long flags, int lane) {
  const unsigned long long lower = flags & ((1ull << lane) - 1ull);
  return lower ? 63 - __clzll((long long)lower) : -1;
}

struct GaeArgs {
  const float* rewards;
  const float* values;
  const void* mask;
  int64_t rows, cols;
  float gamma, gl;
  float* adv;
  float* ret;
  GaeWork wk;
  double* moments;  // [5]: sum m, sum g m, sum g^2 m, count, 1.0 if the rendezvous timed out
  float* stats;     // [4]: mean, rstd, shift
  unsigned spin_limit;
  int lds_held;     // batches per workgroup that wait in LDS (the launch's dynamic LDS holds them)
};

template <bool VEC, class M, bool WHITEN>
__global__ __launch_bounds__(kRcThreads) void gae_kernel(GaeArgs a) {
  const M* __restrict__ mask = static_cast<const M*>(a.mask);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int slot = kRcThreads - 1 - tid;  // thread 0 owns the right-most 4 columns of a segment
  __shared__ float nv_piece_val[kPieces], nv_in_piece[kPieces], g_in_piece[kPieces];
  __shared__ unsigned nv_piece_flag[kPieces];
  __shared__ Lin piece_total[kPieces];
  __shared__ float carry[2];  // nv, g entering the batch
  const float gamma = a.gamma, gl = a.gl;
  const int64_t cols = a.cols;
  const int nseg = (int)((cols + kSeg - 1) / kSeg);
  // With whitening, the advantages of the last batches a workgroup walks stay on chip across the rendezvous (the very
  // last in registers, up to two before it in LDS when the launch brought the room, each thread its own columns): they are neither stored raw nor
  // read back.  At 512 x 4096 that is everything; at 2048 x 16384 on 1024 workgroups three batches of eight.
  extern __shared__ float4 lds_keep_raw[];  // [a.lds_held * kSegBatch][kRcThreads], sized by the launch
  float4(*lds_keep)[kRcThreads] = reinterpret_cast<float4(*)[kRcThreads]>(lds_keep_raw);
  const int kLdsHeld = WHITEN ? a.lds_held : 0;
  const int batches_per_row = (nseg + kSegBatch - 1) / kSegBatch;
  const int64_t own_rows = (a.rows - blockIdx.x + gridDim.x - 1) / gridDim.x;
  const int64_t last_batch = own_rows * batches_per_row - 1;
  int64_t batch_no = 0;
  const bool streaming = streams_past_caches(a.rows * cols);
  float keep[kSegBatch][4];
  float m0 = 0, m1 = 0, m2 = 0, mc = 0;  // masked moments of the raw advantages

  for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x) {
    __syncthreads();
    if (tid == 0) carry[0] = carry[1] = 0.f;
    for (int top = nseg - 1; top >= 0; top -= kSegBatch, ++batch_no) {
      const int64_t from_end = last_batch - batch_no;  // 0: stays in registers; 1..kLdsHeld: stays in LDS
      const bool on_chip = WHITEN && from_end <= kLdsHeld;
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
          ld4<VEC>(a.rewards, i, valid[b], r[b], streaming);
          ld4<VEC>(a.values, i, valid[b], v[b], streaming);
          ldmask4<VEC>(mask, i, valid[b], w[b], streaming);
        }
      }
      // ---- 1. nv: the value the thread leaves behind (its lowest valid column), and who is nearest before it
      float left_val[kSegBatch];
      int src_lane[kSegBatch];
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        bool any = false;
        float val = 0.f;
#pragma unroll
        for (int e = 3; e >= 0; --e) {  // selects, not branches: a wavefront's lanes disagree about every column
          const bool on = w[b][e] != 0.f;
          any = any || on;
          val = on ? v[b][e] : val;
        }
        left_val[b] = val;
        const unsigned long long flags = __ballot(any);
        src_lane[b] = nearest_flagged_below(flags, lane);
        if (lane == 0) {
          nv_piece_flag[b * 4 + wave] = flags != 0ull;
          // the wavefront's last word: its highest flagged lane
          nv_piece_val[b * 4 + wave] = 0.f;
        }
        const int top_lane = flags ? 63 - __clzll((long long)flags) : 0;
        const float wave_val = __shfl(val, top_lane, 64);
        if (lane == 0 && flags) nv_piece_val[b * 4 + wave] = wave_val;
      }
      __syncthreads();
      if (wave == 0) {  // nv entering each piece: the nearest flagged piece before it, else the batch's carry
        const bool mine = lane < kPieces;
        const bool flagged = mine && nv_piece_flag[mine ? lane : 0] != 0u;
        const float val = mine ? nv_piece_val[lane] : 0.f;
        const unsigned long long flags = __ballot(flagged);
        const int src = nearest_flagged_below(flags, lane);
        const float from = __shfl(val, src < 0 ? 0 : src, 64);
        const float c_nv = carry[0];
        if (mine) nv_in_piece[lane] = src < 0 ? c_nv : from;
        if (lane == kPieces - 1) carry[0] = flagged ? val : (src < 0 ? c_nv : from);
      }
      __syncthreads();
      // ---- 2. g: the thread's 4 columns as one map; delta replaces the reward in place
      Lin inc[kSegBatch], exc[kSegBatch];
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        const float from_lane = __shfl(left_val[b], src_lane[b] < 0 ? 0 : src_lane[b], 64);
        float nv = src_lane[b] < 0 ? nv_in_piece[b * 4 + wave] : from_lane;
        Lin f{1.f, 0.f};
#pragma unroll
        for (int e = 3; e >= 0; --e) {
          const bool on = w[b][e] != 0.f;
          const float delta = fmaf(gamma, nv, r[b][e] - v[b][e]);
          f.R = on ? fmaf(gl, f.R, delta) : f.R;
          f.Q = on ? f.Q * gl : f.Q;
          nv = on ? v[b][e] : nv;
          r[b][e] = delta;  // read again only where the column is valid
        }
        inc[b] = f;
      }
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) row_scan_lin(inc[b]);
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) wave_scan_lin_tail(inc[b]);
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        if (lane == 63) piece_total[b * 4 + wave] = inc[b];
        exc[b] = dpp_lin<0x138>(inc[b]);  // wave_shr:1, the identity into lane 0
      }
      __syncthreads();
      if (wave == 0) {  // g entering each piece
        Lin t = lane < kPieces ? piece_total[lane] : Lin{1.f, 0.f};
        row_scan_lin(t);
        const Lin before = dpp_lin<0x111>(t);  // exclusive: the pieces before this one
        const float c_g = carry[1];
        if (lane < kPieces) g_in_piece[lane] = fmaf(before.Q, c_g, before.R);
        if (lane == kPieces - 1) carry[1] = fmaf(t.Q, c_g, t.R);
      }
      __syncthreads();
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        const int seg = top - b;
        if (seg < 0) break;
        float g = fmaf(exc[b].Q, g_in_piece[b * 4 + wave], exc[b].R);
        float a_out[4], r_out[4];
#pragma unroll
        for (int e = 3; e >= 0; --e) {
          const bool on = w[b][e] != 0.f;
          g = on ? fmaf(gl, g, r[b][e]) : g;
          const float gw = on ? g * w[b][e] : 0.f;
          m1 += gw;
          m2 = fmaf(g, gw, m2);
          mc += on ? 1.f : 0.f;
          m0 += w[b][e];
          a_out[e] = g;
          r_out[e] = g + v[b][e];
        }
        if (valid[b] > 0) {
          const int64_t i = row * cols + (int64_t)seg * kSeg + slot * 4;
          st4<VEC>(a.ret, i, valid[b], r_out, streaming);
          if (!on_chip) st4<VEC>(a.adv, i, valid[b], a_out, streaming && !WHITEN);  // WHITEN: read back after the rendezvous
        }
        if (WHITEN && from_end >= 1 && from_end <= kLdsHeld)
          lds_keep[(from_end - 1) * kSegBatch + b][tid] = make_float4(a_out[0], a_out[1], a_out[2], a_out[3]);
#pragma unroll
        for (int e = 0; e < 4; ++e) keep[b][e] = a_out[e];
      }
    }
  }

  __shared__ double smem[16];
  double acc[4] = {m0, m1, m2, mc};
  block_sum<4, kRcThreads>(acc, smem);
  if (tid == 0) store_record<4>(a.wk.partials, blockIdx.x, 0, gridDim.x, 1, acc);
  const bool last = last_block_arrives(a.wk.ticket);
  if (last) {  // fold the workgroups' moments, derive the whitening statistics
    double t[4] = {0, 0, 0, 0};
    sum_records_strided<4>(a.wk.partials, gridDim.x, t);
    block_sum<4, kRcThreads>(t, smem);
    if (tid == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) a.moments[i] = t[i];
      float st[3];
      whiten_stats_from_moments(t[0], t[1], t[2], 1, st);
#pragma unroll
      for (int i = 0; i < 3; ++i) peer_store_f32(a.stats + i, st[i]);
      if (WHITEN) gate_release(a.wk.ticket);  // waits for the stores above before it opens the gate
    }
    __syncthreads();  // the other threads of this workgroup read the statistics next
  }
  if (!WHITEN) {
    if (last) {
      if (tid == 0) a.moments[4] = 0.0;
      ticket_reset(a.wk.ticket);
    }
    return;
  }
  const bool open = last || gate_wait(a.wk.ticket, a.spin_limit);
  // A wait that ran out leaves the advantages raw (the host is told through moments[4]): what is in memory stays as it
  // is, what was kept on chip is stored unchanged.
  const float mean = open ? peer_load_f32(a.stats) : 0.f, rstd = open ? peer_load_f32(a.stats + 1) : 1.f;
  if (last_batch == 0) {  // one row of one batch (512 x 4096 is such a launch): straight from the registers
#pragma unroll
    for (int b = 0; b < kSegBatch; ++b) {
      const int seg = nseg - 1 - b;
      const int64_t c = (int64_t)seg * kSeg + slot * 4;
      const int64_t left = cols - c;
      const int n_ok = seg < 0 ? 0 : (left >= 4 ? 4 : (left > 0 ? (int)left : 0));
      if (n_ok <= 0) continue;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (keep[b][e] - mean) * rstd;
      st4<VEC>(a.adv, (int64_t)blockIdx.x * cols + c, n_ok, o, streaming);
    }
  } else {
  batch_no = 0;
  for (int64_t row = blockIdx.x; row < a.rows; row += gridDim.x)
    for (int top = nseg - 1; top >= 0; top -= kSegBatch, ++batch_no) {  // the same walk: every thread meets its own columns
      const int64_t from_end = last_batch - batch_no;
      if (!open && from_end > kLdsHeld) continue;
      float x[kSegBatch][4];
      int n_ok[kSegBatch];
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        const int seg = top - b;
        const int64_t c = (int64_t)seg * kSeg + slot * 4;
        const int64_t left = cols - c;
        n_ok[b] = seg < 0 ? 0 : (left >= 4 ? 4 : (left > 0 ? (int)left : 0));
        if (n_ok[b] <= 0) continue;
        if (from_end == 0) {
#pragma unroll
          for (int e = 0; e < 4; ++e) x[b][e] = keep[b][e];
        } else if (from_end <= kLdsHeld) {
          const float4 k4 = lds_keep[(from_end - 1) * kSegBatch + b][tid];
          x[b][0] = k4.x, x[b][1] = k4.y, x[b][2] = k4.z, x[b][3] = k4.w;
        } else {
          ld4<VEC>(a.adv, row * cols + c, n_ok[b], x[b], false);
        }
      }
#pragma unroll
      for (int b = 0; b < kSegBatch; ++b) {
        if (n_ok[b] <= 0) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[b][e] = (x[b][e] - mean) * rstd;
        st4<VEC>(a.adv, row * cols + (int64_t)(top - b) * kSeg + slot * 4, n_ok[b], x[b], streaming);
      }
    }
  }
  const unsigned verdict = gate_depart(a.wk.ticket);
  if (verdict != 0 && tid == 0) a.moments[4] = verdict > 1 ? 1.0 : 0.0;
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
  GaeArgs a;
  a.wk.ticket = static_cast<unsigned*>(workspace);
  Carver carve(static_cast<char*>(workspace) + kTicketBytes);
  a.wk.partials = carve.take<double>((size_t)batch * 4);
  double* moments = carve.take<double>(8);
  a.stats = carve.take<float>(4);
  a.moments = moments_out ? moments_out : moments;
  a.rewards = rewards;
  a.values = values;
  a.mask = mask;
  a.rows = batch;
  a.cols = length;
  a.gamma = gamma;
  a.gl = (float)((double)gamma * (double)lam);
  a.adv = advantages;
  a.ret = returns;
  a.spin_limit = gate_spin_limit(kGateSpinLimit);
  // The workgroups wait for each other before whitening, so the grid never exceeds what the device holds at once;
  // beyond that a workgroup walks several rows.
  auto launch = [&](auto kernel) -> int {
    int64_t grid = batch;
    size_t lds = 0;
    a.lds_held = 0;
    if (whiten) {
      // LDS for the batches that wait on chip beside the one in registers: none when a workgroup walks a single batch
      const int64_t batches_per_row = (length + (int64_t)kSeg * kSegBatch - 1) / ((int64_t)kSeg * kSegBatch);
      const void* k = reinterpret_cast<const void*>(kernel);
      grid = balanced_waiting_grid(batch, resident_workgroups(k, kRcThreads, 0));
      if ((batch + grid - 1) / grid * batches_per_row > 1) {
        a.lds_held = kGaeLdsHeld;
        lds = (size_t)kGaeLdsHeld * kSegBatch * kRcThreads * sizeof(float4);
        grid = balanced_waiting_grid(batch, resident_workgroups(k, kRcThreads, lds));
      }
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kRcThreads), lds, s, a);
    return VAMD_OK;
  };
  // whiten == 2, or waiting kernels switched off: the scan launch leaves the statistics, a second launch applies them
  const bool apart = whiten != 0 && (whiten == 2 || !waiting_kernels_allowed());
  if (apart) whiten = 0;
  VAMD_MASK_DISPATCH(mask_dtype, M, {
    const bool vec = can_vectorize(length, {rewards, values, advantages, returns}, mask, sizeof(M));
    if (whiten) {
      if (vec) launch(gae_kernel<true, M, true>);
      else launch(gae_kernel<false, M, true>);
    } else {
      if (vec) launch(gae_kernel<true, M, false>);
      else launch(gae_kernel<false, M, false>);
    }
  });
  VAMD_LAUNCH_CHECK();
  if (apart) return vamd_affine_by_stats(advantages, a.stats, batch * length, advantages, stream);
  return VAMD_OK;
}
