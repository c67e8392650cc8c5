// Fused vocab-projection log-prob / entropy head for gfx950.
//
// Forward : logits tiles are produced by the MFMA tile engine and consumed in registers by an
//           online-softmax epilogue (running max, sum exp, sum z*exp, label logit and, on request,
//           sum exp^2 per token).  The [tokens, vocab] logits are not needed afterwards; on request
//           they are also written out in fp32 as a cache for the backward pass.
// Backward: per vocabulary chunk, d_logits is formed as one bf16 [tokens, vocab_chunk] panel,
//           either from the cached logits (a streaming pass) or from logits tiles recomputed by
//           the tile engine; the same engine then forms
//           d_hidden (+)= panel . W[chunk]  and  d_weight[chunk] = panel^T . hidden  in one launch.
//
// Arithmetic follows LinearCrossEntropy (verl/utils/kernel/linear_cross_entropy.py:40-116) /
// efficient_entropy_forward+backward (verl/utils/kernel/kernels.py:563-753, :1512-1723): bf16
// products, fp32 accumulation, logits scaled by 1/temperature in fp32, fp32 softmax state.
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "common.h"
#include "gemm_core.h"

namespace vamd {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;  // stands in for -inf so that (x - x) and 0 * x stay finite
// What a column past the end of the vocabulary holds in place of its product.  Times any sensible
// log2(e) / temperature it stays below kNegBig, the running maximum's start value (or overflows to -inf, which the
// maximum ignores as well): the maximum is never taken from it, so its exponent is hugely negative against every
// maximum there can be and it contributes exactly 0 to the sums (0 times a finite number).
constexpr float kNoColumn = -3.0e38f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Optional per-kernel timing for benchmarks: when enabled, every head kernel launch (from any
// thread: autograd runs backward on its own) is bracketed by a pair of HIP events on the launch
// stream.
enum : int { kTagForward = 0, kTagMerge = 1, kTagRecompute = 2, kTagDGrad = 3, kTagDLogits = 4, kNumTags = 5 };
struct TimedLaunch {
  int tag;
  hipEvent_t start, stop;
};
static std::atomic<bool> g_timing_on{false};
static std::mutex g_timed_mu;
static std::vector<TimedLaunch> g_timed;

struct ScopedTiming {
  hipStream_t s;
  TimedLaunch t;
  bool on;
  ScopedTiming(int tag, hipStream_t stream) : s(stream), on(g_timing_on.load()) {
    if (!on) return;
    t.tag = tag;
    if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) {
      on = false;
      return;
    }
    (void)hipEventRecord(t.start, s);
  }
  ~ScopedTiming() {
    if (!on) return;
    (void)hipEventRecord(t.stop, s);
    std::lock_guard<std::mutex> lock(g_timed_mu);
    g_timed.push_back(t);
  }
};

// =============================================================================================
// Forward
// =============================================================================================
struct FwdArgs {
  Operand hidden;  // R operand: [n_tokens][H]
  Operand weight;  // C operand: [vocab][H]
  const int64_t* labels;
  int n_tokens, vocab, k_slabs;
  int tok_tiles, voc_tiles, splits;
  float scale2;      // log2(e) / temperature
  float rcp_t;       // 1 / temperature
  float4* partials;  // [splits][tok_tiles * 256] : (max in the log2 domain, sum e, sum e x with x = hidden . weight, label logit)
  float* z_cache;    // optional [n_tokens][vocab] fp32 logits / temperature, kept for the backward
  float* pi2_partials;  // optional [splits][tok_tiles * 256] : sum of e^2 relative to the same max
};

struct SplitSched {
  int r0_, vt_begin, vt_count;
  __device__ __forceinline__ int count() const { return vt_count; }
  __device__ __forceinline__ void tile(int i, int& r0, int& c0) const {
    r0 = r0_;
    c0 = (vt_begin + i) * kTile;
  }
};

// The epilogues that write matrices hand the accumulators through a 4 KB LDS patch private to the
// wavefront (the 32 KB the pipeline leaves free), 32 x 32 values at a time (2 x 2 MFMA blocks), so that
// global accesses are whole 128-byte rows of fp32 (64-byte rows of bf16) touched by 8 consecutive
// lanes instead of 16-byte pieces of 16 different rows.  After the exchange lane L holds columns
// 4 (L % 8) .. + 3 of rows 8 i + L / 8 (i = 0..3) of the 32 x 32 patch.  LDS operations of one wavefront
// execute in issue order, so the patch needs no barrier, only the waits that order its writes and reads.
constexpr int kNB2 = kNB / 2, kMB2 = kMB / 2;  // 32 x 32 patches per wavefront along r and c
struct BlockExchange {
  char* stage;  // this wavefront's patch
  int lx, lq, rd_row, rd_chunk;
  __device__ __forceinline__ void init(char* lds_after_pipeline, const LanePos& p) {
    stage = lds_after_pipeline + (threadIdx.x >> 6) * 4096;
    lx = p.lx;
    lq = p.lq;
    rd_row = (threadIdx.x & 63) >> 3;
    rd_chunk = threadIdx.x & 7;
  }
  // blk[cb][rb]: the four 16 x 16 blocks of the patch, cb along c, rb along r
  __device__ __forceinline__ void run(const f32x4 (&blk)[2][2], f32x4 (&out)[4]) const {
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const int row = 16 * rb + lx;
        *reinterpret_cast<f32x4*>(stage + row * 128 + (((4 * cb + lq) ^ ((row >> 1) & 7)) << 4)) = blk[cb][rb];
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 8 * i + rd_row;
      out[i] = *reinterpret_cast<const f32x4*>(stage + row * 128 + ((rd_chunk ^ ((row >> 1) & 7)) << 4));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  // the patch (mb2, nb2) of an accumulator
  __device__ __forceinline__ void run(const Accum& acc, int mb2, int nb2, f32x4 (&out)[4]) const {
    const f32x4 blk[2][2] = {{acc.a[2 * mb2][2 * nb2], acc.a[2 * mb2][2 * nb2 + 1]},
                             {acc.a[2 * mb2 + 1][2 * nb2], acc.a[2 * mb2 + 1][2 * nb2 + 1]}};
    run(blk, out);
  }
};

constexpr int kCacheStageBytes = (kThreads / 64) * 4096;  // one 32 x 32 fp32 patch per wavefront
constexpr int kFwdTokenLds = kTile * 4 + kThreads * kNB * 4;  // forward without a cache: labels + label-logit sums

// Per-lane online-softmax state for the kNB token slots (nb) the lane owns.  With CACHE the
// scaled logits of every valid (token, vocabulary column) are also written out in fp32, so the
// backward pass can form d_logits without repeating the GEMM.
// With PI2 a fifth running sum, sum_j e_j^2, is carried, from which sum_j softmax(z)_j^2 follows
// (calculate_sum_pi_squared_from_logits, verl/utils/torch_functional.py:680-694).
template <bool CACHE, bool PI2>
struct FwdEpi {
  LanePos p;
  float scale2;
  int vocab;
  float m[kNB], s[kNB], sy[kNB], s2[kNB];
  // The labels of the lane's token rows and the label-logit sums live in LDS behind the pipeline's stages when the
  // kernel has LDS to spare (no logits cache), in registers otherwise: with them in registers the kernel spilled,
  // and every reload of a spilled value waits out the slab transfers in flight (one counter counts both).
  float zl[CACHE ? kNB : 1];
  int lab[CACHE ? kNB : 1];
  unsigned lab_lds, zl_lds;  // LDS byte addresses: labels [256] by tile row; sums [kThreads][kNB]
  float rcp_t;
  float* z_cache;  // CACHE: [n_tokens][vocab]
  BlockExchange ex;  // CACHE
  int tok0;        // CACHE: first token row of the wavefront
  int n_tokens;

  __device__ __forceinline__ void prefetch(int, int, int) {}
  __device__ __forceinline__ void operator()(Accum& acc, int /*r0*/, int c0) {
    const bool ragged = c0 + kTile > vocab;
    if constexpr (CACHE) {
#pragma unroll
      for (int nb2 = 0; nb2 < kNB2; ++nb2)
#pragma unroll
        for (int mb2 = 0; mb2 < kMB2; ++mb2) {
          f32x4 blk[2][2];
#pragma unroll
          for (int cb = 0; cb < 2; ++cb)
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) blk[cb][rb] = acc.a[2 * mb2 + cb][2 * nb2 + rb] * rcp_t;
          f32x4 out[4];
          ex.run(blk, out);
          const int col = c0 + p.wc * 128 + mb2 * 32 + 4 * ex.rd_chunk;
          if (col < vocab) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int tok = tok0 + nb2 * 32 + 8 * i + ex.rd_row;
              if (tok < n_tokens)
                __builtin_nontemporal_store(out[i], reinterpret_cast<f32x4*>(z_cache + (int64_t)tok * vocab + col));
            }
          }
        }
    }
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      // pass 1: tile maximum of the raw products (the vocabulary tail of the last tile replaced in place)
      float xmax = kNegBig;
      if (ragged) {
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float x = (c0 + acc_col(p, mb, v) < vocab) ? acc.a[mb][nb][v] : kNoColumn;
            acc.a[mb][nb][v] = x;
            xmax = fmaxf(xmax, x);
          }
      } else {
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
          for (int v = 0; v < 4; ++v) xmax = fmaxf(xmax, acc.a[mb][nb][v]);
      }
      // label logit: only when some lane's label falls in this wavefront's 128 columns
      typedef int __attribute__((address_space(3))) * lds_i32_t;
      typedef float __attribute__((address_space(3))) * lds_f32_t;
      int label;
      if constexpr (CACHE) label = lab[nb];
      else label = *(lds_i32_t)(uintptr_t)(lab_lds + 4u * (unsigned)acc_row(p, nb));
      const int rel = label - c0 - p.wc * 128;
      if (__any(rel >= 0 && rel < 128)) {
        float add = 0.f;
#pragma unroll
        for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int col = mb * kBlk + 4 * p.lq + v;
            add += (col == rel) ? acc.a[mb][nb][v] * rcp_t : 0.f;
          }
        if constexpr (CACHE) {
          zl[nb] += add;
        } else {
          const lds_f32_t slot = (lds_f32_t)(uintptr_t)(zl_lds + 4u * (threadIdx.x * kNB + nb));
          *slot += add;
        }
      }
      // pass 2: the running state in the log2 domain, three operations and an exponential per element:
      // e = 2^(x scale2 - m), s += e, sy += e x (the raw product: the 1 / temperature goes on at the very end)
      const float m_new = fmaxf(m[nb], xmax * scale2);
      const float resc = fast_exp2(m[nb] - m_new);
      float s_ = s[nb] * resc, sy_ = sy[nb] * resc, s2_ = PI2 ? s2[nb] * resc * resc : 0.f;
#pragma unroll
      for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float x = acc.a[mb][nb][v];
          const float e = fast_exp2(fmaf(x, scale2, -m_new));
          s_ += e;
          sy_ = fmaf(e, x, sy_);
          if (PI2) s2_ = fmaf(e, e, s2_);
        }
      m[nb] = m_new;
      s[nb] = s_;
      sy[nb] = sy_;
      if (PI2) s2[nb] = s2_;
    }
  }
};

__device__ __forceinline__ void merge_state(float& m, float& s, float& sy, float m2, float s2, float sy2) {
  const float mm = fmaxf(m, m2);
  const float a = fast_exp2(m - mm), b = fast_exp2(m2 - mm);
  s = s * a + s2 * b;
  sy = sy * a + sy2 * b;
  m = mm;
}
// the same with the squared sums q
__device__ __forceinline__ void merge_state(float& m, float& s, float& sy, float& q, float m2, float s2, float sy2,
                                            float q2) {
  const float mm = fmaxf(m, m2);
  const float a = fast_exp2(m - mm), b = fast_exp2(m2 - mm);
  s = s * a + s2 * b;
  sy = sy * a + sy2 * b;
  q = q * a * a + q2 * b * b;
  m = mm;
}

template <bool CACHE, bool PI2>
__global__ __launch_bounds__(kThreads) void lce_forward_kernel(FwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  // workgroup -> (token tile, vocabulary split); bands of 8 token tiles x all splits per XCD
  const int nwg = a.tok_tiles * a.splits;
  const int q = xcd_regroup(blockIdx.x, nwg);
  const int band = 8 * a.splits;
  const int bidx = q / band;
  const int first = bidx * 8;
  const int rows = (a.tok_tiles - first) < 8 ? (a.tok_tiles - first) : 8;
  const int w = q - bidx * band;
  const int tn = first + w % rows;
  const int sp = w / rows;

  SplitSched sched;
  sched.r0_ = tn * kTile;
  sched.vt_begin = (int)(((int64_t)sp * a.voc_tiles) / a.splits);
  sched.vt_count = (int)(((int64_t)(sp + 1) * a.voc_tiles) / a.splits) - sched.vt_begin;

  FwdEpi<CACHE, PI2> epi;
  epi.p = lane_pos();
  epi.scale2 = a.scale2;
  epi.vocab = a.vocab;
  epi.rcp_t = a.rcp_t;
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    epi.m[nb] = kNegBig;
    epi.s[nb] = 0.f;
    epi.sy[nb] = 0.f;
    epi.s2[nb] = 0.f;
    if constexpr (CACHE) {
      epi.zl[nb] = 0.f;
      const int tok = sched.r0_ + acc_row(epi.p, nb);
      epi.lab[nb] = tok < a.n_tokens ? (int)a.labels[tok] : -1;
    }
  }
  if constexpr (!CACHE) {
    typedef float __attribute__((address_space(3))) * lds_f32_t;
    epi.lab_lds = lds_address(lds + kLdsBytes);
    epi.zl_lds = epi.lab_lds + kTile * 4;
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) *(lds_f32_t)(uintptr_t)(epi.zl_lds + 4u * (threadIdx.x * kNB + nb)) = 0.f;
    // the low dwords of the tile's 256 labels, 64 per wavefront of the first four, straight into LDS; a token past
    // the end reads as label 0, whose sums nobody looks at.  The transfers are older than every slab transfer, so
    // the pipeline's first wait and barrier cover them.
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (w < 4) {
      const u32x4 rs = span_rsrc(a.labels, (int64_t)a.n_tokens * 8);
      load_to_lds_4(rs, ((unsigned)sched.r0_ + 64u * w + (threadIdx.x & 63u)) * 8u, epi.lab_lds + 64u * w * 4u);
    }
  }
  epi.z_cache = a.z_cache;
  epi.ex.init(lds + kLdsBytes, epi.p);
  epi.tok0 = sched.r0_ + epi.p.wr * (kNB * kBlk);
  epi.n_tokens = a.n_tokens;

  run_tiles<false, false>(a.hidden, a.weight, a.k_slabs, sched, epi, lds);

  float zl[kNB];
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    typedef float __attribute__((address_space(3))) * lds_f32_t;
    if constexpr (CACHE) zl[nb] = epi.zl[nb];
    else zl[nb] = *(lds_f32_t)(uintptr_t)(epi.zl_lds + 4u * (threadIdx.x * kNB + nb));
  }
  // merge the four lane quarters (they hold disjoint vocabulary columns of the same token) ...
#pragma unroll
  for (int step = 16; step <= 32; step *= 2)
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      const float m2 = __shfl_xor(epi.m[nb], step, 64);
      const float s2 = __shfl_xor(epi.s[nb], step, 64);
      const float sy2 = __shfl_xor(epi.sy[nb], step, 64);
      const float z2 = __shfl_xor(zl[nb], step, 64);
      if (PI2) {
        const float q2 = __shfl_xor(epi.s2[nb], step, 64);
        merge_state(epi.m[nb], epi.s[nb], epi.sy[nb], epi.s2[nb], m2, s2, sy2, q2);
      } else {
        merge_state(epi.m[nb], epi.s[nb], epi.sy[nb], m2, s2, sy2);
      }
      zl[nb] += z2;
    }
  // ... then the two wavefronts that share a token quarter (wc = 0/1), through LDS (once every
  // wavefront's last slab transfers have landed).
  __syncthreads();
  float4* red = reinterpret_cast<float4*>(lds);                     // [2][256]
  float* redq = reinterpret_cast<float*>(lds + 2 * kTile * 16);    // [2][256] squared sums
  if (epi.p.lq == 0) {
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      red[epi.p.wc * kTile + acc_row(epi.p, nb)] = make_float4(epi.m[nb], epi.s[nb], epi.sy[nb], zl[nb]);
      if (PI2) redq[epi.p.wc * kTile + acc_row(epi.p, nb)] = epi.s2[nb];
    }
  }
  __syncthreads();
  if (threadIdx.x < kTile) {
    const int t = threadIdx.x;
    float4 x = red[t], y = red[kTile + t];
    const int64_t slot = (int64_t)sp * a.tok_tiles * kTile + tn * kTile + t;
    if (PI2) {
      float q = redq[t];
      merge_state(x.x, x.y, x.z, q, y.x, y.y, y.z, redq[kTile + t]);
      a.pi2_partials[slot] = q;
    } else {
      merge_state(x.x, x.y, x.z, y.x, y.y, y.z);
    }
    x.w += y.w;
    a.partials[slot] = x;
  }
}

struct MergeArgs {
  const float4* partials;
  const float* pi2_partials;  // null unless sum_pi_squared is wanted
  int splits, stride, n_tokens;
  float rcp_t;  // the partial sums of e * (hidden . weight) carry no 1 / temperature yet
  float* logprobs;
  float* entropy;
  float* lse;
  float* mean_z;
  float* sum_pi_squared;
};

__global__ __launch_bounds__(256) void lce_merge_kernel(MergeArgs a) {
  const int tok = blockIdx.x * 256 + threadIdx.x;
  if (tok >= a.n_tokens) return;
  float m = kNegBig, s = 0.f, sy = 0.f, zl = 0.f, q = 0.f;
  for (int sp = 0; sp < a.splits; ++sp) {
    const float4 x = a.partials[(int64_t)sp * a.stride + tok];
    if (a.pi2_partials) merge_state(m, s, sy, q, x.x, x.y, x.z, a.pi2_partials[(int64_t)sp * a.stride + tok]);
    else merge_state(m, s, sy, x.x, x.y, x.z);
    zl += x.w;
  }
  if (a.pi2_partials) a.sum_pi_squared[tok] = q / (s * s);
  const float lse = (m + log2f(s)) * kLn2;
  const float mz = (sy / s) * a.rcp_t;
  a.lse[tok] = lse;
  a.mean_z[tok] = mz;
  a.entropy[tok] = lse - mz;
  a.logprobs[tok] = zl - lse;
}

// =============================================================================================
// Backward
// =============================================================================================
__device__ __forceinline__ u32x2 pack_bf16x4(float a, float b, float c, float d) {
  bf16x4 o;
  o[0] = (__bf16)a;
  o[1] = (__bf16)b;
  o[2] = (__bf16)c;
  o[3] = (__bf16)d;
  return __builtin_bit_cast(u32x2, o);
}

__device__ __forceinline__ float bf16_bits_to_float(unsigned h) { return __uint_as_float(h << 16); }

struct RecomputeArgs {
  Operand hidden;  // R: [n_tokens][H]
  Operand weight;  // C: rows of this vocabulary chunk, x_extent = vocab - chunk_c0
  const int64_t* labels;
  const float* lse;
  const float* mean_z;
  const float* g_lp;   // may be null
  const float* g_ent;  // may be null -> g_ent_scalar
  float g_ent_scalar;
  int n_tokens, vocab_left;  // vocab_left = vocab - chunk_c0
  int chunk_c0;
  int k_slabs, tok_tiles, chunk_tiles;
  float scale2, rcp_t;
  uint16_t* dz;  // [tok_tiles*256][dz_ld] bf16
  int dz_ld;
};

// The same hand-over for a bf16 result: the wavefront's patch holds 32 rows x 32 columns of bf16 (2 KB), rounded
// before the exchange, so the LDS traffic is half that of the fp32 patch and the global stores are 16 bytes per
// lane: a store instruction covers 16 rows x 64 bytes.  16-byte chunk c of row r lives at position c ^ ((r >> 2) & 3)
// so that the 8-byte writes of 16 rows at one column spread over the banks.  After the exchange lane L holds columns
// 8 (L % 4) .. + 7 of rows 16 i + L / 4 (i = 0, 1).
struct BlockExchangeBf16 {
  char* stage;
  int lx, lq, rd_row, rd_chunk;
  __device__ __forceinline__ void init(char* area, const LanePos& p) {
    stage = area + (threadIdx.x >> 6) * 2048;
    lx = p.lx;
    lq = p.lq;
    rd_row = (threadIdx.x & 63) >> 2;
    rd_chunk = threadIdx.x & 3;
  }
  __device__ __forceinline__ void run(const f32x4 (&blk)[2][2], u32x4 (&out)[2]) const {
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const int row = 16 * rb + lx;
        const int chunk = (2 * cb + (lq >> 1)) ^ ((row >> 2) & 3);
        *reinterpret_cast<u32x2*>(stage + row * 64 + chunk * 16 + (lq & 1) * 8) =
            pack_bf16x4(blk[cb][rb][0], blk[cb][rb][1], blk[cb][rb][2], blk[cb][rb][3]);
      }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = 16 * i + rd_row;
      out[i] = *reinterpret_cast<const u32x4*>(stage + row * 64 + ((rd_chunk ^ ((row >> 2) & 3)) << 4));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
};
constexpr int kBf16StageBytes = (kThreads / 64) * 2048;  // one 32 x 32 bf16 patch per wavefront

// Per-token inputs of the d_logits epilogue (lse, mean_z, g_lp, label, g_ent) for the 256 tokens of a tile, staged
// in LDS by memory -> LDS transfers issued when the tile's first slab starts (prefetch): five arrays of 256 dwords,
// two sets used in turn so that a tile's transfers never land in what the previous tile's epilogue still reads.
constexpr int kTokArrays = 5, kTokSetBytes = kTokArrays * kTile * 4;
constexpr int kRecomputeExtraLds = kBf16StageBytes + 2 * kTokSetBytes;
static_assert(kRecomputeExtraLds <= kCacheStageBytes, "the recompute kernel is launched with the cache stage's LDS");

struct RecomputeEpi {
  LanePos p;
  const RecomputeArgs* a;
  BlockExchangeBf16 ex;
  char* tok_stage;  // [2][kTokArrays][256] dwords
  int parity;       // set of the tile whose epilogue runs next

  __device__ __forceinline__ void init(char* lds_after_pipeline, const LanePos& pos, const RecomputeArgs* args) {
    p = pos;
    a = args;
    ex.init(lds_after_pipeline, pos);
    tok_stage = lds_after_pipeline + kBf16StageBytes;
    parity = 0;
  }

  // wavefront w brings in half (w & 1) of array (w >> 1): 0 lse, 1 mean_z, 2 g_lp, 3 labels (low dwords); the
  // wavefronts 0 and 1 also bring in g_ent when it is a tensor
  __device__ __forceinline__ void prefetch(int tile, int r0, int /*c0*/) {
    const RecomputeArgs& A = *a;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const unsigned lane = threadIdx.x & 63u;
    const int arr = w >> 1, half = w & 1;
    const unsigned set_lds = lds_address(tok_stage) + (unsigned)(tile & 1) * kTokSetBytes;
    const void* src = arr == 0 ? (const void*)A.lse : arr == 1 ? (const void*)A.mean_z
                      : arr == 2 ? (const void*)A.g_lp : (const void*)A.labels;
    const unsigned elt = arr == 3 ? 8u : 4u;
    if (src) {  // uniform over the wavefront
      const u32x4 rs = span_rsrc(src, (int64_t)A.n_tokens * elt);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const unsigned tok = (unsigned)r0 + half * 128u + i * 64u + lane;
        load_to_lds_4(rs, tok * elt, set_lds + arr * (kTile * 4) + (half * 128u + i * 64u) * 4u);
      }
    }
    if (A.g_ent && w < 2) {
      const u32x4 rs = span_rsrc(A.g_ent, (int64_t)A.n_tokens * 4);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const unsigned tok = (unsigned)r0 + half * 128u + i * 64u + lane;
        load_to_lds_4(rs, tok * 4u, set_lds + 4 * (kTile * 4) + (half * 128u + i * 64u) * 4u);
      }
    }
  }

  // d_logits of the two token rows (rb) x 128 columns the lane holds of 32-row patch nb2, rounded, handed over and
  // stored.  PLAIN: a tile inside the matrix with no label in the wavefront's 128 columns -- nothing but the
  // arithmetic, four multiply-adds and an exponential per element; otherwise the one-hot term and the zeros for
  // padding rows and columns come in through two comparisons per element (no branches).
  //   code[rb]: 4 mb + v of the element of row rb that holds the label's column, or -1
  //   lim[rb] : columns of the wavefront's 128 that exist for row rb (0 for a padding row), minus 4 lq
  template <bool PLAIN>
  __device__ __forceinline__ void patch_rows(Accum& acc, int nb2, int r0, int c0, const float (&lse2)[2],
                                             const float (&u1)[2], const float (&u0)[2], const float (&glp)[2],
                                             const int (&code)[2], const int (&lim)[2]) {
    const RecomputeArgs& A = *a;
#pragma unroll
    for (int mb2 = 0; mb2 < kMB2; ++mb2) {
      f32x4 d[2][2];
#pragma unroll
      for (int cb = 0; cb < 2; ++cb)
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int mb = 2 * mb2 + cb;
            const float x = acc.a[mb][2 * nb2 + rb][v];
            const float prob = fast_exp2(fmaf(x, A.scale2, -lse2[rb]));
            const float u = fmaf(u1[rb], x, u0[rb]);  // g_lp/T + g_ent/T * (z - mean_z), z = x / T
            if constexpr (PLAIN) {
              d[cb][rb][v] = -prob * u;
            } else {
              const float onehot = code[rb] == 4 * mb + v ? glp[rb] : 0.f;
              const float dzv = fmaf(-prob, u, onehot);
              d[cb][rb][v] = (mb * kBlk + v) < lim[rb] ? dzv : 0.f;  // every row of the panel is written, padding as zeros
            }
          }
      u32x4 o[2];
      ex.run(d, o);
      const int col0 = c0 + p.wc * 128 + mb2 * 32 + 8 * ex.rd_chunk;
      const int64_t row0 = r0 + p.wr * (kNB * kBlk) + nb2 * 32 + ex.rd_row;
#pragma unroll
      for (int i = 0; i < 2; ++i) *reinterpret_cast<u32x4*>(A.dz + (row0 + 16 * i) * A.dz_ld + col0) = o[i];
    }
  }

  __device__ __forceinline__ void operator()(Accum& acc, int r0, int c0) {
    const RecomputeArgs& A = *a;
    // read through LDS-typed pointers: as generic pointers some of these became flat loads, whose wait also
    // waits out every slab transfer in flight
    typedef const float __attribute__((address_space(3))) * lds_f32_t;
    typedef const int __attribute__((address_space(3))) * lds_i32_t;
    const lds_f32_t tokf = (lds_f32_t)(uintptr_t)(lds_address(tok_stage) + (unsigned)parity * kTokSetBytes);
    const lds_i32_t toki = (lds_i32_t)tokf;
    parity ^= 1;
    const bool inside = r0 + kTile <= A.n_tokens && c0 + kTile <= A.vocab_left;  // uniform over the workgroup
    const int cols_left = A.vocab_left - c0 - p.wc * 128 - 4 * p.lq;
#pragma unroll
    for (int nb2 = 0; nb2 < kNB2; ++nb2) {
      // the lane's two token rows of this 32-row patch
      // u = u1 x + u0 with u1 = g_ent / T^2 and u0 = g_lp / T - g_ent / T * mean_z: one multiply-add per element
      float lse2[2], u1[2], u0[2], glp[2];
      int code[2], lim[2];
      bool hit = false;
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const int t = acc_row(p, 2 * nb2 + rb);  // row inside the tile
        lse2[rb] = tokf[t] * kLog2e;
        glp[rb] = (A.g_lp ? tokf[2 * kTile + t] : 0.f) * A.rcp_t;
        const float gent = (A.g_ent ? tokf[4 * kTile + t] : A.g_ent_scalar) * A.rcp_t;
        u1[rb] = gent * A.rcp_t;
        u0[rb] = fmaf(-gent, tokf[kTile + t], glp[rb]);
        const int rel = toki[3 * kTile + t] - A.chunk_c0 - c0 - p.wc * 128;  // label's column among the wavefront's 128
        const bool here = rel >= 0 && rel < 128;
        hit = hit || here;
        // the lane holds columns 16 mb + 4 lq + v: the label's is one of them when its 4-column group is lq
        code[rb] = (here && ((rel >> 2) & 3) == p.lq) ? 4 * (rel >> 4) + (rel & 3) : -1;
        lim[rb] = r0 + t < A.n_tokens ? cols_left : 0;
      }
      if (inside && !__any(hit)) patch_rows<true>(acc, nb2, r0, c0, lse2, u1, u0, glp, code, lim);
      else patch_rows<false>(acc, nb2, r0, c0, lse2, u1, u0, glp, code, lim);
    }
  }
};

__global__ __launch_bounds__(kThreads) void lce_recompute_kernel(RecomputeArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  GroupedSched sched;
  sched.r_tiles = a.tok_tiles;
  sched.c_tiles = a.chunk_tiles;
  sched.nwg = gridDim.x;
  sched.wg = xcd_regroup(blockIdx.x, gridDim.x);
  RecomputeEpi epi;
  epi.init(lds + kLdsBytes, lane_pos(), &a);
  run_tiles<false, false>(a.hidden, a.weight, a.k_slabs, sched, epi, lds);
}

// d_logits panel of one vocabulary chunk from cached logits: the same arithmetic as RecomputeEpi,
// one thread per 8 consecutive columns of a token, 2048 columns per workgroup.
struct DLogitsArgs {
  const float* z_cache;  // [n_tokens][vocab]
  const int64_t* labels;
  const float* lse;
  const float* mean_z;
  const float* g_lp;
  const float* g_ent;
  float g_ent_scalar, rcp_t;
  int n_tokens, vocab, chunk_c0, chunk_cols;  // chunk_cols: panel columns to fill (multiple of 256)
  uint16_t* dz;
  int dz_ld;
};

__global__ __launch_bounds__(256) void lce_dlogits_kernel(DLogitsArgs a) {
  const int tok = blockIdx.x;
  const int j = (blockIdx.y * 256 + threadIdx.x) * 8;  // column inside the chunk
  if (j >= a.chunk_cols) return;
  u32x4 out = {0u, 0u, 0u, 0u};
  const int col = a.chunk_c0 + j;
  if (tok < a.n_tokens && col < a.vocab) {  // vocab % 8 == 0: the 8 columns are all in or all out
    const float lse2 = a.lse[tok] * kLog2e;
    const float glp = (a.g_lp ? a.g_lp[tok] : 0.f) * a.rcp_t;
    const float gent = (a.g_ent ? a.g_ent[tok] : a.g_ent_scalar) * a.rcp_t;
    const float u0 = fmaf(-gent, a.mean_z[tok], glp);  // as in the recompute epilogue, with z in place of x / T
    const int rel = (int)a.labels[tok] - col;
    const f32x4* src = reinterpret_cast<const f32x4*>(a.z_cache + (int64_t)tok * a.vocab + col);
    const f32x4 z0 = __builtin_nontemporal_load(src), z1 = __builtin_nontemporal_load(src + 1);
    float d[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float z = e < 4 ? z0[e] : z1[e - 4];
      const float prob = fast_exp2(fmaf(z, kLog2e, -lse2));
      const float u = fmaf(gent, z, u0);
      d[e] = fmaf(-prob, u, (e == rel) ? glp : 0.f);
    }
    const u32x2 lo = pack_bf16x4(d[0], d[1], d[2], d[3]), hi = pack_bf16x4(d[4], d[5], d[6], d[7]);
    out = u32x4{lo[0], lo[1], hi[0], hi[1]};
  }
  *reinterpret_cast<u32x4*>(a.dz + (int64_t)tok * a.dz_ld + j) = out;
}

// ---------------------------------------------------------------------------------------------
// d_hidden (+)= dz_panel . W[chunk]          R = dz (direct), C = W (kmajor, k = vocab)
// d_weight[chunk] (+)= dz_panel^T . hidden    R = dz (kmajor, k = token), C = hidden (kmajor)
enum : int { kStoreF32 = 0, kAddF32 = 1, kFinalBf16 = 2, kFinalBf16AddPrev = 3 };

struct GemmOutArgs {
  Operand R, C;
  int k_slabs, r_tiles, c_tiles;
  int r_valid, c_valid;  // rows / cols of the output that exist
  int mode;              // d_hidden: one of the enum above; d_weight: a VAMD_DW_* value
  float* acc32;          // fp32 accumulator [r_valid][ld_out]
  uint16_t* out;         // bf16 output
  int64_t ld_out;
};

struct DHiddenEpi {
  LanePos p;
  const GemmOutArgs* a;
  BlockExchange ex;
  __device__ __forceinline__ void prefetch(int, int, int) {}
  __device__ __forceinline__ void operator()(Accum& acc, int r0, int c0) {
    const GemmOutArgs& A = *a;
    const bool read_prev = A.mode == kAddF32 || A.mode == kFinalBf16AddPrev;
    const bool to_f32 = A.mode == kStoreF32 || A.mode == kAddF32;
#pragma unroll
    for (int nb = 0; nb < kNB2; ++nb)
#pragma unroll
      for (int mb = 0; mb < kMB2; ++mb) {
        f32x4 v[4];
        ex.run(acc, mb, nb, v);
        const int col = c0 + p.wc * 128 + mb * 32 + 4 * ex.rd_chunk;
        if (col >= A.c_valid) continue;
        const int row0 = r0 + p.wr * (kNB * kBlk) + nb * 32 + ex.rd_row;
        f32x4 prev[4];
        if (read_prev) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            prev[i] = (row0 + 8 * i < A.r_valid)
                          ? *reinterpret_cast<const f32x4*>(A.acc32 + (int64_t)(row0 + 8 * i) * A.ld_out + col)
                          : f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = row0 + 8 * i;
          if (row >= A.r_valid) continue;
          f32x4 x = v[i];
          if (read_prev) x = x + prev[i];
          const int64_t off = (int64_t)row * A.ld_out + col;
          if (to_f32) *reinterpret_cast<f32x4*>(A.acc32 + off) = x;
          else *reinterpret_cast<u32x2*>(A.out + off) = pack_bf16x4(x[0], x[1], x[2], x[3]);
        }
      }
  }
};

struct DWeightEpi {
  LanePos p;
  const GemmOutArgs* a;
  BlockExchange ex;
  __device__ __forceinline__ void prefetch(int, int, int) {}
  __device__ __forceinline__ void operator()(Accum& acc, int r0, int c0) {
    const GemmOutArgs& A = *a;
#pragma unroll
    for (int nb = 0; nb < kNB2; ++nb)
#pragma unroll
      for (int mb = 0; mb < kMB2; ++mb) {
        f32x4 v[4];
        ex.run(acc, mb, nb, v);
        const int col = c0 + p.wc * 128 + mb * 32 + 4 * ex.rd_chunk;
        if (col >= A.c_valid) continue;
        const int row0 = r0 + p.wr * (kNB * kBlk) + nb * 32 + ex.rd_row;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = row0 + 8 * i;
          if (row >= A.r_valid) continue;
          f32x4 x = v[i];
          const int64_t off = (int64_t)row * A.ld_out + col;
          u32x2* dst = reinterpret_cast<u32x2*>(A.out + off);
          if (A.mode == VAMD_DW_ADD_BF16) {
            const u32x2 o = *dst;
            x[0] += bf16_bits_to_float(o[0] & 0xffffu);
            x[1] += bf16_bits_to_float(o[0] >> 16);
            x[2] += bf16_bits_to_float(o[1] & 0xffffu);
            x[3] += bf16_bits_to_float(o[1] >> 16);
          } else if (A.mode >= VAMD_DW_F32_STORE) {
            f32x4* acc = reinterpret_cast<f32x4*>(A.acc32 + off);
            if (A.mode != VAMD_DW_F32_STORE) x = x + *acc;
            *acc = x;
            if (A.mode != VAMD_DW_F32_ADD_FINISH) continue;
          }
          *dst = pack_bf16x4(x[0], x[1], x[2], x[3]);
        }
      }
  }
};

// Both gradient GEMMs of one vocabulary chunk in a single launch: a workgroup first walks its
// share of the d_hidden tiles, then its share of the d_weight tiles.  The second walk starts at
// the workgroup after the last one that received an extra tile in the first, so the combined
// tile count, not each GEMM's, decides how full the last round is (896 + 896 tiles on 256 CUs:
// 7 full rounds instead of 2 x 3.5).
__global__ __launch_bounds__(kThreads) void lce_dgrad_kernel(GemmOutArgs gh, GemmOutArgs gw) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int nwg = gridDim.x;
  const int wg = xcd_regroup(blockIdx.x, nwg);
  const LanePos pos = lane_pos();
  {
    GroupedSched sched;
    sched.r_tiles = gh.r_tiles;
    sched.c_tiles = gh.c_tiles;
    sched.nwg = nwg;
    sched.wg = wg;
    DHiddenEpi epi;
    epi.p = pos;
    epi.a = &gh;
    epi.ex.init(lds + kLdsBytes, pos);
    run_tiles<false, true>(gh.R, gh.C, gh.k_slabs, sched, epi, lds);
  }
  __syncthreads();
  {
    const int rem = (gh.r_tiles * gh.c_tiles) % nwg;
    GroupedSched sched;
    sched.r_tiles = gw.r_tiles;
    sched.c_tiles = gw.c_tiles;
    sched.nwg = nwg;
    sched.wg = (wg - rem + nwg) % nwg;
    DWeightEpi epi;
    epi.p = pos;
    epi.a = &gw;
    epi.ex.init(lds + kLdsBytes, pos);
    run_tiles<true, true>(gw.R, gw.C, gw.k_slabs, sched, epi, lds);
  }
}

// =============================================================================================
// Host side
// =============================================================================================
template <class K>
static int allow_big_lds(K kernel, int bytes = kLdsBytes) {
  VAMD_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               bytes));
  return VAMD_OK;
}

// The kernels use more LDS than the default launch limit; the limit is a per-device function
// attribute, so it is raised once on every device the library is used on.
static int ensure_lds_attributes() {
  static std::mutex mu;
  static bool done[64];
  int dev = 0;
  VAMD_HIP(hipGetDevice(&dev));
  VAMD_REQUIRE(dev >= 0 && dev < 64, "lce: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (done[dev]) return VAMD_OK;
  int s;
  if ((s = allow_big_lds(lce_forward_kernel<false, false>, kLdsBytes + kFwdTokenLds)) != VAMD_OK) return s;
  if ((s = allow_big_lds(lce_forward_kernel<false, true>, kLdsBytes + kFwdTokenLds)) != VAMD_OK) return s;
  if ((s = allow_big_lds(lce_forward_kernel<true, false>, kLdsBytes + kCacheStageBytes)) != VAMD_OK) return s;
  if ((s = allow_big_lds(lce_forward_kernel<true, true>, kLdsBytes + kCacheStageBytes)) != VAMD_OK) return s;
  if ((s = allow_big_lds(lce_recompute_kernel, kLdsBytes + kCacheStageBytes)) != VAMD_OK) return s;
  if ((s = allow_big_lds(lce_dgrad_kernel, kLdsBytes + kCacheStageBytes)) != VAMD_OK) return s;
  done[dev] = true;
  return VAMD_OK;
}

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Row pitch of the staged d_logits panel: the chunk width plus 256 bytes, so that the rows a
// wavefront touches together (32 .. 64 consecutive tokens at one column) spread over the memory
// channels instead of landing on a power-of-two stride.
static inline int64_t dz_pitch(int64_t cv) { return cv + 128; }

// max_rows: most partial-state rows (splits x padded tokens) the caller's buffer holds; the built-in buffer of the
// entry point that allocates nothing is sized for 256 CUs and must serve a part with more of them too.
static int fwd_splits(int64_t tok_tiles, int64_t voc_tiles, int64_t max_rows = INT64_MAX) {
  const int cus = device_cu_count();
  int64_t sp = cus / tok_tiles;  // as many workgroups as fit in one round over the CUs
  if (sp > max_rows / (tok_tiles * kTile)) sp = max_rows / (tok_tiles * kTile);
  if (sp < 1) sp = 1;
  if (sp > voc_tiles) sp = voc_tiles;
  return (int)sp;
}

// Any vocabulary size is served; only the fp32 logits cache, whose rows are read and written 32 bytes at a time,
// needs a multiple of 8.
static int check_head_shapes(int64_t n, int64_t h, int64_t v, const void* logits_cache) {
  VAMD_REQUIRE(n > 0 && h > 0 && v > 0, "lce: empty problem n=%lld h=%lld v=%lld", (long long)n, (long long)h,
               (long long)v);
  VAMD_REQUIRE(h % 128 == 0, "lce: hidden_size %lld must be a multiple of 128", (long long)h);
  VAMD_REQUIRE(!logits_cache || v % 8 == 0, "lce: a logits cache needs a vocab that is a multiple of 8, got %lld",
               (long long)v);
  VAMD_REQUIRE(n < (1ll << 30) && v < (1ll << 30), "lce: n_tokens / vocab too large");
  VAMD_REQUIRE(reinterpret_cast<uintptr_t>(logits_cache) % 16 == 0, "lce: logits_cache must be 16-byte aligned");
  return VAMD_OK;
}

static int64_t default_vocab_chunk(int64_t n_tokens, int64_t hidden_size, int64_t vocab, int64_t requested) {
  const int64_t n_pad = ceil_div(n_tokens, kTile) * kTile;
  const int64_t v_pad = ceil_div(vocab, kTile) * kTile;
  int64_t cv = requested;
  if (cv <= 0) {
    int64_t budget = 512ll << 20;  // bytes of bf16 d_logits staged at a time
    if (const char* e = getenv("VAMD_LCE_DZ_BUDGET_MB")) {
      const long mb = strtol(e, nullptr, 10);
      if (mb > 0) budget = (int64_t)mb << 20;
    }
    cv = budget / (n_pad * 2) / kTile * kTile;
  }
  cv = ceil_div(cv, kTile) * kTile;
  // the weight rows of a chunk are walked with 32-bit byte offsets from the chunk's first row
  const int64_t cap = ((1ll << 32) - 1) / (hidden_size * 2) / kTile * kTile;
  if (cv > cap) cv = cap;
  if (cv < kTile) cv = kTile;
  if (cv > v_pad) cv = v_pad;
  return cv;
}

}  // namespace vamd

using namespace vamd;

extern "C" int vamd_lce_timing_enable(int on) {
  g_timing_on.store(on != 0);
  return VAMD_OK;
}

extern "C" int vamd_lce_timing_collect(double* ms_by_kernel, int64_t* launches_by_kernel) {
  VAMD_REQUIRE(ms_by_kernel && launches_by_kernel, "timing_collect: null pointer");
  for (int i = 0; i < kNumTags; ++i) {
    ms_by_kernel[i] = 0;
    launches_by_kernel[i] = 0;
  }
  int status = VAMD_OK;
  std::lock_guard<std::mutex> lock(g_timed_mu);
  for (TimedLaunch& t : g_timed) {
    float ms = 0.f;
    if (hipEventSynchronize(t.stop) != hipSuccess || hipEventElapsedTime(&ms, t.start, t.stop) != hipSuccess) {
      set_error("timing_collect: event query failed");
      status = VAMD_EHIP;
    } else {
      ms_by_kernel[t.tag] += ms;
      launches_by_kernel[t.tag] += 1;
    }
    (void)hipEventDestroy(t.start);
    (void)hipEventDestroy(t.stop);
  }
  g_timed.clear();
  return status;
}

extern "C" size_t vamd_lce_forward_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab) {
  (void)hidden_size;
  if (n_tokens <= 0 || vocab <= 0) return 0;
  const int64_t tok_tiles = ceil_div(n_tokens, kTile), voc_tiles = ceil_div(vocab, kTile);
  const int sp = fwd_splits(tok_tiles, voc_tiles);
  return align_up((size_t)sp * tok_tiles * kTile * sizeof(float4), 256) +
         align_up((size_t)sp * tok_tiles * kTile * sizeof(float), 256);  // state + squared sums
}

// Forward launches shared by the two entry points; `workspace` holds at least
// vamd_lce_forward_workspace_bytes() bytes and the arguments have been checked.
static int lce_forward_launch(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                              int64_t hidden_size, int64_t vocab, float rcp_temperature, float* logprobs,
                              float* entropy, float* lse, float* mean_z, float* logits_cache, float* sum_pi_squared,
                              void* workspace, void* stream, int64_t max_rows = INT64_MAX) {

  FwdArgs a;
  a.hidden = Operand{static_cast<const uint16_t*>(hidden), hidden_size, (int)n_tokens, (int)hidden_size};
  a.weight = Operand{static_cast<const uint16_t*>(weight), hidden_size, (int)vocab, (int)hidden_size};
  a.labels = labels;
  a.n_tokens = (int)n_tokens;
  a.vocab = (int)vocab;
  a.k_slabs = (int)(hidden_size / kBK);
  a.tok_tiles = (int)ceil_div(n_tokens, kTile);
  a.voc_tiles = (int)ceil_div(vocab, kTile);
  a.splits = fwd_splits(a.tok_tiles, a.voc_tiles, max_rows);
  a.scale2 = rcp_temperature * kLog2e;
  a.rcp_t = rcp_temperature;
  a.partials = static_cast<float4*>(workspace);
  a.pi2_partials = sum_pi_squared
                       ? reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                                  align_up((size_t)a.splits * a.tok_tiles * kTile * sizeof(float4), 256))
                       : nullptr;
  a.z_cache = logits_cache;
  hipStream_t s = static_cast<hipStream_t>(stream);
  {
    ScopedTiming tm(kTagForward, s);
    const dim3 grid(a.tok_tiles * a.splits), block(kThreads);
    if (logits_cache) {
      if (sum_pi_squared)
        hipLaunchKernelGGL((lce_forward_kernel<true, true>), grid, block, kLdsBytes + kCacheStageBytes, s, a);
      else
        hipLaunchKernelGGL((lce_forward_kernel<true, false>), grid, block, kLdsBytes + kCacheStageBytes, s, a);
    } else {
      if (sum_pi_squared)
        hipLaunchKernelGGL((lce_forward_kernel<false, true>), grid, block, kLdsBytes + kFwdTokenLds, s, a);
      else
        hipLaunchKernelGGL((lce_forward_kernel<false, false>), grid, block, kLdsBytes + kFwdTokenLds, s, a);
    }
  }
  VAMD_LAUNCH_CHECK();

  MergeArgs m;
  m.partials = a.partials;
  m.pi2_partials = a.pi2_partials;
  m.sum_pi_squared = sum_pi_squared;
  m.splits = a.splits;
  m.stride = a.tok_tiles * kTile;
  m.n_tokens = (int)n_tokens;
  m.rcp_t = rcp_temperature;
  m.logprobs = logprobs;
  m.entropy = entropy;
  m.lse = lse;
  m.mean_z = mean_z;
  {
    ScopedTiming tm(kTagMerge, s);
    hipLaunchKernelGGL(lce_merge_kernel, dim3((unsigned)ceil_div(n_tokens, 256)), dim3(256), 0, s, m);
  }
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

static int check_forward_args(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                              int64_t hidden_size, int64_t vocab, float rcp_temperature, const float* logprobs,
                              const float* entropy, const float* lse, const float* mean_z, const float* logits_cache) {
  int st = check_head_shapes(n_tokens, hidden_size, vocab, logits_cache);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(hidden && weight && labels && logprobs && entropy && lse && mean_z, "lce_forward: null pointer");
  VAMD_REQUIRE(rcp_temperature > 0.f, "lce_forward: temperature must be positive");
  return VAMD_OK;
}

extern "C" int vamd_lce_forward(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                                int64_t hidden_size, int64_t vocab, float rcp_temperature, float* logprobs,
                                float* entropy, float* lse, float* mean_z, float* logits_cache,
                                float* sum_pi_squared, void* workspace, size_t workspace_bytes, void* stream) {
  int st = check_forward_args(hidden, weight, labels, n_tokens, hidden_size, vocab, rcp_temperature, logprobs, entropy,
                              lse, mean_z, logits_cache);
  if (st != VAMD_OK) return st;
  const size_t need = vamd_lce_forward_workspace_bytes(n_tokens, hidden_size, vocab);
  if (!workspace || workspace_bytes < need) {
    set_error("lce_forward: workspace %zu bytes, need %zu", workspace_bytes, need);
    return VAMD_EWORKSPACE;
  }
  if ((st = ensure_lds_attributes()) != VAMD_OK) return st;
  return lce_forward_launch(hidden, weight, labels, n_tokens, hidden_size, vocab, rcp_temperature, logprobs, entropy,
                            lse, mean_z, logits_cache, sum_pi_squared, workspace, stream);
}

// ---------------------------------------------------------------------------------------------
// The forward pass for callers that cannot allocate: the per-(token tile, vocabulary split)
// softmax partials live in a file-scope device array instead of a caller workspace.  Every GPU
// holds its own copy of the array at its own address; the address is looked up once per device.
// The array's name is only a host-side handle for that lookup: launches and copies use the
// looked-up pointer.
namespace vamd {
constexpr size_t kStaticScratchBytes = (size_t)VAMD_LCE_STATIC_MAX_TOKENS * (sizeof(float4) + sizeof(float)) + 512;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static int static_scratch_pointer(void** out) {
  static std::mutex mu;
  static void* ptr_by_device[64];
  int dev = 0;
  VAMD_HIP(hipGetDevice(&dev));
  VAMD_REQUIRE(dev >= 0 && dev < 64, "lce: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr_by_device[dev]) {
    void* p = nullptr;
    VAMD_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    VAMD_REQUIRE(p != nullptr, "lce: the static scratch array has no device address");
    ptr_by_device[dev] = p;
  }
  *out = ptr_by_device[dev];
  return VAMD_OK;
}
}  // namespace vamd

extern "C" int vamd_lce_forward_static(const void* hidden, const void* weight, const int64_t* labels,
                                       int64_t n_tokens, int64_t hidden_size, int64_t vocab, float rcp_temperature,
                                       float* logprobs, float* entropy, float* lse, float* mean_z,
                                       float* sum_pi_squared, void* stream) {
  int st = check_forward_args(hidden, weight, labels, n_tokens, hidden_size, vocab, rcp_temperature, logprobs, entropy,
                              lse, mean_z, nullptr);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(n_tokens <= VAMD_LCE_STATIC_MAX_TOKENS,
               "lce_forward_static: %lld tokens; the built-in buffer serves at most %d tokens per call: use "
               "vamd_lce_forward with a caller workspace",
               (long long)n_tokens, (int)VAMD_LCE_STATIC_MAX_TOKENS);
  if ((st = ensure_lds_attributes()) != VAMD_OK) return st;
  void* ws = nullptr;
  if ((st = static_scratch_pointer(&ws)) != VAMD_OK) return st;
  // Every partial the merge kernel reads is written by the forward kernel of the same call, so
  // nothing in the buffer has to start at zero and a previous call's contents do not matter.
  // the vocabulary splits are capped so that splits x padded tokens fits the buffer whatever the CU count
  return lce_forward_launch(hidden, weight, labels, n_tokens, hidden_size, vocab, rcp_temperature, logprobs, entropy,
                            lse, mean_z, nullptr, sum_pi_squared, ws, stream, VAMD_LCE_STATIC_MAX_TOKENS);
}

extern "C" size_t vamd_lce_backward_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab,
                                                    int64_t vocab_chunk) {
  if (n_tokens <= 0 || vocab <= 0 || hidden_size <= 0) return 0;
  const int64_t n_pad = ceil_div(n_tokens, kTile) * kTile;
  const int64_t cv = default_vocab_chunk(n_tokens, hidden_size, vocab, vocab_chunk);
  size_t bytes = align_up((size_t)n_pad * dz_pitch(cv) * 2, 256);
  if (cv < ceil_div(vocab, kTile) * kTile) bytes += align_up((size_t)n_tokens * hidden_size * 4, 256);
  return bytes;
}

extern "C" int vamd_lce_backward(const void* hidden, const void* weight, const int64_t* labels, int64_t n_tokens,
                                 int64_t hidden_size, int64_t vocab, float rcp_temperature, const float* lse,
                                 const float* mean_z, const float* d_logprobs, const float* d_entropy,
                                 float d_entropy_scalar, const float* logits_cache, void* d_hidden, void* d_weight,
                                 int d_weight_mode, float* d_weight_acc32, int64_t vocab_chunk, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  int st = check_head_shapes(n_tokens, hidden_size, vocab, logits_cache);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(hidden && weight && labels && lse && mean_z, "lce_backward: null pointer");
  VAMD_REQUIRE(rcp_temperature > 0.f, "lce_backward: temperature must be positive");
  VAMD_REQUIRE(d_weight_mode >= VAMD_DW_STORE && d_weight_mode <= VAMD_DW_NONE,
               "lce_backward: unknown d_weight_mode %d", d_weight_mode);
  const bool want_dw = d_weight_mode != VAMD_DW_NONE;
  VAMD_REQUIRE(d_hidden || want_dw, "lce_backward: neither d_hidden nor a weight gradient is asked for");
  {
    const bool writes_bf16 = d_weight_mode <= VAMD_DW_ADD_BF16 || d_weight_mode == VAMD_DW_F32_ADD_FINISH;
    const bool uses_f32 = want_dw && d_weight_mode >= VAMD_DW_F32_STORE;
    VAMD_REQUIRE(!writes_bf16 || d_weight, "lce_backward: d_weight_mode %d writes d_weight, which is null", d_weight_mode);
    VAMD_REQUIRE(!uses_f32 || (d_weight_acc32 && reinterpret_cast<uintptr_t>(d_weight_acc32) % 16 == 0),
                 "lce_backward: d_weight_mode %d needs a 16-byte aligned d_weight_acc32", d_weight_mode);
  }
  {  // K-major operands are addressed with 32-bit byte offsets from their tile origin
    const int64_t rows_padded = ceil_div(n_tokens, kTile) * kTile;
    const int64_t row_pitch = dz_pitch(default_vocab_chunk(n_tokens, hidden_size, vocab, vocab_chunk));
    VAMD_REQUIRE(n_tokens * hidden_size * 2 < (1ll << 32) && rows_padded * row_pitch * 2 < (1ll << 32),
                 "lce_backward: hidden states (%lld x %lld) or the d_logits panel exceed 4 GiB; split the tokens into "
                 "chunks and accumulate d_weight", (long long)n_tokens, (long long)hidden_size);
  }
  const size_t need = vamd_lce_backward_workspace_bytes(n_tokens, hidden_size, vocab, vocab_chunk);
  if (!workspace || workspace_bytes < need) {
    set_error("lce_backward: workspace %zu bytes, need %zu", workspace_bytes, need);
    return VAMD_EWORKSPACE;
  }
  if ((st = ensure_lds_attributes()) != VAMD_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cus = device_cu_count();

  const int tok_tiles = (int)ceil_div(n_tokens, kTile);
  const int64_t n_pad = (int64_t)tok_tiles * kTile;
  const int64_t cv = default_vocab_chunk(n_tokens, hidden_size, vocab, vocab_chunk);
  const int n_chunks = (int)ceil_div(vocab, cv);
  Carver carve(workspace);
  const int64_t pitch = dz_pitch(cv);
  uint16_t* dz = carve.take<uint16_t>((size_t)n_pad * pitch);
  float* acc32 = (n_chunks > 1 && d_hidden) ? carve.take<float>((size_t)n_tokens * hidden_size) : nullptr;
  const uint16_t* hid = static_cast<const uint16_t*>(hidden);
  const uint16_t* wgt = static_cast<const uint16_t*>(weight);
  const int h_tiles = (int)ceil_div(hidden_size, kTile);

  for (int ci = 0; ci < n_chunks; ++ci) {
    const int64_t c0 = (int64_t)ci * cv;
    const int64_t left = vocab - c0;                   // vocabulary rows from c0 on
    const int64_t cols = left < cv ? left : cv;        // valid columns in this chunk
    const int chunk_tiles = (int)ceil_div(cols, kTile);

    if (logits_cache) {
      DLogitsArgs d;
      d.z_cache = logits_cache;
      d.labels = labels;
      d.lse = lse;
      d.mean_z = mean_z;
      d.g_lp = d_logprobs;
      d.g_ent = d_entropy;
      d.g_ent_scalar = d_entropy_scalar;
      d.rcp_t = rcp_temperature;
      d.n_tokens = (int)n_tokens;
      d.vocab = (int)vocab;
      d.chunk_c0 = (int)c0;
      d.chunk_cols = chunk_tiles * kTile;
      d.dz = dz;
      d.dz_ld = (int)pitch;
      {
        ScopedTiming tm(kTagDLogits, s);
        hipLaunchKernelGGL(lce_dlogits_kernel, dim3((unsigned)n_pad, (unsigned)ceil_div(d.chunk_cols, 2048)), dim3(256),
                           0, s, d);
      }
      VAMD_LAUNCH_CHECK();
    } else {
      RecomputeArgs r;
      r.hidden = Operand{hid, hidden_size, (int)n_tokens, (int)hidden_size};
      r.weight = Operand{wgt + c0 * hidden_size, hidden_size, (int)left, (int)hidden_size};
      r.labels = labels;
      r.lse = lse;
      r.mean_z = mean_z;
      r.g_lp = d_logprobs;
      r.g_ent = d_entropy;
      r.g_ent_scalar = d_entropy_scalar;
      r.n_tokens = (int)n_tokens;
      r.vocab_left = (int)left;
      r.chunk_c0 = (int)c0;
      r.k_slabs = (int)(hidden_size / kBK);
      r.tok_tiles = tok_tiles;
      r.chunk_tiles = chunk_tiles;
      r.scale2 = rcp_temperature * kLog2e;
      r.rcp_t = rcp_temperature;
      r.dz = dz;
      r.dz_ld = (int)pitch;
      {
        const int tiles = tok_tiles * chunk_tiles;
        const int grid = tiles < cus ? tiles : cus;
        {
          ScopedTiming tm(kTagRecompute, s);
          hipLaunchKernelGGL(lce_recompute_kernel, dim3(grid), dim3(kThreads), kLdsBytes + kCacheStageBytes, s, r);
        }
        VAMD_LAUNCH_CHECK();
      }
    }

    // d_hidden: k runs over the chunk's vocabulary columns (staged zeros beyond `cols`)
    GemmOutArgs gh;
    gh.R = Operand{dz, pitch, (int)n_pad, (int)cv};
    gh.C = Operand{wgt + c0 * hidden_size, hidden_size, (int)hidden_size, (int)left};
    gh.k_slabs = (int)ceil_div(cols, kBK);
    gh.r_tiles = d_hidden ? tok_tiles : 0;  // an input that needs no gradient leaves its GEMM an empty tile list
    gh.c_tiles = h_tiles;
    gh.r_valid = (int)n_tokens;
    gh.c_valid = (int)hidden_size;
    if (n_chunks == 1) gh.mode = kFinalBf16;
    else if (ci == 0) gh.mode = kStoreF32;
    else if (ci == n_chunks - 1) gh.mode = kFinalBf16AddPrev;
    else gh.mode = kAddF32;
    gh.acc32 = acc32;
    gh.out = static_cast<uint16_t*>(d_hidden);
    gh.ld_out = hidden_size;
    // d_weight rows of this chunk: k runs over tokens (staged zeros beyond n_tokens)
    GemmOutArgs gw;
    gw.R = Operand{dz, pitch, (int)(ceil_div(cols, 8) * 8), (int)n_pad};
    gw.C = Operand{hid, hidden_size, (int)hidden_size, (int)n_tokens};
    gw.k_slabs = (int)ceil_div(n_tokens, kBK);
    gw.r_tiles = want_dw ? chunk_tiles : 0;
    gw.c_tiles = h_tiles;
    gw.r_valid = (int)cols;
    gw.c_valid = (int)hidden_size;
    gw.mode = d_weight_mode;
    gw.acc32 = d_weight_acc32 ? d_weight_acc32 + c0 * hidden_size : nullptr;
    gw.out = d_weight ? static_cast<uint16_t*>(d_weight) + c0 * hidden_size : nullptr;
    gw.ld_out = hidden_size;
    {
      const int tiles = gh.r_tiles * gh.c_tiles + gw.r_tiles * gw.c_tiles;
      const int grid = tiles < cus ? tiles : cus;
      ScopedTiming tm(kTagDGrad, s);
      hipLaunchKernelGGL(lce_dgrad_kernel, dim3(grid), dim3(kThreads), kLdsBytes + kCacheStageBytes, s, gh, gw);
    }
    VAMD_LAUNCH_CHECK();
  }
  return VAMD_OK;
}
