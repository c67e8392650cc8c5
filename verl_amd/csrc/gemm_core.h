// bf16 x bf16 -> fp32 MFMA tile engine for gfx950 (MI355X), shared by the four
// GEMM-shaped kernels of the log-prob/entropy head (forward logits, backward
// logit recompute, dHidden, dWeight).
//
// One workgroup = 256 threads = 4 wavefronts laid out 2 x 2 over a 256 x 256
// output tile; each wavefront owns a 128 x 128 sub-tile as 4 x 4 blocks of
// v_mfma_f32_32x32x16_bf16 (256 fp32 accumulators per lane).  The tile engine
// computes
//
//     Out[r][c] = sum_k  R[r][k] * C[c][k]
//
// where the R operand ("rows of the output") feeds the MFMA B input and the C
// operand ("columns of the output") feeds the MFMA A input.  With that choice a
// lane of the accumulator block holds ONE output row (r = lane % 32) and runs
// of 4 consecutive output columns, so row-wise reductions over c (the softmax
// over the vocabulary) stay inside a lane and row-major stores are 8/16-byte
// vectors.
//
// Each operand is staged through LDS as a [256 rows][64 k] bf16 slab (128 B per
// row, 16-byte chunks XOR-swizzled by the row index so that both the staging
// writes and the ds_read_b128 fragment reads are bank-conflict free).  Two slabs per
// operand are double-buffered: 4 x 32 KB = 128 KB of the CU's 160 KB LDS.
//
// An operand may live in memory either K-contiguous ("direct": element (x,k) at
// base[x*ld + k]) or K-major ("kmajor": element (x,k) at base[k*ld + x]).  The
// kmajor loader transposes 8x8 bf16 blocks in registers on the way to LDS, so
// no transposed copy of the weight, the hidden states or dLogits is ever
// written to memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vamd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTile = 256;                   // output tile edge
constexpr int kBK = 64;                      // k extent of one slab
constexpr int kThreads = 256;                // 4 wavefronts
constexpr int kSlabBytes = kTile * kBK * 2;  // 32 KB
constexpr int kLdsBytes = 4 * kSlabBytes;    // R,C x 2 stages = 128 KB

// One GEMM operand as the tile engine sees it.
struct Operand {
  const uint16_t* base;  // bf16 bits
  int64_t ld;            // leading dimension, elements
  int x_extent;          // valid extent along the operand's output index (rows of R / cols of C)
  int k_extent;          // valid extent along k (only used to clamp kmajor row addresses)
};

struct Accum {
  f32x16 a[4][4];  // [mb: 32-wide block along c][nb: 32-wide block along r]
};

__device__ __forceinline__ void accum_zero(Accum& acc) {
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc.a[mb][nb][v] = 0.f;
}

// Position of the calling lane inside the workgroup tile.
struct LanePos {
  int wr;  // wavefront's half along r (0/1)
  int wc;  // wavefront's half along c (0/1)
  int lr;  // lane % 32 : r offset inside a 32-block
  int lh;  // lane / 32 : which 4-column group of every 8 the lane holds
};

__device__ __forceinline__ LanePos lane_pos() {
  LanePos p;
  const int t = threadIdx.x;
  const int w = t >> 6;
  p.wr = w & 1;
  p.wc = w >> 1;
  p.lr = t & 31;
  p.lh = (t >> 5) & 1;
  return p;
}

// Column offset inside the 256-wide tile of accumulator element (mb, v) for this lane.
__device__ __forceinline__ int acc_col(const LanePos& p, int mb, int v) {
  return p.wc * 128 + mb * 32 + 8 * (v >> 2) + 4 * p.lh + (v & 3);
}
// Row offset inside the 256-tall tile of accumulator block nb for this lane.
__device__ __forceinline__ int acc_row(const LanePos& p, int nb) { return p.wr * 128 + nb * 32 + p.lr; }

// LDS swizzle: the 16-byte chunk c of slab row r lives at chunk position c ^ swizzle_of(r).
// ds_read_b128 is served 16 lanes (256 B, all 64 banks) per cycle; a fragment read touches 16
// consecutive rows at one logical chunk, i.e. 8 even and 8 odd rows (two rows span the 64
// banks), so rows of equal parity must land on 8 different chunk positions: (r >> 1) & 7.
// Staging writes go 8 lanes (one whole row) per cycle and are conflict free under any XOR.
__device__ __forceinline__ int swizzle_of(int row) { return (row >> 1) & 7; }

// ---------------------------------------------------------------------------------------------
// Global -> register staging for one 256 x 64 slab of an operand.
//
// Addresses are formed as (wave-uniform 64-bit base) + (per-lane 32-bit byte offset) so that the
// loads use the scalar-base addressing form and cost one VGPR of address each.  Direct operands
// use tile-relative offsets (no size limit); kmajor operands use offsets from the operand base
// (the host checks that a kmajor operand spans less than 4 GiB).
template <bool KMAJOR>
struct SlabLoader {
  u32x4 reg[8];
  unsigned off[KMAJOR ? 1 : 8];

  __device__ __forceinline__ void set_tile(const Operand& op, int x0) {
    const int t = threadIdx.x;
    if constexpr (!KMAJOR) {
      // chunk id c = t + 256*i : row = c / 8, 16-byte chunk kc = c % 8
      const int kc = t & 7;
      const int row_in = t >> 3;
      const int last = op.x_extent - 1 - x0;
      const unsigned ld_bytes = (unsigned)op.ld * 2u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int row = row_in + 32 * i;
        row = row < last ? row : last;
        off[i] = (unsigned)row * ld_bytes + (unsigned)kc * 16u;
      }
    } else {
      // one 8(x) x 8(k) block per thread: kg = t % 8, xg = t / 8
      const int xg = t >> 3;
      int xcol = x0 + xg * 8;
      const int xlast = op.x_extent - 8;
      xcol = xcol < xlast ? xcol : xlast;
      off[0] = (unsigned)xcol * 2u;
    }
  }

  // x0: first output index of the tile, k0: first k of the slab.
  __device__ __forceinline__ void issue(const Operand& op, int x0, int k0) {
    if constexpr (!KMAJOR) {
      const char* tile = reinterpret_cast<const char*>(op.base + (int64_t)x0 * op.ld + k0);
#pragma unroll
      for (int i = 0; i < 8; ++i) reg[i] = *reinterpret_cast<const u32x4*>(tile + off[i]);
    } else {
      const char* base = reinterpret_cast<const char*>(op.base);
      const int kg = threadIdx.x & 7;
      const int klast = op.k_extent - 1;
      const unsigned ld_bytes = (unsigned)op.ld * 2u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int k = k0 + kg * 8 + i;
        k = k < klast ? k : klast;
        reg[i] = *reinterpret_cast<const u32x4*>(base + ((unsigned)k * ld_bytes + off[0]));
      }
    }
  }

  // Write the staged slab into LDS in the [row][k] swizzled layout.
  __device__ __forceinline__ void store(char* slab) const {
    const int t = threadIdx.x;
    if constexpr (!KMAJOR) {
      const int kc = t & 7;
      const int row_in = t >> 3;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = row_in + 32 * i;
        *reinterpret_cast<u32x4*>(slab + row * 128 + ((kc ^ swizzle_of(row)) << 4)) = reg[i];
      }
    } else {
      const int kg = t & 7;
      const int xg = t >> 3;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // output row j of the block: the 8 k values of x = xg*8 + j
        u32x4 o;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const unsigned lo = reg[2 * p][j >> 1];
          const unsigned hi = reg[2 * p + 1][j >> 1];
          o[p] = (j & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
        }
        const int row = xg * 8 + j;
        *reinterpret_cast<u32x4*>(slab + row * 128 + ((kg ^ swizzle_of(row)) << 4)) = o;
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------
// MFMA fragments of one 16-k step: 4 blocks of each operand, 8 ds_read_b128 per lane.
struct Frags {
  bf16x8 c[4], r[4];
};

__device__ __forceinline__ void load_frags(Frags& f, const char* r_lane, const char* c_lane, int chunk) {
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) f.c[mb] = *reinterpret_cast<const bf16x8*>(c_lane + mb * 4096 + chunk);
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) f.r[nb] = *reinterpret_cast<const bf16x8*>(r_lane + nb * 4096 + chunk);
}

__device__ __forceinline__ void mma_frags(const Frags& f, Accum& acc) {
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
      acc.a[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.c[mb], f.r[nb], acc.a[mb][nb], 0, 0, 0);
}

// Workgroup barrier that only waits for this wavefront's LDS traffic: global loads issued for
// later slabs stay in flight across it (a __syncthreads() would drain them too).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Scheduling hint: the next `n` instructions of class `mask` come next in program order.
// 0x008 MFMA, 0x100 DS read, 0x200 DS write, 0x020 VMEM read, 0x002 VALU.
#define VAMD_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)

// ---------------------------------------------------------------------------------------------
// One slab (64 k) of the software pipeline.  On entry: f0 holds the step-0 fragments of this
// slab, the staging registers of both loaders hold slab it+1 (loads issued one iteration ago),
// `cur` is the LDS stage of this slab and `nxt` the other stage (free: its last readers passed
// the previous barrier).  The four 16-k steps interleave, in MFMA issue shadows,
//   step 0 : fragment reads of step 1 | R staging -> LDS(nxt) | R global loads of slab it+2
//   step 1 : fragment reads of step 2 | C staging -> LDS(nxt) | C global loads of slab it+2
//   step 2 : fragment reads of step 3
//   barrier (LDS only)
//   step 3 : step-0 fragment reads of slab it+1 from nxt
// so neither the staging writes, nor the barrier, nor the first fragment reads of a slab sit on
// the critical path; only MFMA issue does.
template <bool RK, bool CK>
__device__ __forceinline__ void slab_iter(SlabLoader<RK>& lr, SlabLoader<CK>& lc, const Operand& R, const Operand& C,
                                          int r2, int c2, int k2, const char* cur, char* nxt, const LanePos& p,
                                          Frags& f0, Accum& acc) {
  const int sw = swizzle_of(p.lr);
  const int lane_r = (p.wr * 128 + p.lr) * 128;
  const int lane_c = kSlabBytes + (p.wc * 128 + p.lr) * 128;
  const char* r_lane = cur + lane_r;
  const char* c_lane = cur + lane_c;
  Frags f1;
  // ---- step 0
  load_frags(f1, r_lane, c_lane, ((2 + p.lh) ^ sw) << 4);
#ifndef VAMD_DBG_NO_STORE
  lr.store(nxt);
#endif
#ifndef VAMD_DBG_NO_GLOBAL
  lr.issue(R, r2, k2);
#endif
  mma_frags(f0, acc);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    VAMD_SGB(0x008, 1);
    VAMD_SGB(0x100, 1);
    if (RK) VAMD_SGB(0x002, 4);
    VAMD_SGB(0x008, 1);
    VAMD_SGB(0x200, 1);
    VAMD_SGB(0x020, 1);
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- step 1
  load_frags(f0, r_lane, c_lane, ((4 + p.lh) ^ sw) << 4);
#ifndef VAMD_DBG_NO_STORE
  lc.store(nxt + kSlabBytes);
#endif
#ifndef VAMD_DBG_NO_GLOBAL
  lc.issue(C, c2, k2);
#endif
  mma_frags(f1, acc);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    VAMD_SGB(0x008, 1);
    VAMD_SGB(0x100, 1);
    if (CK) VAMD_SGB(0x002, 4);
    VAMD_SGB(0x008, 1);
    VAMD_SGB(0x200, 1);
    VAMD_SGB(0x020, 1);
  }
  __builtin_amdgcn_sched_barrier(0);
  // ---- step 2
  load_frags(f1, r_lane, c_lane, ((6 + p.lh) ^ sw) << 4);
  mma_frags(f0, acc);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    VAMD_SGB(0x008, 2);
    VAMD_SGB(0x100, 1);
  }
  __builtin_amdgcn_sched_barrier(0);
  lds_barrier();
  __builtin_amdgcn_sched_barrier(0);
  // ---- step 3
  load_frags(f0, nxt + lane_r, nxt + lane_c, ((0 + p.lh) ^ sw) << 4);
  mma_frags(f1, acc);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    VAMD_SGB(0x008, 2);
    VAMD_SGB(0x100, 1);
  }
  __builtin_amdgcn_sched_barrier(0);
}

// ---------------------------------------------------------------------------------------------
// Persistent, software-pipelined walk over a list of output tiles.
//
//   Sched : int count();  void tile(int i, int& r0, int& c0);
//   Epi   : void operator()(Accum& acc, int r0, int c0);   (registers + global memory only)
//
// All (tile, slab) pairs of the workgroup form one stream of slabs; slab it+1 is staged into
// LDS and slab it+2 is fetched from memory while slab it is multiplied, across tile boundaries
// too, so only the very first slab pays a cold start and epilogues find their next slab ready.
template <bool R_KMAJOR, bool C_KMAJOR, class Sched, class Epi>
__device__ __forceinline__ void run_tiles(const Operand& R, const Operand& C, int k_slabs, Sched& sched, Epi& epi,
                                          char* lds) {
  const int ntiles = sched.count();
  if (ntiles <= 0) return;
  const LanePos pos = lane_pos();
  SlabLoader<R_KMAJOR> lr;
  SlabLoader<C_KMAJOR> lc;

  // slab 0 -> LDS stage 0
  int r0, c0;
  sched.tile(0, r0, c0);
  lr.set_tile(R, r0);
  lc.set_tile(C, c0);
  lr.issue(R, r0, 0);
  lc.issue(C, c0, 0);
  lr.store(lds);
  lc.store(lds + kSlabBytes);
  // slab 1 -> staging registers; (t2, k2, r2, c2) then names slab 2.  Past the end of the
  // stream the cursor stays on the last slab: the pipeline re-fetches it instead of branching.
  int t2 = 0, k2 = 0, r2 = r0, c2 = c0;
  bool new_tile = false;
  auto advance = [&]() {
    new_tile = false;
    if (t2 == ntiles - 1 && k2 == k_slabs - 1) return;
    if (++k2 == k_slabs) {
      k2 = 0;
      ++t2;
      sched.tile(t2, r2, c2);
      new_tile = true;
    }
  };
  advance();
  if (new_tile) {
    lr.set_tile(R, r2);
    lc.set_tile(C, c2);
  }
  lr.issue(R, r2, k2 * kBK);
  lc.issue(C, c2, k2 * kBK);
  advance();
  lds_barrier();
  Frags f0;
  {
    const int sw = swizzle_of(pos.lr);
    load_frags(f0, lds + (pos.wr * 128 + pos.lr) * 128, lds + kSlabBytes + (pos.wc * 128 + pos.lr) * 128,
               ((0 + pos.lh) ^ sw) << 4);
  }

  int it = 0, stage = 0;
  for (int tile = 0; tile < ntiles; ++tile) {
    Accum acc;
    accum_zero(acc);
    sched.tile(tile, r0, c0);
    for (int kt = 0; kt < k_slabs; ++kt, ++it) {
      const char* cur = lds + stage * 2 * kSlabBytes;
      char* nxt = lds + (stage ^ 1) * 2 * kSlabBytes;
      if (new_tile) {
        lr.set_tile(R, r2);
        lc.set_tile(C, c2);
      }
      slab_iter<R_KMAJOR, C_KMAJOR>(lr, lc, R, C, r2, c2, k2 * kBK, cur, nxt, pos, f0, acc);
      advance();
      stage ^= 1;
    }
    epi(acc, r0, c0);
  }
}

// ---------------------------------------------------------------------------------------------
// Tile order for a plain (r_tiles x c_tiles) problem walked by `nwg` persistent workgroups.
//
// Hardware hands workgroup b to XCD b % 8.  The ids are first regrouped so that every XCD
// owns a contiguous run of the tile sequence, then the sequence walks r fastest inside bands
// of 8 r-tiles, so the 32 workgroups resident on one XCD cover an 8 x 4 patch and share their
// R / C slabs through that XCD's L2.
struct GroupedSched {
  int r_tiles, c_tiles, nwg, wg;
  __device__ __forceinline__ int count() const {
    const int total = r_tiles * c_tiles;
    return (total - wg + nwg - 1) / nwg;
  }
  __device__ __forceinline__ void tile(int i, int& r0, int& c0) const {
    const int q = i * nwg + wg;
    const int band = 8 * c_tiles;
    const int b = q / band;
    const int first_r = b * 8;
    const int rows = (r_tiles - first_r) < 8 ? (r_tiles - first_r) : 8;
    const int w = q - b * band;
    r0 = (first_r + w % rows) * kTile;
    c0 = (w / rows) * kTile;
  }
};

// Regroup a hardware workgroup id so that XCD x owns ids [x*n/8, (x+1)*n/8).
__device__ __forceinline__ int xcd_regroup(int b, int n) {
  if ((n & 7) != 0) return b;
  return (b & 7) * (n >> 3) + (b >> 3);
}

}  // namespace vamd
