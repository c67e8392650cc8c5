// bf16 x bf16 -> fp32 MFMA tile engine for gfx950 (MI355X), shared by the four
// GEMM-shaped kernels of the log-prob/entropy head (forward logits, backward
// logit recompute, dHidden, dWeight).
//
// One workgroup = 512 threads = 8 wavefronts (two per SIMD, so that one wavefront's
// loads, LDS traffic and epilogue arithmetic issue in the shadow of the other's
// MFMAs) laid out 4 x 2 over a 256 x 256 output tile; each wavefront owns a
// 64 (rows) x 128 (columns) sub-tile as 2 x 4 blocks of v_mfma_f32_32x32x16_bf16
// (128 fp32 accumulators per lane).  The tile engine computes
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
// writes and the ds_read_b128 fragment reads are bank-conflict free).  Two slabs
// per operand are double-buffered: 4 x 32 KB = 128 KB of the CU's 160 KB LDS.
//
// An operand may live in memory either K-contiguous ("direct": element (x,k) at
// base[x*ld + k]) or K-major ("kmajor": element (x,k) at base[k*ld + x]).  The
// kmajor loader transposes 8x4 bf16 blocks in registers on the way to LDS, so
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

constexpr int kTile = 256;                    // output tile edge
constexpr int kBK = 64;                       // k extent of one slab
constexpr int kWavesR = 4;                    // wavefronts along r
constexpr int kWavesC = 2;                    // wavefronts along c
constexpr int kThreads = 64 * kWavesR * kWavesC;
constexpr int kNB = kTile / 32 / kWavesR;     // 32-row blocks per wavefront    (2)
constexpr int kMB = kTile / 32 / kWavesC;     // 32-column blocks per wavefront (4)
constexpr int kLoads = kTile * 8 / kThreads;  // 16-byte staging loads per lane per operand slab (4)
constexpr int kSlabBytes = kTile * kBK * 2;   // 32 KB
constexpr int kLdsBytes = 4 * kSlabBytes;     // R,C x 2 stages = 128 KB
static_assert(kNB == 2 && kMB == 4 && kLoads == 4, "slab_iter's slot schedule is written for this layout");

// One GEMM operand as the tile engine sees it.
struct Operand {
  const uint16_t* base;  // bf16 bits
  int64_t ld;            // leading dimension, elements
  int x_extent;          // extent along the operand's output index (rows of R / columns of C)
  int k_extent;          // extent along k (kmajor operands: number of rows in memory)
};

struct Accum {
  f32x16 a[kMB][kNB];  // [mb: 32-wide block along c][nb: 32-wide block along r]
};

__device__ __forceinline__ void accum_zero(Accum& acc) {
#pragma unroll
  for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc.a[mb][nb][v] = 0.f;
}

// Position of the calling lane inside the workgroup tile.
struct LanePos {
  int wr;  // wavefront's quarter along r (0..3)
  int wc;  // wavefront's half along c (0/1)
  int lr;  // lane % 32 : r offset inside a 32-block
  int lh;  // lane / 32 : which 4-column group of every 8 the lane holds
};

__device__ __forceinline__ LanePos lane_pos() {
  LanePos p;
  const int t = threadIdx.x;
  const int w = t >> 6;
  p.wr = w % kWavesR;
  p.wc = w / kWavesR;
  p.lr = t & 31;
  p.lh = (t >> 5) & 1;
  return p;
}

// Column offset inside the 256-wide tile of accumulator element (mb, v) for this lane.
__device__ __forceinline__ int acc_col(const LanePos& p, int mb, int v) {
  return p.wc * (kMB * 32) + mb * 32 + 8 * (v >> 2) + 4 * p.lh + (v & 3);
}
// Row offset inside the 256-tall tile of accumulator block nb for this lane.
__device__ __forceinline__ int acc_row(const LanePos& p, int nb) { return p.wr * (kNB * 32) + nb * 32 + p.lr; }

// LDS swizzle: the 16-byte chunk c of slab row r lives at chunk position c ^ swizzle_of(r).
// ds_read_b128 is served 16 lanes (256 B, all 64 banks) per cycle; a fragment read touches 16
// consecutive rows at one logical chunk, i.e. 8 even and 8 odd rows (two rows span the 64
// banks), so rows of equal parity must land on 8 different chunk positions: (r >> 1) & 7.
// Transposing (kmajor) staging writes 8-byte half chunks of rows that are 8 apart from
// consecutive lanes; XOR-ing in (r >> 4) spreads those over all 8 chunk positions as well
// while only adding a constant to any run of 16 consecutive rows.
// Direct staging writes cover whole 128 B rows with consecutive lanes and are conflict free
// under any XOR of the chunk index.
__device__ __forceinline__ int swizzle_of(int row) { return ((row >> 1) ^ (row >> 4)) & 7; }

// Byte offset inside a slab of the fragment chunk `logical_chunk` for the lane whose block-local
// row is lr, in the 32-row block that starts at row `block_row` of the slab: the lane part; the
// caller XORs (block index within the wavefront) << 5, which is the compile-time part of
// swizzle_of(block_row + 32 i + lr).
__device__ __forceinline__ int frag_chunk_off(int logical_chunk, int block_row, int lr) {
  return (logical_chunk ^ swizzle_of(block_row + lr)) << 4;
}

// ---------------------------------------------------------------------------------------------
// Where one slab of an operand comes from: a buffer resource whose base is the operand's tile
// origin, plus the scalar byte offset of the slab's first k.  Reads past the end of the operand
// return zero (buffer bounds check), which is what rows / k beyond the valid extent must
// contribute, so the loaders carry no clamping arithmetic.
struct SlabSrc {
  __amdgpu_buffer_rsrc_t rsrc;
  unsigned soff;
};

template <bool KMAJOR>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const Operand& op, int x0) {
  // direct: rows x0.. of [x_extent][ld];  kmajor: columns x0.. of [k_extent][ld]
  const int64_t first = KMAJOR ? (int64_t)x0 : (int64_t)x0 * op.ld;
  const int64_t total = (KMAJOR ? (int64_t)op.k_extent : (int64_t)op.x_extent) * op.ld;
  int64_t bytes = (total - first) * 2;
  if (bytes < 0) bytes = 0;
  if (bytes > 0xffffffffll) bytes = 0xffffffffll;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(op.base + first), 0, (int)(unsigned)bytes, 0x00020000);
}

template <bool KMAJOR>
__device__ __forceinline__ unsigned slab_soff(const Operand& op, int k0) {
  return KMAJOR ? (unsigned)k0 * ((unsigned)op.ld * 2u) : (unsigned)k0 * 2u;
}

// Global -> register -> LDS staging for one 256 x 64 slab of an operand: 4 x 16 bytes per lane.
//
// direct : load i is row (t/8 + 64 i), 16-byte chunk t%8 of the slab; 8 lanes fetch one 128 B row
//          and store i writes load i as one 16-byte chunk.
// kmajor : thread (xg, kq) owns the 8(x) x 4(k) block at x = 8 xg, k = 4 kq, with xg = lane%8 +
//          8 (wave%4) and kq = lane/8 + 8 (wave/4): load i is the 8 x-values of k = 4 kq + i, so 8
//          consecutive lanes fetch one whole 128 B line of a memory row; the block is transposed
//          in registers and store j writes the 4 k-values of x = 8 xg + j as one 8-byte half
//          chunk, so no transposed copy of an operand ever exists in memory.
// Either way the per-lane address is ONE 32-bit offset; everything that changes between loads,
// slabs and tiles is scalar (buffer resource + scalar offset).
template <bool KMAJOR>
struct SlabLoader {
  static constexpr int kStores = KMAJOR ? 8 : kLoads;
  u32x4 reg[kLoads];
  unsigned voff;     // per-lane byte offset of load 0 inside the tile
  unsigned step;     // scalar byte offset between consecutive loads
  unsigned lds_off;  // per-lane byte offset of store 0 inside a slab
  unsigned lds_xor;  // kmajor: chunk position before the (j >> 1) XOR

  __device__ __forceinline__ void init(const Operand& op) {
    const unsigned t = threadIdx.x;
    const unsigned ld_bytes = (unsigned)op.ld * 2u;
    if constexpr (!KMAJOR) {
      const unsigned kc = t & 7, row = t >> 3;  // rows 0..63, + 64 per load
      voff = row * ld_bytes + kc * 16u;
      step = 64u * ld_bytes;
      // swizzle_of(row + 64 i) == swizzle_of(row) ^ 4 (i & 1): store i flips bit 6 of the offset
      lds_off = row * 128u + ((kc ^ (unsigned)swizzle_of((int)row)) << 4);
      lds_xor = 0;
    } else {
      const unsigned lane = t & 63u, w = t >> 6;
      const unsigned xg = (lane & 7u) + 8u * (w & 3u), kq = (lane >> 3) + 8u * (w >> 2);
      voff = kq * 4u * ld_bytes + xg * 16u;
      step = ld_bytes;
      lds_off = xg * 1024u + (kq & 1u) * 8u;
      // swizzle_of(8 xg + j) = (((xg & 1) << 2) | (j >> 1)) ^ ((xg >> 1) & 7)
      lds_xor = (kq >> 1) ^ ((xg & 1u) << 2) ^ ((xg >> 1) & 7u);
    }
  }

  __device__ __forceinline__ void issue_one(int i, const SlabSrc& src) {
    reg[i] = __builtin_amdgcn_raw_buffer_load_b128(src.rsrc, (int)voff, (int)(src.soff + (unsigned)i * step), 0);
  }

  __device__ __forceinline__ void store_one(int j, char* slab) const {
    if constexpr (!KMAJOR) {
      *reinterpret_cast<u32x4*>(slab + (lds_off ^ ((unsigned)(j & 1) << 6)) + j * 8192) = reg[j];
    } else {
      // x = 8 xg + j : bf16 #j of each of the 4 loads (k = 4 kq .. 4 kq + 3)
      u32x2 o;
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const unsigned lo = reg[2 * p][j >> 1];
        const unsigned hi = reg[2 * p + 1][j >> 1];
        o[p] = (j & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
      }
      *reinterpret_cast<u32x2*>(slab + lds_off + j * 128 + ((lds_xor ^ (unsigned)(j >> 1)) << 4)) = o;
    }
  }
};

// ---------------------------------------------------------------------------------------------
// MFMA fragments of one 16-k step: kMB blocks of C and kNB blocks of R, 6 ds_read_b128 per lane.
struct Frags {
  bf16x8 c[kMB], r[kNB];
};

// Workgroup barrier that only waits for this wavefront's LDS traffic: global loads issued for
// later slabs stay in flight across it (a __syncthreads() would drain them too).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---------------------------------------------------------------------------------------------
// One slab (64 k = four 16-k steps of 8 MFMAs per wavefront) of the software pipeline.
//
// The body is written as 32 slots "one MFMA + a few short memory instructions", each closed by
// a scheduling barrier so the compiler keeps the order; memory instructions are spread evenly so
// the vector-memory and LDS pipes see a steady duty instead of bursts:
//
//   step 0 : fragment reads of step 1 | R staging -> LDS(nxt)  | loads C[2..3] of slab it+1
//   step 1 : fragment reads of step 2 |                        | loads R[0..1] of slab it+2
//   step 2 : fragment reads of step 3 | C staging -> LDS(nxt)  | loads R[2..3] of slab it+2
//   -- LDS-only barrier --
//   step 3 : step-0 fragment reads of slab it+1 from nxt       | loads C[0..1] of slab it+2
//
// Every staging register has at least two steps between its load and its LDS write, and
// neither the barrier nor the first fragment reads of a slab sit at the head of the stream.
template <bool RK, bool CK>
__device__ __forceinline__ void slab_iter(SlabLoader<RK>& lr, SlabLoader<CK>& lc, const SlabSrc& c1,
                                          const SlabSrc& r2, const SlabSrc& c2, const char* cur, char* nxt,
                                          const LanePos& p, Frags& f0, Accum& acc) {
  const int row_r = p.wr * (kNB * 32), row_c = p.wc * (kMB * 32);
  const int lane_r = (row_r + p.lr) * 128;
  const int lane_c = kSlabBytes + (row_c + p.lr) * 128;
  Frags f1;
#define VAMD_MFMA(F, i)                                                                                            \
  acc.a[(i) >> 1][(i) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F.c[(i) >> 1], F.r[(i) & 1],                    \
                                                                     acc.a[(i) >> 1][(i) & 1], 0, 0, 0)
#define VAMD_FRAG(G, base, i, lc)                                                                              \
  do {                                                                                                         \
    if ((i) < kMB)                                                                                             \
      G.c[(i)] = *reinterpret_cast<const bf16x8*>((base) + lane_c + (i) * 4096 +                                \
                                                  (frag_chunk_off((lc) + p.lh, row_c, p.lr) ^ ((i) << 5)));     \
    else if ((i) < kMB + kNB)                                                                                  \
      G.r[(i) - kMB] = *reinterpret_cast<const bf16x8*>((base) + lane_r + ((i) - kMB) * 4096 +                  \
                                                        (frag_chunk_off((lc) + p.lh, row_r, p.lr) ^            \
                                                         (((i) - kMB) << 5)));                                 \
  } while (0)
#define VAMD_SLOT_END __builtin_amdgcn_sched_barrier(0)
  constexpr int kRS = SlabLoader<RK>::kStores, kCS = SlabLoader<CK>::kStores;

  // ---- step 0 : MFMA(f0); f1 <- step 1 fragments; R staging -> nxt; C[2..3] of slab it+1
  {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      VAMD_MFMA(f0, i);
      VAMD_FRAG(f1, cur, i, 2);
#ifndef VAMD_DBG_NO_STORE
      if (kRS == 8 || i < 4) lr.store_one(i, nxt);
#endif
#ifndef VAMD_DBG_NO_GLOBAL
      if (i == 5) lc.issue_one(2, c1);
      if (i == 7) lc.issue_one(3, c1);
#endif
      VAMD_SLOT_END;
    }
  }
  // ---- step 1 : MFMA(f1); f0 <- step 2 fragments; R[0..1] of slab it+2
  {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      VAMD_MFMA(f1, i);
      VAMD_FRAG(f0, cur, i, 4);
#ifndef VAMD_DBG_NO_GLOBAL
      if (i == 1) lr.issue_one(0, r2);
      if (i == 5) lr.issue_one(1, r2);
#endif
      VAMD_SLOT_END;
    }
  }
  // ---- step 2 : MFMA(f0); f1 <- step 3 fragments; C staging -> nxt; R[2..3] of slab it+2
  {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      VAMD_MFMA(f0, i);
      VAMD_FRAG(f1, cur, i, 6);
#ifndef VAMD_DBG_NO_STORE
      if (kCS == 8 || i < 4) lc.store_one(i, nxt + kSlabBytes);
#endif
#ifndef VAMD_DBG_NO_GLOBAL
      if (i == 5) lr.issue_one(2, r2);
      if (i == 7) lr.issue_one(3, r2);
#endif
      VAMD_SLOT_END;
    }
  }
  lds_barrier();
  VAMD_SLOT_END;
  // ---- step 3 : MFMA(f1); f0 <- step 0 fragments of the next slab; C[0..1] of slab it+2
  {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      VAMD_MFMA(f1, i);
      VAMD_FRAG(f0, nxt, i, 0);
#ifndef VAMD_DBG_NO_GLOBAL
      if (i == 1) lc.issue_one(0, c2);
      if (i == 5) lc.issue_one(1, c2);
#endif
      VAMD_SLOT_END;
    }
  }
#undef VAMD_MFMA
#undef VAMD_FRAG
#undef VAMD_SLOT_END
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
// Past the end of the stream the fetch cursor stays on the last slab (two redundant fetches)
// instead of branching, which keeps the loop body a single basic block.
template <bool R_KMAJOR, bool C_KMAJOR, class Sched, class Epi>
__device__ __forceinline__ void run_tiles(const Operand& R, const Operand& C, int k_slabs, Sched& sched, Epi& epi,
                                          char* lds) {
  const int ntiles = sched.count();
  if (ntiles <= 0) return;
  const LanePos pos = lane_pos();
  SlabLoader<R_KMAJOR> lr;
  SlabLoader<C_KMAJOR> lc;
  lr.init(R);
  lc.init(C);

  // fetch cursor: (t2, k2) names the slab whose sources are (src_r, src_c)
  int t2 = 0, k2 = 0, r0, c0;
  sched.tile(0, r0, c0);
  __amdgpu_buffer_rsrc_t rs_r = tile_rsrc<R_KMAJOR>(R, r0), rs_c = tile_rsrc<C_KMAJOR>(C, c0);
  SlabSrc src_r{rs_r, 0u}, src_c{rs_c, 0u};
  auto advance = [&]() {
    if (t2 == ntiles - 1 && k2 == k_slabs - 1) return;
    if (++k2 == k_slabs) {
      k2 = 0;
      ++t2;
      int tr, tc;
      sched.tile(t2, tr, tc);
      rs_r = tile_rsrc<R_KMAJOR>(R, tr);
      rs_c = tile_rsrc<C_KMAJOR>(C, tc);
    }
#ifdef VAMD_DBG_SAME_SLAB
    src_r = SlabSrc{rs_r, 0u};
    src_c = SlabSrc{rs_c, (unsigned)(k2 & 1) * 128u};
#else
    src_r = SlabSrc{rs_r, slab_soff<R_KMAJOR>(R, k2 * kBK)};
    src_c = SlabSrc{rs_c, slab_soff<C_KMAJOR>(C, k2 * kBK)};
#endif
  };

  // slab 0 -> LDS stage 0
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    lr.issue_one(i, src_r);
    lc.issue_one(i, src_c);
  }
#pragma unroll
  for (int j = 0; j < SlabLoader<R_KMAJOR>::kStores; ++j) lr.store_one(j, lds);
#pragma unroll
  for (int j = 0; j < SlabLoader<C_KMAJOR>::kStores; ++j) lc.store_one(j, lds + kSlabBytes);
  // slab 1 -> staging registers, except C[2..3] which the first iteration fetches itself
  advance();
#pragma unroll
  for (int i = 0; i < kLoads; ++i) lr.issue_one(i, src_r);
#pragma unroll
  for (int i = 0; i < kLoads / 2; ++i) lc.issue_one(i, src_c);
  SlabSrc c1 = src_c;
  advance();  // cursor now on slab 2
  lds_barrier();
  Frags f0;
  {
    const int row_r = pos.wr * (kNB * 32), row_c = pos.wc * (kMB * 32);
#pragma unroll
    for (int i = 0; i < kMB; ++i)
      f0.c[i] = *reinterpret_cast<const bf16x8*>(lds + kSlabBytes + (row_c + pos.lr) * 128 + i * 4096 +
                                                 (frag_chunk_off(pos.lh, row_c, pos.lr) ^ (i << 5)));
#pragma unroll
    for (int i = 0; i < kNB; ++i)
      f0.r[i] = *reinterpret_cast<const bf16x8*>(lds + (row_r + pos.lr) * 128 + i * 4096 +
                                                 (frag_chunk_off(pos.lh, row_r, pos.lr) ^ (i << 5)));
  }

  int stage = 0;
  for (int tile = 0; tile < ntiles; ++tile) {
    Accum acc;
    accum_zero(acc);
    sched.tile(tile, r0, c0);
    for (int kt = 0; kt < k_slabs; ++kt) {
      const char* cur = lds + stage * 2 * kSlabBytes;
      char* nxt = lds + (stage ^ 1) * 2 * kSlabBytes;
      slab_iter<R_KMAJOR, C_KMAJOR>(lr, lc, c1, src_r, src_c, cur, nxt, pos, f0, acc);
      c1 = src_c;
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
