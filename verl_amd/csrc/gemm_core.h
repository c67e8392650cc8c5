// bf16 x bf16 -> fp32 MFMA tile engine for gfx950 (MI355X), shared by the GEMM-shaped kernels
// of the log-prob/entropy head (forward logits, backward logit recompute, d_hidden, d_weight).
//
// One workgroup = 512 threads = 8 wavefronts (two per SIMD, so that one wavefront's LDS traffic
// and epilogue arithmetic issue in the shadow of the other's MFMAs) laid out 4 x 2 over a
// 256 x 256 output tile; each wavefront owns a 64 (rows) x 128 (columns) sub-tile as 4 x 8
// blocks of v_mfma_f32_16x16x32_bf16 (128 fp32 accumulators per lane).  The 16 x 16 x 32 shape is
// chosen for energy: it touches half the accumulator registers per flop of the 32 x 32 x 16 shape,
// and on operands that toggle the board sustains 2.12 against 1.87 PFLOP/s with it in a pure MFMA
// loop (the clock this part holds is set by power, so flops per joule are flops per second).
// The engine computes
//
//     Out[r][c] = sum_k  R[r][k] * C[c][k]
//
// where the R operand ("rows of the output") feeds the MFMA B input and the C operand
// ("columns of the output") feeds the MFMA A input.  With that choice a lane of the accumulator
// block holds ONE output row (r = lane % 16) and 4 consecutive output columns (4 (lane / 16) ..),
// so row-wise reductions over c (the softmax over the vocabulary) stay inside a lane and
// row-major stores are 8/16-byte vectors.
//
// Operand slabs (256 x 64 k, 32 KB) travel from memory straight into LDS with
// buffer_load_dwordx4 ... lds: no staging registers, no LDS store instructions, and a wavefront
// waits for its loads once per slab (just before the barrier that publishes the slab) instead of
// before every staging store.  Two slabs per operand are double-buffered: 4 x 32 KB = 128 KB of
// the CU's 160 KB LDS.  A load writes the 64 lanes' 16-byte pieces to 1 KB of consecutive LDS, so
// the bank swizzle is applied on the memory side: each lane fetches the chunk that belongs at
// its LDS position.
//
// An operand may live in memory K-contiguous ("direct": element (x,k) at base[x*ld + k]) or
// K-major ("kmajor": element (x,k) at base[k*ld + x]).  A direct slab is kept as [256 x][64 k]
// and read with ds_read_b128; a kmajor slab is kept exactly as it lies in memory, [64 k][256 x],
// and read with ds_read_b64_tr_b16, which hands every lane the 4 consecutive k of its own x.  No
// transposed copy of the weight, the hidden states or d_logits is ever written anywhere.
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
constexpr int kWaves = kWavesR * kWavesC;
constexpr int kThreads = 64 * kWaves;
constexpr int kBlk = 16;                      // edge of an MFMA output block
constexpr int kNB = kTile / kBlk / kWavesR;   // 16-row blocks per wavefront    (4)
constexpr int kMB = kTile / kBlk / kWavesC;   // 16-column blocks per wavefront (8)
constexpr int kLoads = kTile * 8 / kThreads;  // 16-byte memory -> LDS transfers per lane per operand slab (4)
constexpr int kSteps = kBK / 32;              // 32-k MFMA steps per slab (2)
constexpr int kSlabBytes = kTile * kBK * 2;   // 32 KB
constexpr int kLdsBytes = 4 * kSlabBytes;     // R,C x 2 stages = 128 KB
static_assert(kNB == 4 && kMB == 8 && kLoads == 4 && kSteps == 2, "slab_iter's slot schedule is written for this layout");
// A four-wavefront layout (128 x 128 per wavefront, one per SIMD, accumulators in the AGPRs) issues a third fewer LDS
// reads but was measured slower, and hungrier per flop: with one wavefront per SIMD nothing fills the cycles it spends
// at the barriers and in the epilogue (forward 14.0 against 12.9 ms, gradient GEMMs 35.4 against 25.9 ms per step at
// 16384 x 152064 x 3584 with this instruction and schedule; 869 against 795 W per PFLOP/s above the idle board).

// One GEMM operand as the tile engine sees it.
struct Operand {
  const uint16_t* base;  // bf16 bits
  int64_t ld;            // leading dimension, elements
  int x_extent;          // extent along the operand's output index (rows of R / columns of C)
  int k_extent;          // extent along k (kmajor operands: number of rows in memory)
};

struct Accum {
  f32x4 a[kMB][kNB];  // [mb: 16-wide block along c][nb: 16-wide block along r]
};

__device__ __forceinline__ void accum_zero(Accum& acc) {
#pragma unroll
  for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc.a[mb][nb][v] = 0.f;
}

// Position of the calling lane inside the workgroup tile.
struct LanePos {
  int wr;  // wavefront's quarter along r (0..3)
  int wc;  // wavefront's half along c (0/1)
  int lx;  // lane % 16 : r offset inside a 16-block
  int lq;  // lane / 16 : which 4-column group of a block's 16 the lane holds
};

__device__ __forceinline__ LanePos lane_pos() {
  LanePos p;
  const int t = threadIdx.x;
  const int w = t >> 6;
  p.wr = w % kWavesR;
  p.wc = w / kWavesR;
  p.lx = t & 15;
  p.lq = (t >> 4) & 3;
  return p;
}

// Column offset inside the 256-wide tile of accumulator element (mb, v) for this lane.
__device__ __forceinline__ int acc_col(const LanePos& p, int mb, int v) {
  return p.wc * (kMB * kBlk) + mb * kBlk + 4 * p.lq + v;
}
// Row offset inside the 256-tall tile of accumulator block nb for this lane.
__device__ __forceinline__ int acc_row(const LanePos& p, int nb) { return p.wr * (kNB * kBlk) + nb * kBlk + p.lx; }

// ---------------------------------------------------------------------------------------------
// LDS layouts and their swizzles.
//
// direct slab : row x (128 B = 8 chunks of 16 B); chunk c lives at position c ^ ((x >> 1) & 7).
//   ds_read_b128 is served 16 lanes (256 B, all 64 banks) per cycle; a fragment read touches 16
//   consecutive rows at one logical chunk, i.e. 8 even and 8 odd rows (two rows span the banks),
//   so rows of equal parity must land on 8 different chunk positions.
// kmajor slab : row k (512 B = 32 chunks of 16 B); chunk c lives at position c ^ (4 (k & 3)) ^ (2 ((k >> 3) & 1)).
//   A transposing 8-byte read is served 32 lanes at a time, and those address 8 k rows (k = 8 lq + 0..3 for two
//   values of lq) x 32 B at one x block; rows are 512 B apart (the same banks), so the first XOR moves the 4 rows of
//   a quad to 4 different 64 B groups and the second puts the rows of the odd lq in the other 32 B half: the 8 rows
//   cover the 64 banks once (with the first XOR alone the two lq groups collided: 45 % of the LDS cycles of the
//   gradient GEMMs were bank-conflict cycles).
__device__ __forceinline__ int swizzle_direct(int row) { return (row >> 1) & 7; }

// Where one slab of an operand comes from: a buffer resource whose base is the operand's tile
// origin, plus the scalar byte offset of the slab's first k.  Reads past the end of the operand
// return zero (buffer bounds check), which is what rows / k beyond the valid extent must
// contribute, so the loaders carry no clamping arithmetic.
struct SlabSrc {
  u32x4 rsrc;  // buffer resource words: base, base high | stride 0, byte count, raw 32-bit format
  unsigned soff;
};

template <bool KMAJOR>
__device__ __forceinline__ u32x4 tile_rsrc(const Operand& op, int x0) {
  // direct: rows x0.. of [x_extent][ld];  kmajor: columns x0.. of [k_extent][ld]
  const int64_t first = KMAJOR ? (int64_t)x0 : (int64_t)x0 * op.ld;
  const int64_t total = (KMAJOR ? (int64_t)op.k_extent : (int64_t)op.x_extent) * op.ld;
  int64_t bytes = (total - first) * 2;
  if (bytes < 0) bytes = 0;
  if (bytes > 0xffffffffll) bytes = 0xffffffffll;
  const uint64_t base = reinterpret_cast<uint64_t>(op.base + first);
  return u32x4{(unsigned)base, (unsigned)(base >> 32) & 0xffffu, (unsigned)bytes, 0x00020000u};
}

template <bool KMAJOR>
__device__ __forceinline__ unsigned slab_soff(const Operand& op, int k0) {
  return KMAJOR ? (unsigned)k0 * ((unsigned)op.ld * 2u) : (unsigned)k0 * 2u;
}

// LDS byte address of a pointer into the workgroup's LDS allocation.
__device__ __forceinline__ unsigned lds_address(const char* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// buffer_load_dwordx4 ... lds: lane L's 16 bytes from (resource, voff + soff) land at LDS address
// lds_base + 16 L (lds_base is wave-uniform and travels in M0).  Written as inline assembly so
// that the compiler's wait-count bookkeeping does not see an outstanding LDS write and fence
// every later LDS read against it; the engine waits for its transfers itself, once per slab.
__device__ __forceinline__ void load_to_lds_16(const u32x4& rsrc, unsigned voff, unsigned soff, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_base)
               : "memory", "m0");
}

// The same for 4 bytes per lane: lane L's dword lands at lds_base + 4 L (256 consecutive bytes per instruction).
__device__ __forceinline__ void load_to_lds_4(const u32x4& rsrc, unsigned voff, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dword %0, %1, 0 offen lds"
               :
               : "v"(voff), "s"(rsrc), "s"(lds_base)
               : "memory", "m0");
}
// Buffer resource over `bytes` bytes at p (raw 32-bit format, reads past the end return zero).
__device__ __forceinline__ u32x4 span_rsrc(const void* p, int64_t bytes) {
  if (bytes < 0) bytes = 0;
  if (bytes > 0xffffffffll) bytes = 0xffffffffll;
  const uint64_t base = reinterpret_cast<uint64_t>(p);
  return u32x4{(unsigned)base, (unsigned)(base >> 32) & 0xffffu, (unsigned)bytes, 0x00020000u};
}

// Memory -> LDS transfer of one operand slab: kLoads loads of 16 bytes per lane.  Load i of wavefront
// w fills the 1 KB LDS block (w + kWaves i) of the slab:
//   direct : block b = rows 8 b .. 8 b + 7; lane L sits at row 8 b + L / 8, chunk position L % 8,
//            and fetches logical chunk (L % 8) ^ swizzle of that row -- 8 lanes cover one whole
//            128 B line of the memory row;
//   kmajor : block b = k rows 2 b, 2 b + 1; lane L sits at k row 2 b + L / 32, chunk position
//            L % 32, and fetches logical chunk (L % 32) ^ 4 (k & 3) ^ 2 ((k >> 3) & 1) -- 32 lanes cover 512
//            contiguous bytes of the memory row.
// Both swizzles are unchanged by the + 64 rows (direct) / + 16 k rows (kmajor) between loads, so
// the per-lane address is ONE 32-bit offset; everything that changes between loads, slabs and
// tiles is scalar (buffer resource, scalar offset, LDS base in M0).
template <bool KMAJOR>
struct SlabDma {
  unsigned voff;      // per-lane byte offset of load 0 inside the tile
  unsigned step;      // scalar byte offset between consecutive loads
  unsigned lds_wave;  // byte offset of this wavefront's first block inside the slab

  __device__ __forceinline__ void init(const Operand& op) {
    const unsigned lane = threadIdx.x & 63u, w = threadIdx.x >> 6;
    const unsigned ld_bytes = (unsigned)op.ld * 2u;
    if constexpr (!KMAJOR) {
      const unsigned row = 8u * w + (lane >> 3);
      voff = row * ld_bytes + (((lane & 7u) ^ (unsigned)swizzle_direct((int)row)) << 4);
      step = (8u * kWaves) * ld_bytes;
    } else {
      const unsigned k = 2u * w + (lane >> 5);
      voff = k * ld_bytes + (((lane & 31u) ^ (4u * (k & 3u)) ^ (2u * ((k >> 3) & 1u))) << 4);
      step = (2u * kWaves) * ld_bytes;
    }
    lds_wave = __builtin_amdgcn_readfirstlane(w * 1024u);
  }

  // slab_lds: LDS byte address of the operand's slab in the stage being filled
  __device__ __forceinline__ void issue_one(int i, const SlabSrc& src, unsigned slab_lds) const {
    load_to_lds_16(src.rsrc, voff, src.soff + (unsigned)i * step, slab_lds + lds_wave + (unsigned)i * (kWaves * 1024u));
  }
};

// ---------------------------------------------------------------------------------------------
// Per-lane LDS addressing of MFMA fragments.  A fragment of the 16 x 16 x 32 instruction is, for lane
// (lx = lane % 16, lq = lane / 16), the 8 consecutive k (k = 32 s + 8 lq + 0..7 of k-step s) of slab row
// x = 16 * block + lx.
//   direct : one ds_read_b128 at  x * 128 + (((4 s + lq) ^ swizzle(x)) << 4);
//   kmajor : two transposing 8-byte reads.  Within the 16 lanes of one lq, lane i addresses the 8 bytes at
//            (k row k0 + i / 4, x0 + 4 (i % 4)) and receives the 4 k (k0 .. k0 + 3) of x0 + i; the second read
//            takes k0 + 4.
template <bool KMAJOR>
struct FragAddr {
  // direct: off[s] = lane part for k-step s, block adds 2048 b.  kmajor: off[b] = lane part for
  // block b of the wavefront, k-step adds 16384 s (+ 2048 for the second read).
  int off[KMAJOR ? kMB : kSteps];

  // first_block: index of the wavefront's first 16-row block inside the slab
  __device__ __forceinline__ void init(int first_block, int nblocks) {
    const int l = threadIdx.x & 63;
    const int lx = l & 15, lq = l >> 4;
    if constexpr (!KMAJOR) {
#pragma unroll
      for (int s = 0; s < kSteps; ++s)
        off[s] = (first_block * kBlk + lx) * 128 + (((4 * s + lq) ^ swizzle_direct(lx)) << 4);
    } else {
      const int q = lx >> 2;  // (k & 3) of the addressed row: every k offset added later is a multiple of 4
      const int k0 = 8 * lq + q;
#pragma unroll
      for (int b = 0; b < kMB; ++b) {
        const int blk = first_block + b;
        off[b] = b < nblocks ? k0 * 512 + 64 * ((blk >> 1) ^ q) + 32 * ((blk & 1) ^ (lq & 1)) + 8 * (lx & 3) : 0;
      }
    }
  }

  __device__ __forceinline__ bf16x8 read(const char* slab, int s, int b) const {
    if constexpr (!KMAJOR) {
      return *reinterpret_cast<const bf16x8*>(slab + off[s] + b * (kBlk * 128));
    } else {
      typedef bf16x4 __attribute__((address_space(3))) * tr_ptr_t;
      const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((tr_ptr_t)(slab + off[b] + s * 16384));
      const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((tr_ptr_t)(slab + off[b] + s * 16384 + 2048));
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }
};

// MFMA fragments in flight.  The kNB blocks of R of both k-steps of a slab are held whole; the blocks of C stream
// through a ring of four: group G of a slab (G = 8 * k-step + mb, four MFMAs each) reads ring slot G % 4.
struct Frags {
  bf16x8 r[kSteps][kNB];
  bf16x8 c[4];
};

// ---------------------------------------------------------------------------------------------
// One slab (64 k = two 32-k steps of 32 MFMAs per wavefront) of the software pipeline.
//
// The body is 64 slots "one MFMA + at most two memory instruction groups", each closed by a scheduling barrier so
// the compiler keeps the order.  Slot j = 4 G + nb multiplies block (mb = G % 8, nb) of k-step G / 8.
//
//   slots  0..51 : the C fragment of group G + 3 is read from `cur` in the first slot of group G (its ring slot was
//                  last used by group G - 1); the R fragments of k-step 1 are read in groups 1..4
//   after slot 21: every R fragment of the slab is in registers; a first workgroup barrier frees the R half of `cur`,
//                  and the R transfers of slab it+2 go into it one at a time in slots 26, 34, 42 and 50 (with them,
//                  in slots 30 and 38, the two transfers of a K-major C slab that cover k-step 0, which nobody reads
//                  after slot 16: 25.2 against 25.6 ms per step in the gradient GEMMs)
//   after slot 55: wait for this wavefront's LDS reads and for its transfers of slab it+1 (all but its four or six
//                  newest transfers, which belong to slab it+2), second workgroup barrier: nobody reads `cur` any more, and
//                  `nxt` is complete
//   slots 56..63 : the fragments the next slab starts with (R of k-step 0, C of groups 0..2) are read from `nxt`,
//                  and the C transfers of slab it+2 into `cur` are issued
//
// so a transfer has at least 56 slots of MFMA work to land before anyone waits for it, nothing inside the slots
// depends on memory, and the eight wavefronts never hand the memory pipeline more than four transfers each at one
// time: issuing all eight after the closing barrier cost a fifth of the throughput whenever the clock was not held
// down by the power limit (1.57 against 1.92 PFLOP/s on all-zero operands at 16384 x 152064 x 3584).  On entry f holds
// R of k-step 0 and C of groups 0..2 of this slab.
template <bool RK, bool CK>
__device__ __forceinline__ void slab_iter(const SlabDma<RK>& dr, const SlabDma<CK>& dc, const SlabSrc& r2,
                                          const SlabSrc& c2, char* cur, const char* nxt, const FragAddr<RK>& fr,
                                          const FragAddr<CK>& fc, Frags& f, Accum& acc) {
#pragma unroll
  for (int j = 0; j < 64; ++j) {
    const int G = j >> 2, nb = j & 3, ks = G >> 3, mb = G & 7;
    acc.a[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.c[G & 3], f.r[ks][nb], acc.a[mb][nb], 0, 0, 0);
    if (j < 52) {
      if (nb == 0) {
        const int g3 = G + 3;  // <= 15: still this slab
        f.c[g3 & 3] = fc.read(cur + kSlabBytes, g3 >> 3, g3 & 7);
      }
      if (nb == 1 && G >= 1 && G <= kNB) f.r[1][G - 1] = fr.read(cur, 1, G - 1);
      // LDS reads return in order: with at most one read outstanding (it belongs to the C fragment of slot 20) the
      // last R fragment, read in slot 17, has arrived
      if (j == 21) asm volatile("s_waitcnt lgkmcnt(1)\n\ts_barrier" ::: "memory");
      if (j >= 26 && (j - 26) % 8 == 0) dr.issue_one((j - 26) / 8, r2, lds_address(cur));
      // a K-major C slab lies in LDS k row by k row: the rows of k-step 0 (its transfers 0 and 1) were last read in
      // slot 16, so they are as free as R by now
      if (CK && (j == 30 || j == 38)) dc.issue_one((j - 30) / 8, c2, lds_address(cur) + kSlabBytes);
    } else if (j >= 56) {
      const int k = j - 56;
      if (k == 0) f.c[0] = fc.read(nxt + kSlabBytes, 0, 0);
      if (k < kNB) f.r[0][k] = fr.read(nxt, 0, k);
      if (k == 4) f.c[1] = fc.read(nxt + kSlabBytes, 0, 1);
      if (k == 5) f.c[2] = fc.read(nxt + kSlabBytes, 0, 2);
      // the C transfers that are left, in slots that carry at most one read
      if (CK) {
        if (k == 3 || k == 6) dc.issue_one(k == 3 ? 2 : 3, c2, lds_address(cur) + kSlabBytes);
      } else {
        if (k == 1 || k == 3 || k == 6 || k == 7)
          dc.issue_one(k == 1 ? 0 : k == 3 ? 1 : k - 4, c2, lds_address(cur) + kSlabBytes);
      }
    }
    // transfers complete in issue order, so "at most n outstanding" leaves only the n transfers of slab it+2 issued
    // so far: four for R, and two more when C is K-major
    if (j == 55) {
      if (CK) asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}
static_assert(kLoads == 4, "the s_waitcnt vmcnt(4 / 6) of slab_iter counts the transfers of slab it+2 issued before it");

// ---------------------------------------------------------------------------------------------
// Persistent, software-pipelined walk over a list of output tiles.
//
//   Sched : int count();  void tile(int i, int& r0, int& c0);
//   Epi   : void operator()(Accum& acc, int r0, int c0);   (registers + global memory only, or LDS
//           beyond the first kLdsBytes)
//           void prefetch(int tile, int r0, int c0);  called by every wavefront before the first slab of tile
//           `tile` is multiplied: memory -> LDS transfers issued here have landed, and are visible to the
//           whole workgroup, when that tile's epilogue runs (they are older than every slab transfer the tile
//           issues, and the slab pipeline's waits and barriers cover them); an epilogue that needs per-row
//           values stages them this way instead of loading them itself, which would have it wait out its own
//           loads AND every slab transfer in flight (one counter counts both)
//
// All (tile, slab) pairs of the workgroup form one stream of slabs; slab it+1 is landing in LDS
// and slab it+2 is requested while slab it is multiplied, across tile boundaries too, so only the
// very first slab pays a cold start and epilogues find their next slab ready.  Past the end of
// the stream the fetch cursor stays on the last slab (two redundant transfers) instead of
// branching, which keeps the loop body a single basic block.  On return every transfer of the
// calling wavefront has landed; the caller must pass a workgroup barrier before it reuses the
// first kLdsBytes of LDS.
template <bool R_KMAJOR, bool C_KMAJOR, class Sched, class Epi>
__device__ __forceinline__ void run_tiles(const Operand& R, const Operand& C, int k_slabs, Sched& sched, Epi& epi,
                                          char* lds) {
  const int ntiles = sched.count();
  if (ntiles <= 0) return;
  const LanePos pos = lane_pos();
  SlabDma<R_KMAJOR> dr;
  SlabDma<C_KMAJOR> dc;
  dr.init(R);
  dc.init(C);
  FragAddr<R_KMAJOR> fr;
  FragAddr<C_KMAJOR> fc;
  fr.init(pos.wr * kNB, kNB);
  fc.init(pos.wc * kMB, kMB);

  // fetch cursor: (t2, k2) names the slab whose sources are (src_r, src_c)
  int t2 = 0, k2 = 0, r0, c0;
  sched.tile(0, r0, c0);
  u32x4 rs_r = tile_rsrc<R_KMAJOR>(R, r0), rs_c = tile_rsrc<C_KMAJOR>(C, c0);
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
    src_r = SlabSrc{rs_r, slab_soff<R_KMAJOR>(R, k2 * kBK)};
    src_c = SlabSrc{rs_c, slab_soff<C_KMAJOR>(C, k2 * kBK)};
  };

  // slab 0 -> stage 0, slab 1 -> stage 1
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    dr.issue_one(i, src_r, lds_address(lds));
    dc.issue_one(i, src_c, lds_address(lds) + kSlabBytes);
  }
  advance();
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    dr.issue_one(i, src_r, lds_address(lds) + 2 * kSlabBytes);
    dc.issue_one(i, src_c, lds_address(lds) + 3 * kSlabBytes);
  }
  advance();  // cursor now on slab 2
  epi.prefetch(0, r0, c0);
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  Frags f;
#pragma unroll
  for (int i = 0; i < kNB; ++i) f.r[0][i] = fr.read(lds, 0, i);
#pragma unroll
  for (int i = 0; i < 3; ++i) f.c[i] = fc.read(lds + kSlabBytes, 0, i);

  int stage = 0;
  for (int tile = 0; tile < ntiles; ++tile) {
    Accum acc;
    accum_zero(acc);
    sched.tile(tile, r0, c0);
    if (tile > 0) epi.prefetch(tile, r0, c0);
    for (int kt = 0; kt < k_slabs; ++kt) {
      char* cur = lds + stage * 2 * kSlabBytes;
      const char* nxt = lds + (stage ^ 1) * 2 * kSlabBytes;
      slab_iter<R_KMAJOR, C_KMAJOR>(dr, dc, src_r, src_c, cur, nxt, fr, fc, f, acc);
      advance();
      stage ^= 1;
    }
    epi(acc, r0, c0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
