// Shared skeleton of the HBM-bound [rows, cols] kernels (masked reductions, losses, GRPO).
//
// A launch covers the matrix with workgroups of 256 threads; workgroup (row, chunk) owns
// kChunk = 4096 consecutive columns of one row and each thread walks them in float4 steps that
// are contiguous across the wavefront (64 lanes x 16 B = 1 KiB per load instruction); all of a
// thread's loads are issued before any arithmetic so that a workgroup keeps 16 KiB per input in
// flight.  Partial sums leave the workgroup as doubles in a fixed tree order, one record per
// (row, chunk); the workgroup that finishes last (ticket counter at the head of the workspace)
// combines the records in index order inside the same launch, so results are bit-reproducible,
// no floating-point atomics are used and a reduction costs one kernel launch.
//
// Workspace contract of these kernels: the first 256 bytes hold the ticket counter; they must be
// zero on entry and are zero again when the kernel has finished.
#pragma once
#include "common.h"

namespace vamd {

constexpr int kRcThreads = 256;
constexpr int kChunk = 4096;  // columns per workgroup
constexpr int kGroups = kChunk / (kRcThreads * 4);  // float4 groups per thread per input (4)
constexpr int kTicketGroups = 64;   // first-level arrival counters
constexpr int kTicketStride = 256;  // bytes between counters
constexpr size_t kTicketBytes = (size_t)(kTicketGroups + 1) * kTicketStride;
static_assert(kTicketBytes == VAMD_TICKET_BYTES, "the header documents the size of the counter area");

inline int64_t chunks_of(int64_t cols) { return cols <= 0 ? 1 : (cols + kChunk - 1) / kChunk; }

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Streaming hint.  A launch of this many workgroups (4096 columns each: 64 MB per fp32 tensor, and these kernels
// touch three to six tensors) moves more than the 256 MB Infinity Cache holds, so nothing it reads or writes will be
// found there again: its loads and stores are issued non-temporal, which on this part is worth 7 - 9 % of HBM
// bandwidth at 128 MB per tensor (two-tensor read 6.3 -> 6.9 TB/s, four-in one-out 5.5 -> 6.2 TB/s) and 10 - 20 % at
// 64 MB (2048 x 8192: policy loss with gradient 71.5 -> 64.6 us, GRPO 47.0 -> 38.9 us).  It measured faster still at
// 32 MB per tensor on cold buffers, but there the working set fits the cache and a consumer may find it there, so
// smaller launches keep the default policy: their tensors (8 MB at the benchmark size) are usually still cached from
// the kernel that produced them, and are read again by the next one.
// The test is uniform over the launch, so it costs one scalar branch per access.
// Kernels whose grid is not one workgroup per 4096 columns pass the flag themselves (streams_past_caches(elements)).
constexpr unsigned kStreamingGrid = 4096;
__device__ __forceinline__ bool launch_streams_past_caches() { return gridDim.x >= kStreamingGrid; }
__device__ __forceinline__ bool streams_past_caches(int64_t elements) {
  return elements >= (int64_t)kStreamingGrid * 4096;
}

typedef float nt_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned nt_u32x4 __attribute__((ext_vector_type(4)));

template <bool VEC>
__device__ __forceinline__ void ld4(const float* __restrict__ p, int64_t i, int valid, float (&x)[4],
                                    bool streaming = launch_streams_past_caches()) {
  if constexpr (VEC) {
    // the two loads are kept apart on purpose (a branch, not a select): merged into one they lose the hint
    if (streaming) {
      const nt_f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_f32x4*>(p + i));
      x[0] = v[0]; x[1] = v[1]; x[2] = v[2]; x[3] = v[3];
    } else {
      const float4 v = *reinterpret_cast<const float4*>(p + i);
      x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = e < valid ? p[i + e] : 0.f;
  }
}

template <bool VEC>
__device__ __forceinline__ void st4(float* __restrict__ p, int64_t i, int valid, const float (&x)[4],
                                    bool streaming = launch_streams_past_caches()) {
  if constexpr (VEC) {
    if (streaming) {  // kept apart from the default store by type, or the two are merged and the hint is lost
      const nt_u32x4 v = {__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
      __builtin_nontemporal_store(v, reinterpret_cast<nt_u32x4*>(p + i));
    } else {
      *reinterpret_cast<float4*>(p + i) = make_float4(x[0], x[1], x[2], x[3]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (e < valid) p[i + e] = x[e];
  }
}
// mask -> float weights; elements past `valid` read as 0 (excluded)
template <bool VEC, class M>
__device__ __forceinline__ void ldmask4(const M* __restrict__ p, int64_t i, int valid, float (&w)[4],
                                        bool streaming = launch_streams_past_caches()) {
  if constexpr (VEC) {
    struct alignas(sizeof(M) * 4) Pack { M v[4]; };
    Pack k;
    if (streaming) {
      if constexpr (sizeof(M) == 4 && static_cast<M>(0.5f) != static_cast<M>(0)) {  // fp32 mask: load as integers
        const nt_u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p + i));
        k = __builtin_bit_cast(Pack, raw);
      } else if constexpr (sizeof(M) == 4) {  // int32 mask: load as floats (a type the default path does not use)
        const nt_f32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const nt_f32x4*>(p + i));
        k = __builtin_bit_cast(Pack, raw);
      } else if constexpr (sizeof(M) == 8) {
        struct Two { nt_u32x4 lo, hi; };
        Two raw;
        raw.lo = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p + i));
        raw.hi = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p + i) + 1);
        k = __builtin_bit_cast(Pack, raw);
      } else {
        const unsigned raw = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(p + i));
        k = __builtin_bit_cast(Pack, raw);
      }
    } else {
      k = *reinterpret_cast<const Pack*>(p + i);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = static_cast<float>(k.v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = e < valid ? static_cast<float>(p[i + e]) : 0.f;
  }
}

// Iterate the 4-element groups of this workgroup's chunk: f(flat_index, valid_count)
template <class F>
__device__ __forceinline__ void for_each_group(int64_t row, int chunk, int64_t cols, F&& f) {
  const int64_t c_begin = (int64_t)chunk * kChunk;
  const int64_t c_end = (c_begin + kChunk) < cols ? (c_begin + kChunk) : cols;
  for (int64_t c = c_begin + (int64_t)threadIdx.x * 4; c < c_end; c += kRcThreads * 4) {
    const int64_t left = c_end - c;
    f(row * cols + c, left < 4 ? (int)left : 4);
  }
}

// The 4-element groups one thread owns in its workgroup's chunk.
struct ChunkPos {
  int64_t idx[kGroups];  // flat index of the group's first element
  int valid[kGroups];    // 0..4 elements of the group exist
  // `thread`: position among the 256 threads that walk the chunk (a workgroup that holds several chunks of a row
  // passes threadIdx.x % 256 and gives every 256 threads a chunk; a chunk past the end of the row has no valid group)
  __device__ __forceinline__ ChunkPos(int64_t row, int chunk, int64_t cols, int thread = threadIdx.x) {
    const int64_t c_begin = (int64_t)chunk * kChunk;
    const int64_t c_end = (c_begin + kChunk) < cols ? (c_begin + kChunk) : cols;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      const int64_t c = c_begin + ((int64_t)g * kRcThreads + thread) * 4;
      const int64_t left = c_end - c;
      valid[g] = left >= 4 ? 4 : (left > 0 ? (int)left : 0);
      idx[g] = row * cols + c;
    }
  }
};

template <bool VEC>
__device__ __forceinline__ void load_groups(const float* __restrict__ p, const ChunkPos& pos, float (&x)[kGroups][4],
                                            bool streaming = launch_streams_past_caches()) {
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    if (pos.valid[g] > 0) {
      ld4<VEC>(p, pos.idx[g], pos.valid[g], x[g], streaming);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[g][e] = 0.f;
    }
  }
}

template <bool VEC, class M>
__device__ __forceinline__ void load_mask_groups(const M* __restrict__ p, const ChunkPos& pos, float (&w)[kGroups][4],
                                                 bool streaming = launch_streams_past_caches()) {
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    if (pos.valid[g] > 0) {
      ldmask4<VEC>(p, pos.idx[g], pos.valid[g], w[g], streaming);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) w[g][e] = 0.f;
    }
  }
}

template <bool VEC>
__device__ __forceinline__ void store_groups(float* __restrict__ p, const ChunkPos& pos, const float (&x)[kGroups][4],
                                             bool streaming = launch_streams_past_caches()) {
#pragma unroll
  for (int g = 0; g < kGroups; ++g)
    if (pos.valid[g] > 0) st4<VEC>(p, pos.idx[g], pos.valid[g], x[g], streaming);
}

// Publishing a record to the workgroup that will fold it, without a device-wide fence (an
// agent-scope fence writes back / invalidates a whole XCD's L2 and costs tens of microseconds
// when every workgroup issues one): the record is written with device-coherent stores, the
// writer waits for their acknowledgement, then takes a ticket with a device-scope atomic; the
// folding workgroup reads the records with device-coherent loads.
__device__ __forceinline__ void peer_store(double* p, double v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ double peer_load(const double* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Ticket: true in exactly one workgroup of the launch, the one that arrives last.  Thread 0 must
// have issued its peer_store()s before the call.  The last workgroup calls ticket_reset() when done.
// Arrivals are counted in two levels -- workgroup b takes a ticket from counter 1 + b % G, and the
// last arrival of each of the G counters takes one from counter 0 -- because same-address atomics
// are served one after the other (about 15 ns each here): a single counter costs 8 us for 512
// workgroups and bounds large launches, G = 64 counters on separate lines cost a few hundred ns.
__device__ __forceinline__ unsigned ticket_groups() {
  return gridDim.x < (unsigned)kTicketGroups ? gridDim.x : (unsigned)kTicketGroups;
}
__device__ __forceinline__ bool last_block_arrives(unsigned* counters) {
  __shared__ unsigned last;
  if (threadIdx.x == 0) {
    const unsigned n = gridDim.x, G = ticket_groups();
    const unsigned g = blockIdx.x % G;
    const unsigned members = (n - g + G - 1) / G;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned is_last = 0;
    const unsigned t = __hip_atomic_fetch_add(counters + (1 + g) * (kTicketStride / 4), 1u, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
    if (t == members - 1) {
      const unsigned t2 = __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = t2 == G - 1 ? 1u : 0u;
    }
    last = is_last;
  }
  __syncthreads();
  return last != 0;
}
// The two levels taken apart, for launches whose last workgroup of each first-level counter has work to do
// (folding that counter's share of the records) before it arrives at the second level.
__device__ __forceinline__ bool share_last_arrives(unsigned* counters) {
  __shared__ unsigned last;
  if (threadIdx.x == 0) {
    const unsigned n = gridDim.x, G = ticket_groups();
    const unsigned g = blockIdx.x % G;
    const unsigned members = (n - g + G - 1) / G;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned t = __hip_atomic_fetch_add(counters + (1 + g) * (kTicketStride / 4), 1u, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
    last = t == members - 1 ? 1u : 0u;
  }
  __syncthreads();
  return last != 0;
}
// Called by the workgroups share_last_arrives() was true in, after thread 0 issued the peer_store()s of the share.
__device__ __forceinline__ bool launch_last_arrives(unsigned* counters) {
  __shared__ unsigned last;
  if (threadIdx.x == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const unsigned t = __hip_atomic_fetch_add(counters, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last = t == ticket_groups() - 1 ? 1u : 0u;
  }
  __syncthreads();
  return last != 0;
}
__device__ __forceinline__ void ticket_reset(unsigned* counters) {
  if (threadIdx.x <= ticket_groups())
    __hip_atomic_store(counters + threadIdx.x * (kTicketStride / 4), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------------
// Rendezvous of a whole launch, for kernels that need a launch-wide result (whitening statistics, group
// statistics) before their last pass and would otherwise pay a second launch for it -- which costs as much as
// streaming 8 MB does.  REQUIREMENT: every workgroup of the launch is resident at the same time; the host side
// caps the grid at what the device holds (resident_workgroups) and lets workgroups loop over rows beyond that.
//   arrival   : last_block_arrives() as above; the workgroup it is true in computes the result, publishes it with
//               device-coherent stores and calls gate_release();
//   waiting   : the others poll the release word in gate_wait(), at most spin_limit times (a sleep between
//               polls), so that every wavefront exits whatever happens; false = timed out;
//   departure : every workgroup calls gate_depart() last; the final one to leave zeroes the counter area, so the
//               workspace contract (zero on entry, zero on exit) holds, and reports whether anyone timed out.
// The words live inside the counter area: departures at word 16 of each counter's 256-byte slot, the release flag
// at word 32 and the timed-out flag at word 48 of slot 0.
constexpr int kDepartWord = 16, kReleaseWord = 32, kTimedOutWord = 48;
// Word 33 of slot 0 is an epoch that only ever advances (a meeting without a departure count releases its waiters by
// changing it): the one word of the area that is NOT zero between calls; nothing else reads it.
constexpr int kEpochWord = 33;
// Word 34 of slot 0 counts the workgroups that ever gave up a bounded wait on this buffer (and carried on by other
// means): like the epoch it is not zero between calls and no kernel reads it.  A host reads it now and then to learn
// that the waiting kernels time out on this device (they recover by themselves, at the price of their spin limit).
constexpr int kGaveUpWord = 34;
static_assert(kGaveUpWord * 4 == VAMD_TICKET_GAVE_UP_OFFSET, "the header documents where the count lives");
__device__ __forceinline__ void note_gave_up(unsigned* counters) {  // one thread of the workgroup that gave up
  __hip_atomic_fetch_add(counters + kGaveUpWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr unsigned kGateSpinLimit = 1u << 22;  // polls of about half a microsecond: seconds, not forever

__device__ __forceinline__ void gate_release(unsigned* counters) {  // thread 0, after its peer stores
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __hip_atomic_store(counters + kReleaseWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool gate_wait(unsigned* counters, unsigned spin_limit) {
  __shared__ unsigned released;
  if (threadIdx.x == 0) {
    unsigned seen = 0;
    for (unsigned spins = 0;; ++spins) {
      seen = __hip_atomic_load(counters + kReleaseWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (seen != 0 || spins >= spin_limit) break;
      __builtin_amdgcn_s_sleep(4);
    }
    if (seen == 0) {
      __hip_atomic_store(counters + kTimedOutWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      note_gave_up(counters);
    }
    released = seen;
  }
  __syncthreads();
  return released != 0;
}
// Returns, in the workgroup that leaves last only, 1 + (someone timed out); 0 everywhere else.
__device__ __forceinline__ unsigned gate_depart(unsigned* counters) {
  __shared__ unsigned verdict;
  if (threadIdx.x == 0) {
    const unsigned n = gridDim.x, G = ticket_groups();
    const unsigned g = blockIdx.x % G;
    const unsigned members = (n - g + G - 1) / G;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned v = 0;
    const unsigned t = __hip_atomic_fetch_add(counters + (1 + g) * (kTicketStride / 4) + kDepartWord, 1u,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (t == members - 1) {
      const unsigned t2 = __hip_atomic_fetch_add(counters + kDepartWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (t2 == G - 1)
        v = 1u + __hip_atomic_load(counters + kTimedOutWord, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    verdict = v;
  }
  __syncthreads();
  if (verdict != 0) {
    if (threadIdx.x <= ticket_groups()) {
      unsigned* slot = counters + threadIdx.x * (kTicketStride / 4);
      __hip_atomic_store(slot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slot + kDepartWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (threadIdx.x == 0) {
      __hip_atomic_store(counters + kReleaseWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(counters + kTimedOutWord, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  return verdict;
}
__device__ __forceinline__ void peer_store_f32(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float peer_load_f32(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// "My partial result is in memory" bytes, one per producer (a response, a (row, chunk) record), inside the counter
// area and therefore zero on entry and to be left zero on exit: the second 128-byte line of the 256-byte slots
// 1..64, which no counter uses.  A byte per producer rather than a bit: setting it is a plain device-scope store, not
// a read-modify-write that queues up behind its neighbours'.
constexpr int64_t kReadyBytes = 128 * kTicketGroups;
__device__ __forceinline__ unsigned char* ready_byte(unsigned* ticket, int64_t i) {
  return reinterpret_cast<unsigned char*>(ticket) + (1 + (i >> 7)) * kTicketStride + 128 + (i & 127);
}
// thread 0, after the device-coherent stores of the result
__device__ __forceinline__ void ready_byte_set(unsigned* ticket, int64_t i) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __hip_atomic_store(ready_byte(ticket, i), (unsigned char)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Polls byte i at most `limit` more times in total (`polls` counts across calls); false = gave up.
__device__ __forceinline__ bool ready_byte_wait(unsigned* ticket, int64_t i, unsigned& polls, unsigned limit) {
  const unsigned char* flag = ready_byte(ticket, i);
  while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
    if (polls++ >= limit) return false;
    __builtin_amdgcn_s_sleep(4);
  }
  return true;
}
// The whole workgroup: bytes 0 .. count-1 back to zero (four bytes per word), by whoever leaves the launch last.
template <int NT>
__device__ __forceinline__ void ready_bytes_clear(unsigned* ticket, int64_t count) {
  for (int64_t w = threadIdx.x; w < (count + 3) / 4; w += NT)
    __hip_atomic_store(reinterpret_cast<unsigned*>(ready_byte(ticket, w * 4)), 0u, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// Lane exchange inside the vector ALU (data-parallel primitives): a lane without a source in the pattern, or in a
// row the mask leaves out, receives `none`.  The wavefront scans use the shifts by 1, 2, 4, 8 inside a row of 16
// lanes (0x111 .. 0x118), the last lane of rows 0 / 2 into rows 1 / 3 (0x142, row mask 0xA), lane 31 into rows 2
// and 3 (0x143, row mask 0xC), and the shift by one lane over the whole wavefront (0x138); with `none` the identity
// of the scanned operation no lane test is needed.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float x, float none) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(none), __float_as_int(x), CTRL, ROW_MASK, 0xF, false));
}
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ double dpp_f64(double x, double none) {
  const int lo = __builtin_amdgcn_update_dpp(__double2loint(none), __double2loint(x), CTRL, ROW_MASK, 0xF, false);
  const int hi = __builtin_amdgcn_update_dpp(__double2hiint(none), __double2hiint(x), CTRL, ROW_MASK, 0xF, false);
  return __hiloint2double(hi, lo);
}
// Inclusive running sum over the wavefront, lane 0 first.
__device__ __forceinline__ double wave_running_sum(double x) {
  x += dpp_f64<0x111>(x, 0.0);
  x += dpp_f64<0x112>(x, 0.0);
  x += dpp_f64<0x114>(x, 0.0);
  x += dpp_f64<0x118>(x, 0.0);
  x += dpp_f64<0x142, 0xA>(x, 0.0);
  x += dpp_f64<0x143, 0xC>(x, 0.0);
  return x;
}

// Records of the (row, chunk) workgroups are kept slot-major: slot i of workgroup (row, chunk) lives at
// ((i * chunks + chunk) * rows + row).  The workgroup that folds them gives consecutive rows to consecutive threads,
// so a wavefront's loads of one slot are 512 contiguous bytes; with one record per workgroup stored contiguously
// they would be 64 separate cache lines, and the single CU doing the fold is bound by its request rate.
__device__ __forceinline__ int64_t record_at(int slot, int64_t row, int chunk, int64_t rows, int chunks) {
  return ((int64_t)slot * chunks + chunk) * rows + row;
}

// Thread 0 of workgroup (row, chunk) publishes its record.
template <int NV>
__device__ __forceinline__ void store_record(double* __restrict__ records, int64_t row, int chunk, int64_t rows,
                                             int chunks, const double (&v)[NV]) {
#pragma unroll
  for (int i = 0; i < NV; ++i) peer_store(records + record_at(i, row, chunk, rows, chunks), v[i]);
}

// A record slot as the folding workgroup reads it: through the device-coherent path when the writers belong to
// the same launch (COHERENT), as an ordinary load when the records come from an earlier launch.
template <bool COHERENT>
__device__ __forceinline__ double record_load(const double* p) {
  if constexpr (COHERENT) return peer_load(p);
  else return *p;
}

// Fold the chunk records of ROWS rows, slot by slot: slots [0, NSUM) add up, slots [NSUM, NV) take the maximum
// (records hold minima negated).  Every record load is a round trip to the memory side, and the workgroup
// doing the fold is the only one left running, so the loads of up to FLIGHT chunks of every row of the trip are
// issued together; the order of the additions (chunk 0 first) does not depend on that.
template <int NV, int NSUM, int ROWS, bool COHERENT = true, int FLIGHT = 4>
__device__ __forceinline__ void fold_row_records(const double* __restrict__ records, const int64_t (&row)[ROWS],
                                                 const bool (&have)[ROWS], int64_t rows, int chunks,
                                                 double (&out)[ROWS][NV]) {
  const double ninf = -__longlong_as_double(0x7ff0000000000000ll);
#pragma unroll
  for (int k = 0; k < ROWS; ++k)
#pragma unroll
    for (int i = 0; i < NV; ++i) out[k][i] = i < NSUM ? 0.0 : ninf;
  for (int c0 = 0; c0 < chunks; c0 += FLIGHT) {
    double t[ROWS][FLIGHT][NV];
#pragma unroll
    for (int k = 0; k < ROWS; ++k)
#pragma unroll
      for (int u = 0; u < FLIGHT; ++u) {
        const bool ok = have[k] && c0 + u < chunks;
#pragma unroll
        for (int i = 0; i < NV; ++i)
          t[k][u][i] = ok ? record_load<COHERENT>(records + record_at(i, row[k], c0 + u, rows, chunks))
                          : (i < NSUM ? 0.0 : ninf);
      }
#pragma unroll
    for (int k = 0; k < ROWS; ++k)
#pragma unroll
      for (int u = 0; u < FLIGHT; ++u)
#pragma unroll
        for (int i = 0; i < NV; ++i) out[k][i] = i < NSUM ? out[k][i] + t[k][u][i] : fmax(out[k][i], t[k][u][i]);
  }
}

// acc[i] += slot i of records tid, tid + 256, ... below n (n = rows * chunks records, slot-major), in that order,
// four records in flight at a time.
template <int NV>
__device__ __forceinline__ void sum_records_strided(const double* __restrict__ records, int64_t n, double (&acc)[NV]) {
  for (int64_t k0 = threadIdx.x; k0 < n; k0 += 4 * kRcThreads) {
    double t[4][NV];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t k = k0 + (int64_t)u * kRcThreads;
#pragma unroll
      for (int i = 0; i < NV; ++i) t[u][i] = k < n ? peer_load(records + (int64_t)i * n + k) : 0.0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < NV; ++i) acc[i] += t[u][i];
  }
}

// Sum of every slot over all n = rows * chunks records of the launch (slot-major, record_at).  Returns true in
// exactly one workgroup, whose thread 0 then holds the totals.  Up to kOneLevelRecords records the workgroup that
// arrives last adds them all; a larger launch would leave that one workgroup with dozens of dependent trips to
// memory while the rest of the device idles, so there the last workgroup to arrive at each of the G first-level
// counters adds the records of that counter's workgroups (b = g, g + G, ...: a fixed set, so the result does not
// depend on the order of arrival) and publishes NV share totals behind the records, and the last of those G adds
// the shares.  The shares of early counters are folded while later workgroups still stream.
constexpr int64_t kOneLevelRecords = 4096;
template <int NV>
__device__ __forceinline__ bool sum_all_records(unsigned* counters, double* __restrict__ records, int64_t rows,
                                                int chunks, double (&tot)[NV], double* smem /* NV * 4 */) {
  const int64_t n = rows * chunks;
#pragma unroll
  for (int i = 0; i < NV; ++i) tot[i] = 0;
  if (n <= kOneLevelRecords) {
    if (!last_block_arrives(counters)) return false;
    sum_records_strided<NV>(records, n, tot);
    block_sum<NV, kRcThreads>(tot, smem);
    return true;
  }
  if (!share_last_arrives(counters)) return false;
  const unsigned G = ticket_groups(), g = blockIdx.x % G;
  const int64_t members = (n - g + G - 1) / G;
  double* shares = records + n * NV;  // [NV][G]
  for (int64_t m0 = threadIdx.x; m0 < members; m0 += 4 * kRcThreads) {
    double t[4][NV];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t m = m0 + (int64_t)u * kRcThreads;
      const int64_t b = g + m * G;  // the workgroup whose record this is
      const int64_t k = (b % chunks) * rows + b / chunks;
#pragma unroll
      for (int i = 0; i < NV; ++i) t[u][i] = m < members ? peer_load(records + (int64_t)i * n + k) : 0.0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < NV; ++i) tot[i] += t[u][i];
  }
  block_sum<NV, kRcThreads>(tot, smem);
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < NV; ++i) peer_store(shares + i * G + g, tot[i]);
  if (!launch_last_arrives(counters)) return false;
#pragma unroll
  for (int i = 0; i < NV; ++i) tot[i] = threadIdx.x < G ? peer_load(shares + i * G + threadIdx.x) : 0.0;
  block_sum<NV, kRcThreads>(tot, smem);
  return true;
}
// Doubles a record area needs behind its rows * chunks * nv record slots for sum_all_records().
constexpr size_t kShareSlots = kTicketGroups;

// 4096-column chunks one workgroup of a wide-record statistics pass walks (1, 2 or 4): as many as leave the launch
// a couple of thousand workgroups.
inline int record_span(int64_t rows, int chunks) {
  int span = 4;
  while (span > 1 && (span > chunks || rows * ((chunks + span - 1) / span) < 2048)) span /= 2;
  return span;
}

// Cross-workgroup step of a fold launch that gives every workgroup a share of the rows: on entry thread 0 of each
// workgroup holds NS sums and NX maxima of its share; returns true in exactly one workgroup, whose thread 0 then
// holds them over all shares (a launch of one workgroup returns at once).  shares: gridDim.x * (NS + NX) doubles;
// counter: zero when the launch starts (the streaming pass before it clears it).
template <int NS, int NX, int NT>
__device__ __forceinline__ bool fold_across_workgroups(double (&t)[NS], double (&x)[NX], double* __restrict__ shares,
                                                       unsigned* counter,
                                                       double* stage /* as block_reduce_wide, max(NS, NX) values */) {
  const unsigned nb = gridDim.x;
  if (nb == 1) return true;
  __shared__ unsigned last;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < NS; ++i) peer_store(shares + (size_t)i * nb + blockIdx.x, t[i]);
#pragma unroll
    for (int i = 0; i < NX; ++i) peer_store(shares + (size_t)(NS + i) * nb + blockIdx.x, x[i]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    last = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nb - 1 ? 1u : 0u;
  }
  __syncthreads();
  if (!last) return false;
  const double ninf = -__longlong_as_double(0x7ff0000000000000ll);
#pragma unroll
  for (int i = 0; i < NS; ++i) t[i] = 0.0;
#pragma unroll
  for (int i = 0; i < NX; ++i) x[i] = ninf;
  for (unsigned b = threadIdx.x; b < nb; b += NT) {
    double ts[NS], xs[NX];
#pragma unroll
    for (int i = 0; i < NS; ++i) ts[i] = peer_load(shares + (size_t)i * nb + b);
#pragma unroll
    for (int i = 0; i < NX; ++i) xs[i] = peer_load(shares + (size_t)(NS + i) * nb + b);
#pragma unroll
    for (int i = 0; i < NS; ++i) t[i] += ts[i];
#pragma unroll
    for (int i = 0; i < NX; ++i) x[i] = fmax(x[i], xs[i]);
  }
  block_reduce_wide<NS, NT>(t, stage, SumOp());
  block_reduce_wide<NX, NT>(x, stage, MaxOp());
  return true;
}

// (mean, rsqrt(var_unbiased + 1e-8), shift) from the masked moments sum(m), sum(v m), sum(v^2 m),
// following masked_mean / masked_var / masked_whiten (verl/utils/torch_functional.py:287-339).
__device__ __forceinline__ void whiten_stats_from_moments(double s0, double s1, double s2, int shift_mean,
                                                          float* __restrict__ stats) {
  const float mean = (float)s1 / ((float)s0 + 1e-8f);
  const double md = (double)mean;
  // masked_mean((v - mean)^2) with the same epsilon in the denominator
  float var = (float)((s2 - 2.0 * md * s1 + md * md * s0)) / ((float)s0 + 1e-8f);
  var = var * ((float)s0 / ((float)s0 - 1.f));  // Bessel factor M / (M - 1)
  stats[0] = mean;
  stats[1] = rsqrtf(var + 1e-8f);
  stats[2] = shift_mean ? 0.f : mean;
}

// The vector path needs 4-element groups that never straddle a row and 16-byte aligned rows.
inline bool can_vectorize(int64_t cols, std::initializer_list<const void*> f32_ptrs, const void* mask,
                          size_t mask_elem) {
  if (cols % 4 != 0) return false;
  for (const void* p : f32_ptrs)
    if (p && !aligned_to(p, 16)) return false;
  if (mask && !aligned_to(mask, mask_elem * 4)) return false;
  return true;
}

// ---------------------------------------------------------------------------------------------
// agg_loss combination of per-row sums (verl/trainer/ppo/core_algos.py:1025-1080).
struct AggParams {
  int mode;
  double dp_size, batch_num_tokens, global_batch_size, loss_scale_factor;  // < 0 : None
};

inline AggParams make_agg_params(int mode, double dp, double bnt, double gbs, double lsf) {
  AggParams a;
  a.mode = mode;
  a.dp_size = dp;
  a.batch_num_tokens = bnt;
  a.global_batch_size = gbs;
  a.loss_scale_factor = lsf;
  return a;
}

// Called by ONE workgroup of NT threads (the last one of the launch to arrive, or a launch of its own).  partials: slot-major records (record_at) with slot 0 =
// sum(loss * w) and slot 1 = sum(w); slots >= 2 are summed over everything into extra[].
// Writes loss (double, thread 0) and coef[rows].  FLIGHT: chunk records of a row loaded together in the first pass
// (registers for FLIGHT x 2 x NV doubles; 1 where a row has a single record).
template <int NV, int NT = kRcThreads, bool COHERENT = true, int FLIGHT = 4>
__device__ void finalize_agg(const double* __restrict__ partials, int64_t rows, int chunks, int64_t cols,
                             const AggParams& ap, float* __restrict__ coef, double& loss_out, double& msum_out,
                             double (&extra)[NV > 2 ? NV - 2 : 1], double* smem) {
  // pass 1: totals
  double tot[NV + 1];  // slot NV: number of rows with a non-empty mask
#pragma unroll
  for (int i = 0; i <= NV; ++i) tot[i] = 0;
  double seq_mean_sum = 0;  // sum over kept rows of S_i / (M_i + 1e-8)
  double seq_sum = 0;       // sum over kept rows of S_i
  // two rows per trip, all their chunk records in flight together
  for (int64_t r0 = threadIdx.x; r0 < rows; r0 += 2 * NT) {
    const int64_t rr[2] = {r0, r0 + NT};
    const bool have[2] = {true, rr[1] < rows};
    double row[2][NV];
    fold_row_records<NV, NV, 2, COHERENT, FLIGHT>(partials, rr, have, rows, chunks, row);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      if (!have[k]) break;
#pragma unroll
      for (int i = 0; i < NV; ++i) tot[i] += row[k][i];
      if (row[k][1] > 0) {
        tot[NV] += 1;
        seq_sum += row[k][0];
        seq_mean_sum += (double)((float)row[k][0] / ((float)row[k][1] + 1e-8f));
      }
    }
  }
  double red[NV + 3];
#pragma unroll
  for (int i = 0; i <= NV; ++i) red[i] = tot[i];
  red[NV + 1] = seq_mean_sum;
  red[NV + 2] = seq_sum;
  block_sum<NV + 3, NT>(red, smem);
  __shared__ double bc[NV + 3];
  if (threadIdx.x == 0)
#pragma unroll
    for (int i = 0; i < NV + 3; ++i) bc[i] = red[i];
  __syncthreads();
  const double S = bc[0], Msum = bc[1], kept = bc[NV], smean = bc[NV + 1], ssum = bc[NV + 2];
  double loss = 0, c_all = 0;
  double gbs = ap.global_batch_size < 0 ? kept : ap.global_batch_size;
  switch (ap.mode) {
    case VAMD_AGG_TOKEN_MEAN: {
      const double denom = ap.batch_num_tokens < 0 ? Msum : ap.batch_num_tokens;
      loss = S / denom * ap.dp_size;
      c_all = ap.dp_size / denom;
    } break;
    case VAMD_AGG_SEQ_MEAN_TOKEN_SUM:
      loss = ssum / gbs * ap.dp_size;
      break;
    case VAMD_AGG_SEQ_MEAN_TOKEN_MEAN:
      loss = smean / gbs * ap.dp_size;
      break;
    default: {
      const double f = ap.loss_scale_factor < 0 ? (double)cols : ap.loss_scale_factor;
      loss = S / f;
      c_all = 1.0 / f;
    } break;
  }
  if (coef) {
    const bool per_row = ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_SUM || ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_MEAN;
    for (int64_t r0 = threadIdx.x; r0 < rows; r0 += 4 * NT) {
      double m[4] = {0, 0, 0, 0};
      if (per_row)  // the rows' mask sums again, all loads of the trip in flight together
        for (int c0 = 0; c0 < chunks; c0 += 4) {
          double t[4][4];
#pragma unroll
          for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int64_t r = r0 + (int64_t)k * NT;
              t[k][u] = (r < rows && c0 + u < chunks)
                            ? record_load<COHERENT>(partials + record_at(1, r, c0 + u, rows, chunks)) : 0.0;
            }
#pragma unroll
          for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int u = 0; u < 4; ++u) m[k] += t[k][u];
        }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int64_t r = r0 + (int64_t)k * NT;
        if (r >= rows) break;
        double c = c_all;
        if (per_row) {
          c = 0;
          if (m[k] > 0) c = (ap.mode == VAMD_AGG_SEQ_MEAN_TOKEN_SUM ? 1.0 : 1.0 / (m[k] + 1e-8)) * ap.dp_size / gbs;
        }
        coef[r] = (float)c;
      }
    }
  }
  loss_out = loss;
  msum_out = Msum;
#pragma unroll
  for (int i = 2; i < NV; ++i) extra[i - 2] = bc[i];
}

// =============================================================================================
// Folding the (row, chunk) records of the loss kernels.  Small launches let the workgroup that arrives last
// do it (one launch in all); large ones leave it to a launch of its own: the fold's registers would otherwise
// be charged to every wavefront of the streaming kernel and halve its occupancy.
// =============================================================================================
constexpr int kFoldThreads = 512;
constexpr int64_t kInlineFoldRecords = 2048;  // up to this many (row, chunk) records the last workgroup folds

enum { kEpiAgg, kEpiPolicy, kEpiValue, kEpiKl };

template <int EPI, int NX>
__device__ __forceinline__ void loss_epilogue(double loss, double msum, const double (&extra)[NX], float* __restrict__ out) {
  const float denom = (float)msum + 1e-8f;  // masked_mean's denominator
  if (EPI == kEpiPolicy) {
    out[0] = (float)loss;
    out[1] = (float)extra[1] / denom;  // pg_clipfrac
    out[2] = (float)extra[0] / denom;  // ppo_kl
    out[3] = (float)extra[NX > 2 ? 2 : 0] / denom;  // pg_clipfrac_lower
  } else if (EPI == kEpiValue) {
    out[0] = 0.5f * (float)loss;
    out[1] = (float)extra[0] / denom;
  } else {
    out[0] = (float)loss;
  }
}

template <int NV, int EPI>
__global__ __launch_bounds__(kFoldThreads) void fold_loss_kernel(const double* __restrict__ records, int64_t rows,
                                                                 int chunks, int64_t cols, AggParams ap,
                                                                 float* __restrict__ coef, float* __restrict__ out) {
  __shared__ double smem[(NV + 3) * (kFoldThreads / 64)];
  double loss, msum, extra[NV > 2 ? NV - 2 : 1];
  finalize_agg<NV, kFoldThreads, false>(records, rows, chunks, cols, ap, coef, loss, msum, extra, smem);
  if (threadIdx.x == 0) loss_epilogue<EPI>(loss, msum, extra, out);
}

}  // namespace vamd
