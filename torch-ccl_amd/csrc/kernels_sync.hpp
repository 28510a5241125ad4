// Cross-rank synchronisation on device flags: what the reference does with its one-thread sync
// kernels between the data kernels of the large allreduce (src/gpu/allreduce.h:731-769, 835-877)
// and with the rank barrier inside the small one (src/gpu/allreduce_small.h:193-273).
//
// A rank owns one 64-bit flag word in device memory that its peers can address (their own mapping
// of the same allocation).  The barrier is one wavefront: lane 0 publishes this rank's epoch, lane r
// then polls rank r's word until it has reached the epoch.  Epochs only grow, so a word never has
// to be cleared and a late reader can never miss a value.  What makes the data of the earlier
// kernels of the stream visible to the peers is the kernel boundary (writes of a finished kernel
// are written back, a starting kernel begins with invalidated caches); the flag itself travels with
// system-scope release / acquire accesses.
//
// Every wait is bounded: a lane that has polled for `limit_ticks` ticks of the 100 MHz wall clock
// records the rank it was waiting for and the kernel returns.  No host thread is involved and no
// wavefront can spin for good.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels_common.hpp"
#include "mccl.h"

namespace {

constexpr int kSyncRanks = MCCL_MAX_RANKS;  // one lane per rank

struct BarrierArgs {
  uint64_t* flag[kSyncRanks];
  uint64_t epoch;
  uint64_t limit_ticks;
  uint32_t* status;  // status[0] = 1 + rank that was late, status[1] = low half of the epoch; null = not reported
  int n;
  int rank;
};

// A barrier of at most 8 ranks travels in an argument block below the size at which launches get
// slower (see LeanReduceArgs).
constexpr int kLeanSyncRanks = 8;
struct LeanBarrierArgs {
  uint64_t* flag[kLeanSyncRanks];
  uint64_t epoch;
  uint64_t limit_ticks;
  uint32_t* status;
  int n;
  int rank;
};
static_assert(sizeof(LeanBarrierArgs) <= 104, "lean barrier arguments must stay below the launch-cost step");

// 16 bytes written through to memory / read past the caches (system scope), as two 64-bit accesses
// the compiler keeps track of.  For data that a wavefront of another rank (or another workgroup of
// this kernel) produces or consumes while this kernel runs: coherence per access instead of a
// cache-wide write-back or invalidate per tile, which with thousands of tiles and several
// processes on the GPU costs far more than the data movement itself.
__device__ __forceinline__ void store_vec_coherent(u32x4* p, u32x4 x) {
  uint64_t* q = (uint64_t*)p;
  __hip_atomic_store(q, (uint64_t)x.x | ((uint64_t)x.y << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(q + 1, (uint64_t)x.z | ((uint64_t)x.w << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ u32x4 load_vec_coherent(const u32x4* p) {
  const uint64_t* q = (const uint64_t*)p;
  const uint64_t lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const uint64_t hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  return (u32x4){(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}

// The same for a wavefront that walks a tile: `tile` is the same address in every lane, lane l
// accesses tile + off (off below 4 GiB).  One 16-byte access per lane through a buffer descriptor,
// which is how the compiler can be given all three cache bits and still keep count of the access:
// system scope (read past / written through the caches) and, for the load, non-temporal.  The hint
// matters: eight read streams run at 6.5 TB/s with it and at 5.3 without, and as pairs of 8-byte
// accesses at 4.8.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_descriptor(const char* tile) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(tile), 0, -1, 0x00020000);  // raw bytes, no bound
}
constexpr int kAuxSc0 = 1, kAuxNt = 2, kAuxSc1 = 16;
__device__ __forceinline__ u32x4 load_tile_coherent(const char* tile, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(tile_descriptor(tile), off, 0, kAuxSc0 | kAuxSc1 | kAuxNt);
}
// without the non-temporal hint: for bytes that other ranks read as well in the same collective
__device__ __forceinline__ u32x4 load_tile_coherent_keep(const char* tile, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(tile_descriptor(tile), off, 0, kAuxSc0 | kAuxSc1);
}
__device__ __forceinline__ void store_tile_through(char* tile, uint32_t off, u32x4 x) {
  __builtin_amdgcn_raw_buffer_store_b128(x, tile_descriptor(tile), off, 0, kAuxSc0 | kAuxSc1);
}

// 16 bytes written through to memory with one store, at any alignment the element type allows.
// The wait state after it covers a following write of the data registers.
__device__ __forceinline__ void store_vec_through(char* p, u32x4 x) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(p), "v"(x) : "memory");
}

// Everything this wavefront has stored has reached its destination (for written-through stores:
// memory) -- what has to hold before a flag that announces the data is stored.
__device__ __forceinline__ void wait_own_stores() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Stores a flag that announces what this wavefront has stored before it.  Those stores are written
// through and have been acknowledged (wait_own_stores); what earlier kernels of the stream wrote is in
// memory since they ended.  A release of system scope on the store itself would add a write-back of
// the whole L2 the wavefront happens to run on -- other processes' lines included -- and make the
// peers wait for it.
__device__ __forceinline__ void publish_flag64(uint64_t* word, uint64_t value) {
  wait_own_stores();
  __hip_atomic_store(word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Pause between two polls of a flag: half a microsecond at first, then about an eighth of the time
// waited so far, up to 40 us.  Thousands of wavefronts of several processes may be polling the
// same few words, past the caches: at a fixed half microsecond the waiting ranks of a collective
// put tens of billions of uncached requests per second on the memory channels that hold the
// words, for as long as a late rank needs -- and slow that rank down while it is at it.
__device__ __forceinline__ void poll_pause(uint64_t waited_ticks) {
  const uint32_t long_naps = (uint32_t)(waited_ticks >> 12);  // one per 41 us waited (100 MHz ticks)
  if (long_naps == 0) {
    __builtin_amdgcn_s_sleep(16);
  } else {
    const uint32_t naps = long_naps < 10u ? long_naps : 10u;
    for (uint32_t i = 0; i < naps; ++i) __builtin_amdgcn_s_sleep(127);  // about 4 us each
  }
}

// Polls *word until it is at least `epoch` (64-bit, monotonic).  Returns false at the time limit.
__device__ __forceinline__ bool wait_flag64(const uint64_t* word, uint64_t epoch, uint64_t limit_ticks) {
  if (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) >= epoch) return true;
  const uint64_t t0 = wall_clock64();
  do {
    const uint64_t waited = wall_clock64() - t0;
    if (waited > limit_ticks) return false;
    poll_pause(waited);
  } while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) < epoch);
  return true;
}

// The same for 32-bit epochs, which wrap: compared as a signed distance.
__device__ __forceinline__ bool wait_flag32(const uint32_t* word, uint32_t epoch, uint64_t limit_ticks) {
  if ((int32_t)(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - epoch) >= 0) return true;
  const uint64_t t0 = wall_clock64();
  do {
    const uint64_t waited = wall_clock64() - t0;
    if (waited > limit_ticks) return false;
    poll_pause(waited);
  } while ((int32_t)(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - epoch) < 0);
  return true;
}

__device__ __forceinline__ void report_late(uint32_t* status, int late_rank, uint32_t epoch_lo) {
  if (!status) return;
  __hip_atomic_store(status + 1, epoch_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(status, (uint32_t)(late_rank + 1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The same two waits folded into a data kernel, so that a collective is ONE launch per rank: with
// several processes on one GPU every launch of a process waits for its turn at the dispatcher
// (on the order of 15-20 us per process), which makes the number of launches per collective the
// cost that matters.
//   begin: workgroup 0 publishes `ready_epoch` in this rank's word ("this rank's stream has reached
//          the collective: its input is complete"); every workgroup waits until all words have
//          reached it.  Workgroups dispatched later find the words set and pass with one load each.
//          What the peers wrote before their launch is in memory by then (a finished kernel's
//          writes are written back), but a stale copy may sit in a cache of this kernel's own: the
//          callers read the peers' buffers past the caches (load_vec_coherent) instead of
//          invalidating per workgroup.
//   end:   every workgroup counts itself out; the last one publishes `done_epoch` ("this rank has
//          finished reading the peers' buffers") and waits until every rank has done the same, so the
//          kernel -- and with it the stream -- does not complete before the peers are done with
//          this rank's buffers.  done_epoch == 0: no closing wait.
// A launch that uses these must fit on the GPU together with the launches of all its peers
// (waiting workgroups occupy their slots): the host caps its grid accordingly.
struct XSync {
  uint64_t* word[kLeanSyncRanks];  // rank r's 64-bit word
  uint64_t ready_epoch;
  uint64_t done_epoch;
  uint32_t* done_count;            // this rank's counters (MCCL_SYNC_COUNTER_BYTES): zero between launches
  uint64_t limit_ticks;
  uint32_t* status;
  int n;
  int rank;
};

// The unit of work of the cross-rank kernels is the wavefront: which one this is, and of how many.
// WPG wavefronts share a workgroup.  One, normally.  kPackedWaves for launches whose waiting
// wavefronts must sit on few compute units (a workgroup lives on one): ranks that share a GPU with
// each other's other kernels.  The wavefronts of a workgroup never depend on each other; they meet
// once, in xsync_end.
struct Wave {
  uint32_t lane;
  uint32_t index;  // uniform
  uint32_t count;  // uniform
};
constexpr int kPackedWaves = 16;

template <int WPG>
__device__ __forceinline__ Wave this_wave() {
  if constexpr (WPG == 1) {
    return Wave{threadIdx.x, blockIdx.x, gridDim.x};
  } else {
    const uint32_t in_group = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    return Wave{threadIdx.x % kWave, blockIdx.x * WPG + in_group, gridDim.x * WPG};
  }
}

constexpr uint32_t kDoneGroups = 16;
// 32-bit words between two counters: 256 bytes.  Counters on neighbouring 64-byte lines still got in
// each other's way (a shard reduction of 8 x 64 MiB with one workgroup per tile: 104 us with the
// counters 64 bytes apart, 93 us at 256 bytes and beyond, 90 us without any counting).
constexpr uint32_t kDoneStride = 64;
static_assert(kDoneGroups * kDoneStride * 4 <= MCCL_SYNC_COUNTER_BYTES, "counters must fit the block the caller provides");
static_assert(kDoneGroups <= kWave, "one lane of the watching wavefront per counter");
// A word of the same block that the closing count leaves alone (128 bytes into the first counter's
// 256): counts the workgroups of a one-launch all-to-all whose share of the copy-in is done.
constexpr uint32_t kStagedCountWord = 32;

// Returns false (for the whole wavefront) when a peer did not arrive in time.
// publish = false: the kernel stores this rank's word itself, once something else has happened first.
__device__ __forceinline__ bool xsync_begin(const XSync& x, bool publish = true) {
  if (x.ready_epoch == 0) return true;  // the caller has ordered the ranks on the host
  const int lane = threadIdx.x & (kWave - 1);
  if (publish && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0)
    publish_flag64(x.word[x.rank], x.ready_epoch);
  bool ok = true;
  // (publish = false: this rank's own word says that all its workgroups are through with what comes
  // before -- waited for like the peers')
  if (lane < x.n && (lane != x.rank || !publish)) {
    ok = wait_flag64(x.word[lane], x.ready_epoch, x.limit_ticks);
    if (!ok) report_late(x.status, lane, (uint32_t)x.ready_epoch);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // nothing below moves above the wait
  return __builtin_amdgcn_ballot_w64(!ok) == 0;
}

// Call once per workgroup, by all its lanes, after the workgroup's last access to a peer's buffer.
//
// Every workgroup counts itself out with an atomic add whose result nobody reads: the wavefront
// does not wait for it and ends.  The counting is spread over sixteen counters on cache lines of
// their own, 256 bytes apart (atomics on one address are carried out one after the other, about 7 ns
// each).  The
// workgroup with the highest index -- dispatched last, so that it holds its slot for the shortest
// time -- watches the counters, one lane each, until every workgroup of the launch is out, clears
// them for the next launch, publishes the closing epoch and waits for the peers'.  No workgroup
// depends on the watching one, so the order in which the hardware starts workgroups only decides
// how long that one wavefront stays.  (Counting with a returned value, so that the last workgroup
// out could tell, kept every workgroup for the round trip of its atomic: with one tile per workgroup
// that doubled the duration of a 64 MiB shard reduction.)
//
// wrote_to_peers: the kernel stores into the peers' buffers (written through), and the closing epoch
// also says that those stores have arrived; a kernel that only reads them (its loads have returned
// once their values were used) does not wait for the stores into its own output, which the end of
// the kernel covers -- a wavefront that waits for its stores keeps its slot for their whole way to
// memory, and a launch of fresh workgroups lives on slots turning over.
__device__ __forceinline__ void xsync_end(const XSync& x, uint32_t workgroups, bool wrote_to_peers = true) {
  if (x.done_epoch == 0) return;
  if (wrote_to_peers) wait_own_stores();  // (no cache needs writing back: the stores were written through)
  else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x >= kWave) return;  // the first wavefront of the workgroup does the rest
  const uint32_t lane = threadIdx.x;
  const uint32_t groups = workgroups < kDoneGroups ? workgroups : kDoneGroups;
  // Relaxed: the ordering that matters (this workgroup's accesses are complete) was established
  // above, and an acquire-release atomic would add a cache write-back and invalidate per workgroup.
  if (lane == 0) (void)__hip_atomic_fetch_add(x.done_count + kDoneStride * (blockIdx.x % groups), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (blockIdx.x != workgroups - 1) return;
  // lane g watches counter g: workgroups g, g + groups, ... count there
  const uint32_t members = lane < groups ? (workgroups - lane + groups - 1) / groups : 0u;
  const uint64_t t0 = wall_clock64();
  for (;;) {
    const uint32_t c = lane < groups ? __hip_atomic_load(x.done_count + kDoneStride * lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    if (__builtin_amdgcn_ballot_w64(c != members) == 0) break;
    if (wall_clock64() - t0 > x.limit_ticks) {  // (a workgroup of this launch never ended: reported as this rank itself)
      if (lane == 0) report_late(x.status, x.rank, (uint32_t)x.done_epoch);
      return;
    }
    __builtin_amdgcn_s_sleep(4);
  }
  if (lane < groups) __hip_atomic_store(x.done_count + kDoneStride * lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  if (lane == 0) publish_flag64(x.word[x.rank], x.done_epoch);
  if ((int)lane < x.n && (int)lane != x.rank) {
    if (!wait_flag64(x.word[lane], x.done_epoch, x.limit_ticks)) report_late(x.status, lane, (uint32_t)x.done_epoch);
  }
}

// The barrier that also carries every rank's offer for the coming collective and resolves the
// peers' offers against this rank's table of mapped allocations.
struct OfferBarrierArgs {
  uint64_t* flag[MCCL_OFFER_RANKS];
  uint64_t* offer[MCCL_OFFER_RANKS];  // rank r's offer slot (four 64-bit words)
  uint64_t epoch;
  uint64_t limit_ticks;
  uint32_t* status;
  uint64_t mine[4];                   // this rank's offer, as the words of an mccl_offer_t
  uint64_t my_buffer;
  const mccl_import_table_t* imports;
  uint64_t* resolved;
  int n;
  int rank;
};

// This rank's offer into its slot (by the one thread that stores the rank's flag afterwards).
__device__ __forceinline__ void publish_offer(uint64_t* slot, const uint64_t (&mine)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) __hip_atomic_store(slot + i, mine[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Where rank `r`'s buffer is in this rank's address space, from the offer in its slot (read after
// its flag has arrived) and this rank's table of mappings; 0 when this rank has not mapped it.
__device__ __forceinline__ uint64_t resolve_offer(const uint64_t* slot, const mccl_import_table_t* imports, int r) {
  const uint64_t w0 = __hip_atomic_load(slot + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const uint64_t gen = __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const uint64_t off = __hip_atomic_load(slot + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  const uint32_t entry = (uint32_t)w0, which = (uint32_t)(w0 >> 32);
  if (entry == MCCL_OFFER_STAGED) {
    const uint64_t b = imports->staging[r][which & (MCCL_OFFER_SLOTS - 1u)];
    return b ? b + off : 0;
  }
  if (entry < MCCL_OFFER_ENTRIES) {
    const uint64_t b = imports->base[r][entry];
    if (b && imports->generation[r][entry] == gen) return b + off;
  }
  return 0;
}

__global__ __launch_bounds__(kWave) void rank_barrier_offers_kernel(const OfferBarrierArgs a) {
  const int lane = threadIdx.x;
  if (lane == 0) {
    // the offer first, then the flag that says it is there
    publish_offer(a.offer[a.rank], a.mine);
    publish_flag64(a.flag[a.rank], a.epoch);
  }
  if (lane >= a.n) return;
  uint64_t where = a.my_buffer;
  if (lane != a.rank) {
    where = 0;
    if (!wait_flag64(a.flag[lane], a.epoch, a.limit_ticks)) {
      report_late(a.status, lane, (uint32_t)a.epoch);
    } else {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the offer is read after the flag
      where = resolve_offer(a.offer[lane], a.imports, lane);
      if (!where) report_late(a.status, lane, MCCL_STATUS_UNMAPPED);
    }
  }
  a.resolved[lane] = where;
}

// The barrier of a collective in which every rank hands every peer a different piece: a rank
// publishes a row of offers (entry k: the piece for rank k, and its length) and resolves the column
// addressed to it.
struct OfferEachArgs {
  uint64_t* flag[MCCL_OFFER_RANKS];
  uint64_t* row[MCCL_OFFER_RANKS];    // rank r's row of n offers, four 64-bit words each
  uint64_t epoch;
  uint64_t limit_ticks;
  uint32_t* status;
  uint64_t mine[MCCL_OFFER_RANKS][4];  // this rank's row
  uint64_t expect[MCCL_OFFER_RANKS];   // bytes this rank expects from rank r
  uint64_t my_source;
  const mccl_import_table_t* imports;
  uint64_t* resolved;
  int n;
  int rank;
};

// Where rank r's piece for this rank is, from r's offer for this rank (read after r's flag has
// arrived): null when it is empty, not of the expected length, or in memory this rank has not mapped
// (the latter two reported).
__device__ __forceinline__ uint64_t resolve_piece(const uint64_t* slot, uint64_t expect, const mccl_import_table_t* imports, int r,
                                                  uint32_t* status) {
  const uint64_t bytes = __hip_atomic_load(slot + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  if (bytes != expect) {
    report_late(status, r, MCCL_STATUS_MISMATCH);
    return 0;
  }
  if (bytes == 0) return 0;
  const uint64_t where = resolve_offer(slot, imports, r);
  if (!where) report_late(status, r, MCCL_STATUS_UNMAPPED);
  return where;
}

__global__ __launch_bounds__(kWave) void rank_barrier_offers_each_kernel(const OfferEachArgs a) {
  const int lane = threadIdx.x;
  if (lane == 0) {
    // the whole row by the thread that stores the flag after it (its release covers them)
    uint64_t* row = a.row[a.rank];
#pragma unroll
    for (int k = 0; k < MCCL_OFFER_RANKS; ++k) {
      if (k < a.n) {
#pragma unroll
        for (int i = 0; i < 4; ++i) __hip_atomic_store(row + 4 * k + i, a.mine[k][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
    publish_flag64(a.flag[a.rank], a.epoch);
  }
  if (lane >= a.n) return;
  uint64_t where = a.my_source;
  if (lane != a.rank) {
    where = 0;
    if (!wait_flag64(a.flag[lane], a.epoch, a.limit_ticks)) {
      report_late(a.status, lane, (uint32_t)a.epoch);
    } else {
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the offer is read after the flag
      where = resolve_piece(a.row[lane] + 4 * a.rank, a.expect[lane], a.imports, lane, a.status);
    }
  }
  a.resolved[lane] = where;
}

// Stream-ordered update of the table that rank_barrier_offers_kernel resolves against: one lane
// per update, the values are kernel arguments.
struct ImportUpdateArgs {
  mccl_import_table_t* table;
  mccl_import_update_t update[MCCL_IMPORT_UPDATES];
  int n;
};

__global__ __launch_bounds__(kWave) void import_table_update_kernel(const ImportUpdateArgs a) {
  const int lane = threadIdx.x;
  if (lane >= a.n) return;
  const mccl_import_update_t u = a.update[lane];
  if (u.entry == MCCL_OFFER_STAGED) {
    a.table->staging[u.rank][u.slot & (MCCL_OFFER_SLOTS - 1u)] = u.base;
  } else {
    a.table->generation[u.rank][u.entry] = u.generation;
    a.table->base[u.rank][u.entry] = u.base;
  }
}

template <typename ARGS>
__global__ __launch_bounds__(kWave) void rank_barrier_kernel(const ARGS a) {
  const int lane = threadIdx.x;
  if (lane == 0) publish_flag64(a.flag[a.rank], a.epoch);
  if (lane < a.n && lane != a.rank) {
    if (!wait_flag64(a.flag[lane], a.epoch, a.limit_ticks)) report_late(a.status, lane, (uint32_t)a.epoch);
  }
}

}  // namespace
