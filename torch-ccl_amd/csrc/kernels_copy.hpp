// Segmented copy kernel: the data movement of allgather / alltoall(v) (ccl::allgatherv,
// ccl::alltoall(v): src/gpu/dpcpp_ccl.cpp:1176-1182, 1403-1455) and of the pack / unpack loops
// (src/gpu/dpcpp_ccl.cpp:1505-1538).
#pragma once

#include "kernels_common.hpp"
#include "kernels_sync.hpp"

namespace {

// One segment as the kernel sees it.  The host splits it into a head (bytes up to the first
// 128-byte boundary of dst: the body starts on a cache line), `nfull` chunks of kCopyChunk bytes and one last chunk of `last`
// bytes, so that the device needs 32-bit uniform arithmetic only.
struct CopySeg {
  const char* src;
  char* dst;
  uint32_t head;   // bytes before the body
  uint32_t nfull;  // full chunks in the body
  uint32_t last;   // bytes of the final partial chunk (0 = none)
  uint32_t pad_;
};

struct CopyArgs {
  CopySeg seg[kMaxSegs];
  uint32_t chunk_prefix[kMaxSegs + 1];  // exclusive prefix sum of chunks per segment
  int nseg;
};

// The same plus the cross-rank waits of a one-launch collective between rank processes: the
// sources are the peers' buffers, complete once every rank has reached the collective.
struct SyncCopyArgs {
  CopyArgs copy;
  XSync sync;
  uint32_t invalidate;  // some bytes are read through the caches: invalidate once per workgroup first
  uint32_t shared;      // other ranks read the same sources: leave them in the memory-side cache
  // INDIRECT kernel: segment s is read from src_table[src_rank[s]] + (its src taken as a byte offset)
  // when src_rank[s] >= 0 -- the table a barrier kernel in front has resolved the ranks' offers into
  const uint64_t* src_table;
  int8_t src_rank[kMaxSegs];
};

// Where the sources of the segments are when the host does not know: a table in memory (INDIRECT 1),
// or lane r of the wavefront holds rank r's address (INDIRECT 2).
struct CopySources {
  const uint64_t* table;
  const int8_t* rank;
  uint64_t held;
};

// A copy of at most MCCL_OFFER_RANKS segments: the same as CopyArgs to the kernels, an eighth of it to the launch.
struct LeanCopyArgs {
  CopySeg seg[MCCL_OFFER_RANKS];
  uint32_t chunk_prefix[MCCL_OFFER_RANKS + 1];
  int nseg;
};

// Segmented copy.  One wavefront per workgroup, one 2 KiB chunk per wavefront, chunks
// handed out in order.  The body moves as 16-byte vectors aligned on dst (non-temporal both
// ways for full chunks); a source that is not congruent with dst mod 16 is read with unaligned
// vector loads.
// COHERENT: the sources are buffers of other ranks, complete in memory but possibly stale in this
// kernel's caches: 8-byte aligned sources are read past the caches (the host requests a cache
// invalidate per workgroup for the others).
// UNROLL: 16-byte vectors per lane per chunk (chunk = 64 x 16 x UNROLL bytes; the host computes
// the segment geometry for the same value).  STREAM: full chunks are written through past the
// caches (`sc1`) instead of with the non-temporal hint.
// THROUGH: every store is written through to memory (for readers in other processes that are running at
// the same time and are told by a flag), not only the full chunks.
template <bool COHERENT, int UNROLL, bool STREAM, int INDIRECT = 0, typename ARGS = CopyArgs, bool THROUGH = false>
__device__ __forceinline__ void copy_segments_body(const ARGS& a, const Wave& w, bool shared_sources = false,
                                                   const CopySources from = CopySources{nullptr, nullptr, 0}) {
  constexpr uint32_t CHUNK = (uint32_t)kWave * 16u * UNROLL;
  const uint32_t total = a.chunk_prefix[a.nseg];
  for (uint32_t chunk = w.index; chunk < total; chunk += w.count) {
    // binary search: largest s with chunk_prefix[s] <= chunk
    int lo = 0, hi = a.nseg;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (a.chunk_prefix[mid] <= chunk) lo = mid; else hi = mid;
    }
    const uint32_t c = chunk - a.chunk_prefix[lo];
    const uint32_t head = a.seg[lo].head;
    const uint32_t nfull = a.seg[lo].nfull;
    const uint32_t len = (c < nfull) ? CHUNK : a.seg[lo].last;
    const uint32_t t = w.lane;
    const char* src = a.seg[lo].src;
    char* dst = a.seg[lo].dst;
    if constexpr (INDIRECT != 0) {
      const int r = from.rank[lo];  // uniform
      if (r >= 0) {
        uint64_t base;
        if constexpr (INDIRECT == 1) {
          // written by the kernel in front on the stream, constant while this one runs: a scalar load
          base = ((const __attribute__((address_space(4))) uint64_t*)from.table)[r];
        } else {
          const uint32_t lo32 = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)from.held, r);
          const uint32_t hi32 = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(from.held >> 32), r);
          base = ((uint64_t)hi32 << 32) | lo32;
        }
        if (base == 0) continue;  // not resolved: whoever resolved it has reported why
        src = (const char*)(base + (uint64_t)(uintptr_t)src);
      }
    }
    if (c == 0) {
      for (uint32_t i = t; i < head; i += kWave) {  // head < 128
        if constexpr (THROUGH) __hip_atomic_store((unsigned char*)dst + i, (unsigned char)src[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        else dst[i] = src[i];
      }
    }
    const size_t off = (size_t)head + (size_t)c * CHUNK;  // start of this chunk
    src += off;
    dst += off;

    const u32x4_unaligned* sv = (const u32x4_unaligned*)src;
    u32x4* dv = (u32x4*)dst;
    if (len == CHUNK) {
      u32x4 x[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (COHERENT && (((uintptr_t)src) & 7u) == 0)
          x[u] = shared_sources ? load_tile_coherent_keep(src, (t + u * kWave) * 16u) : load_tile_coherent(src, (t + u * kWave) * 16u);
        else x[u] = __builtin_nontemporal_load(&sv[t + u * kWave]);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if constexpr (THROUGH) store_vec_through((char*)&dv[t + u * kWave], x[u]);
        else if constexpr (STREAM) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(&dv[t + u * kWave]), "v"(x[u]) : "memory");
        else __builtin_nontemporal_store(x[u], &dv[t + u * kWave]);
      }
    } else {
      const uint32_t nv = len >> 4;
      for (uint32_t v = t; v < nv; v += kWave) {
        if constexpr (THROUGH) store_vec_through((char*)&dv[v], (u32x4)sv[v]);
        else dv[v] = sv[v];
      }
      const uint32_t rem = len & 15u;
      if (t < rem) {
        if constexpr (THROUGH) __hip_atomic_store((unsigned char*)dst + (nv << 4) + t, (unsigned char)src[(nv << 4) + t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        else dst[(nv << 4) + t] = src[(nv << 4) + t];
      }
    }
  }
}

template <int UNROLL, bool STREAM>
__global__ __launch_bounds__(kWave) void copy_segments_kernel(const CopyArgs a) {
  copy_segments_body<false, UNROLL, STREAM>(a, this_wave<1>());
}

template <int WPG>
__global__ __launch_bounds__(kWave * WPG) void copy_segments_sync_kernel(const SyncCopyArgs a) {
  if (xsync_begin(a.sync)) {
    // heads, partial chunks and misaligned sources go through the caches
    if (a.invalidate) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
    copy_segments_body<true, kCopyUnroll, false>(a.copy, this_wave<WPG>(), a.shared != 0);
  }
  xsync_end(a.sync, gridDim.x);
}

// The same behind a barrier kernel that has resolved where the sources are: no opening wait, and the
// peers' data were complete before this kernel started, so the loads go through the caches like any
// copy's (they start clean at a kernel boundary) and the launch has the plain copy's geometry --
// one chunk per workgroup -- plus the closing count.
template <bool STREAM>
__global__ __launch_bounds__(kWave) void copy_segments_resolved_kernel(const SyncCopyArgs a) {
  copy_segments_body<false, kCopyUnroll, STREAM, 1>(a.copy, this_wave<1>(), false, CopySources{a.src_table, a.src_rank, 0});
  xsync_end(a.sync, gridDim.x, /*wrote_to_peers=*/false);
}

// An all-to-all between rank processes as ONE launch, on few compute units (every launch of a process
// waits for its turn at the dispatcher, which at small sizes costs more than the data).  The pieces
// this rank does not offer in place go into its outboxes first, by all workgroups; when the last
// of them is there -- counted in a word of the rank's counter block, which only this launch touches
// then -- the first workgroup publishes the rank's row of offers and its flag.  Every workgroup waits
// for all flags, this rank's own included (the pulls may write where the copies read: an output that
// overlaps the input), every wavefront resolves the column addressed to this rank (lane r: rank r's
// piece) and they pull.  The outboxes are written and read past the caches of the two kernels, which
// run at the same time.
struct ExchangeArgs {
  LeanCopyArgs stage;                  // this rank's pieces -> its outboxes
  LeanCopyArgs pull;                   // the peers' pieces -> this rank's output; src = offset from the resolved address
  int8_t src_rank[MCCL_OFFER_RANKS];   // of the pull segments (< 0: src is an address as it stands)
  uint64_t* row[MCCL_OFFER_RANKS];
  uint64_t mine[MCCL_OFFER_RANKS][4];
  uint64_t expect[MCCL_OFFER_RANKS];
  uint64_t my_source;
  const mccl_import_table_t* imports;
  uint32_t* staged_count;              // zero between launches
  uint32_t invalidate;                 // a pull has a head or a partial chunk, or an odd offset: those bytes go through the caches
  XSync sync;
};

template <int WPG>
__global__ __launch_bounds__(kWave * WPG) void exchange_offers_kernel(const ExchangeArgs a) {
  const Wave w = this_wave<WPG>();
  const int n = a.sync.n, me = a.sync.rank;
  const bool staging = a.stage.nseg != 0;  // (nothing to copy: the row and the flag go out at once, as in every other one-launch form)
  if (staging) {
    copy_segments_body<false, kCopyUnroll, false, 0, LeanCopyArgs, /*THROUGH=*/true>(a.stage, w);
    // what this workgroup has put into the outboxes -- written through -- is in memory before it counts
    // itself in (a release fence of system scope instead would write back all of the L2 this workgroup
    // runs on, other processes' lines included)
    wait_own_stores();
    __syncthreads();
    if (threadIdx.x == 0) (void)__hip_atomic_fetch_add(a.staged_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (staging) {
      const uint64_t t0 = wall_clock64();
      while (__hip_atomic_load(a.staged_count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != gridDim.x) {
        if (wall_clock64() - t0 > a.sync.limit_ticks) {  // (a workgroup of this launch never got there: reported as this rank itself)
          report_late(a.sync.status, me, (uint32_t)a.sync.ready_epoch);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the flag below stays below the count (the copies were written through: no cache to invalidate)
      __hip_atomic_store(a.staged_count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
    }
    uint64_t* row = a.row[me];
#pragma unroll
    for (int k = 0; k < MCCL_OFFER_RANKS; ++k) {
      if (k < n) {
#pragma unroll
        for (int i = 0; i < 4; ++i) __hip_atomic_store(row + 4 * k + i, a.mine[k][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
    publish_flag64(a.sync.word[me], a.sync.ready_epoch);
  }
  if (xsync_begin(a.sync, /*publish=*/false)) {  // (publish = false also makes it wait for this rank's own flag)
    uint64_t where = a.my_source;
    const int r = (int)w.lane;
    if (r >= n) where = 0;
    else if (r != me) where = resolve_piece(a.row[r] + 4 * me, a.expect[r], a.imports, r, a.sync.status);
    // Full chunks of 8-byte aligned sources are read past the caches; whatever else there is (heads,
    // partial chunks, sources at odd addresses) is read through them, after an invalidate -- only then:
    // with several processes on the GPU an invalidate is everybody's loss.
    if (a.invalidate || __builtin_amdgcn_ballot_w64((where & 7u) != 0) != 0) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
    copy_segments_body<true, kCopyUnroll, false, 2, LeanCopyArgs>(a.pull, w, false, CopySources{nullptr, a.src_rank, where});
  }
  xsync_end(a.sync, gridDim.x, /*wrote_to_peers=*/false);
}

// allgather as pushes: this rank's contribution goes into every rank's output in one pass -- read
// once, written ndst times -- where pulls make every rank read all contributions (W reads of every
// byte over the group, served by the memory-side cache only while the ranks keep in step).  The
// peers' outputs are written through, like the shards of the in-place allreduce, so that the closing
// epoch tells their owners that the data is there.  Any alignment: vectors are 16 bytes of the
// message, wherever source and destinations start; the bytes after the last vector go one per lane.
struct FanoutArgs {
  const char* src;
  char* dst[kLeanSyncRanks];
  uint32_t nvec;     // whole 16-byte vectors
  uint32_t tail;     // bytes after them (< 16)
  uint32_t tiles;    // 1 KiB tiles that cover the vectors
  uint32_t aligned;  // every destination is 16-byte aligned
  int ndst;
  // The destinations from device memory instead (INDIRECT kernels): rank k's buffer + dst_off, for
  // every rank k < sync.n whose bit is set in dst_mask -- resolved by the barrier kernel in front
  // (dst_table), or from the ranks' offers by this launch itself (offer / mine / imports / my_buffer).
  const uint64_t* dst_table;
  uint64_t dst_off;
  uint32_t dst_mask;
  uint64_t* offer[kLeanSyncRanks];
  uint64_t mine[4];
  const mccl_import_table_t* imports;
  uint64_t my_buffer;
  XSync sync;
};

struct FanoutDst {  // only ever indexed with constants: scalar registers
  char* p[kLeanSyncRanks];
};

__device__ __forceinline__ u32x4 fanout_load(const FanoutArgs& a, uint32_t tile, uint32_t lane) {
  const uint32_t v = tile * kWave + lane;  // the host keeps tiles * 64 below 2^32
  if (v >= a.nvec) return (u32x4){0u, 0u, 0u, 0u};
  return __builtin_nontemporal_load(&((const u32x4_unaligned*)a.src)[v]);
}

__device__ __forceinline__ void fanout_store(const FanoutArgs& a, uint32_t tile, uint32_t lane, u32x4 x) {
  if (tile * kWave + lane >= a.nvec) return;
#pragma unroll
  for (int k = 0; k < kLeanSyncRanks; ++k) {
    if (k < a.ndst) {
      char* tb = a.dst[k] + (size_t)tile * (kWave * 16u);  // uniform
      if (a.aligned) store_tile_through(tb, lane * 16u, x);
      else store_vec_through(tb + lane * 16u, x);
    }
  }
}

// The same with the destinations in `d` (any alignment), those whose bit is set in the mask.
__device__ __forceinline__ void fanout_store_to(const FanoutArgs& a, const FanoutDst& d, uint32_t tile, uint32_t lane, u32x4 x) {
  if (tile * kWave + lane >= a.nvec) return;
#pragma unroll
  for (int k = 0; k < kLeanSyncRanks; ++k)
    if (a.dst_mask & (1u << k)) store_vec_through(d.p[k] + (size_t)tile * (kWave * 16u) + lane * 16u, x);
}

// INDIRECT 1: behind a barrier kernel that has resolved the ranks' offers; INDIRECT 2: the launch
// exchanges the offers itself (see xrank_reduce_kernel).
template <int WPG, int INDIRECT>
__global__ __launch_bounds__(kWave * WPG) void fanout_indirect_kernel(const FanoutArgs a) {
  const Wave w = this_wave<WPG>();
  const int n = a.sync.n;
  FanoutDst d;
  bool resolved = true;
  if constexpr (INDIRECT == 1) {
    const auto* table = (const __attribute__((address_space(4))) uint64_t*)a.dst_table;
#pragma unroll
    for (int k = 0; k < kLeanSyncRanks; ++k) {
      const uint64_t p = table[k];
      if (k < n) resolved = resolved && p != 0;
      d.p[k] = (char*)(p + a.dst_off);
    }
  } else {
    if (blockIdx.x == 0 && threadIdx.x == 0) publish_offer(a.offer[a.sync.rank], a.mine);  // before xsync_begin stores this rank's flag
  }
  bool begun = resolved && xsync_begin(a.sync);
  if constexpr (INDIRECT == 2) {
    if (begun) {
      uint64_t where = a.my_buffer;
      const int r = (int)w.lane;
      if (r < n && r != a.sync.rank) {
        where = resolve_offer(a.offer[r], a.imports, r);
        if (!where) report_late(a.sync.status, r, MCCL_STATUS_UNMAPPED);
      }
      begun = __builtin_amdgcn_ballot_w64(r < n && where == 0) == 0;
      where += a.dst_off;
#pragma unroll
      for (int k = 0; k < kLeanSyncRanks; ++k) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)where, k);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(where >> 32), k);
        d.p[k] = (char*)(((uint64_t)hi << 32) | lo);
      }
    } else {
#pragma unroll
      for (int k = 0; k < kLeanSyncRanks; ++k) d.p[k] = nullptr;
    }
  }
  if (begun) {
    const uint32_t T = a.tiles, G = w.count;
    for (uint32_t t0 = w.index; t0 < T; t0 += 2 * G) {  // two tiles' loads in flight
      const uint32_t t1 = t0 + G;
      const u32x4 x0 = fanout_load(a, t0, w.lane);
      u32x4 x1 = (u32x4){0u, 0u, 0u, 0u};
      if (t1 < T) x1 = fanout_load(a, t1, w.lane);
      fanout_store_to(a, d, t0, w.lane, x0);
      if (t1 < T) fanout_store_to(a, d, t1, w.lane, x1);
    }
    if (a.tail && w.index == w.count - 1 && w.lane < a.tail) {
      const size_t i = (size_t)a.nvec * 16u + w.lane;
      const unsigned char b = (unsigned char)a.src[i];
#pragma unroll
      for (int k = 0; k < kLeanSyncRanks; ++k)
        if (a.dst_mask & (1u << k)) __hip_atomic_store((unsigned char*)d.p[k] + i, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  xsync_end(a.sync, gridDim.x);
}

template <int WPG>
__global__ __launch_bounds__(kWave * WPG) void fanout_sync_kernel(const FanoutArgs a) {
  const Wave w = this_wave<WPG>();
  if (xsync_begin(a.sync)) {
    const uint32_t T = a.tiles, G = w.count;
    for (uint32_t t0 = w.index; t0 < T; t0 += 2 * G) {  // two tiles' loads in flight
      const uint32_t t1 = t0 + G;
      const u32x4 x0 = fanout_load(a, t0, w.lane);
      u32x4 x1 = (u32x4){0u, 0u, 0u, 0u};
      if (t1 < T) x1 = fanout_load(a, t1, w.lane);
      fanout_store(a, t0, w.lane, x0);
      if (t1 < T) fanout_store(a, t1, w.lane, x1);
    }
    if (a.tail && w.index == w.count - 1 && w.lane < a.tail) {
      const size_t i = (size_t)a.nvec * 16u + w.lane;
      const unsigned char b = (unsigned char)a.src[i];
#pragma unroll
      for (int k = 0; k < kLeanSyncRanks; ++k)
        if (k < a.ndst) __hip_atomic_store((unsigned char*)a.dst[k] + i, b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  xsync_end(a.sync, gridDim.x);
}

}  // namespace
