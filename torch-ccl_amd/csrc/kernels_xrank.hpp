// One-launch reductions between rank processes that read the peers' tensors in place.
//
// With several processes on one GPU every kernel launch of a process waits for its turn at the
// dispatcher, so a collective made of five launches (barrier, reduce, barrier, gather, barrier)
// costs five turns per rank.  This kernel is the whole collective in one launch:
//
//   begin    every rank's input is complete (xsync_begin: the launch itself says "my stream has
//            reached the collective"; all workgroups wait for all ranks' words)
//   phase 1  this rank reduces ITS shard of all ranks' tensors (ascending-rank chain, as
//            reduce_vec_kernel) into out1 -- its staging buffer for an allreduce, the caller's
//            output for a reduce_scatter -- and (allreduce) publishes one flag per 4 KiB chunk
//   phase 2  (allreduce) chunk by chunk, all finished shards are copied from the owners' staging
//            buffers into the caller's tensor; a chunk waits for its owner's flag only
//   end      (reduce_scatter) xsync_end: nobody's kernel completes before all ranks are done reading
//
// which is the two-shot allreduce of the reference's large path (reduce-scatter through scratch,
// then all-gather: src/gpu/allreduce.h:306-533) without its nine launches.  The allreduce needs no
// closing wait: a rank's tensor is read by phase 1 of the shard owners only, chunk (q, c) of it is
// overwritten by this rank's phase 2 only after owner q has published flag c, and this rank's
// kernel ends only when it has copied -- hence seen the flag of -- every chunk of every owner.
//
// The grid is persistent and small enough that the launches of all ranks are resident together
// (waiting workgroups hold their slots); phase 1 never waits for anything but `begin`, so every
// flag a phase 2 waits for is always on its way.  All waits are bounded.
#pragma once

#include "kernels_common.hpp"
#include "kernels_fused.hpp"
#include "kernels_sync.hpp"

namespace {

constexpr int kXRanks = kLeanSyncRanks;
constexpr uint32_t kXTileBytes = kWave * 16;  // 1 KiB: one vector per lane
// Tiles per flag of the allreduce: a wavefront reduces this many consecutive tiles, waits once for
// its (written-through) stores and publishes one flag; waiting and publishing per tile would put a
// store round trip between every two tiles.
constexpr uint32_t kXChunkTiles = MCCL_SYNC_FLAG_BYTES / kXTileBytes;

// All extents are 32-bit and precomputed by the host: the device does no uniform 64-bit compares.
struct XRankArgs {
  const char* in[kXRanks];            // phase 1 inputs in rank order, already at this rank's shard
  char* out1;                         // phase 1 output
  uint32_t* my_flags;                 // phase 1 publishes my_flags[c] = tile_epoch per chunk of tiles (null: no flags)
  uint32_t nvec1;                     // phase 1: whole vectors ...
  uint32_t tail1;                     // ... and elements after them (< elements per vector)
  uint32_t tiles1;                    // tiles that cover both
  uint32_t tile_epoch;
  // phase 2: shard q of the message is copied from shard_src[q] to shard_dst[q], chunk c of it once
  // shard_flags[q][c] has reached tile_epoch
  const char* shard_src[kXRanks];
  const uint32_t* shard_flags[kXRanks];
  char* shard_dst[kXRanks];
  uint32_t full2[kXRanks];            // whole tiles of shard q
  uint32_t last2[kXRanks];            // bytes of the partial tile after them (0: none)
  uint32_t tiles2;                    // tiles of the longest shard; 0 = no phase 2
  uint32_t stream_out;                // write out1 past the caches (large reduce_scatter outputs)
  uint32_t aligned_in;                // every in[k] is 8-byte aligned: read past the caches
  XSync sync;
};

// A vector of a peer's tensor: past the caches when the tensor is 8-byte aligned (always, for whole
// tensors out of an allocator), else as an ordinary unaligned load after a cache invalidate the
// host asked for (aligned_in == 0 makes the kernel invalidate once per workgroup).
__device__ __forceinline__ u32x4 load_in(const char* base, uint32_t v, uint32_t aligned) {
  if (aligned) return load_vec_coherent(&((const u32x4*)base)[v]);
  return __builtin_nontemporal_load(&((const u32x4_unaligned*)base)[v]);
}

template <int DT, int OP>
__device__ __forceinline__ void xrank_reduce_tile(const XRankArgs& a, uint32_t tile, int n) {
  using S = typename Elem<DT>::store_t;
  using A = typename Elem<DT>::acc_t;
  constexpr int VE = vec_elems<DT>();
  const int lane = threadIdx.x;
  const uint32_t v = tile * kWave + (uint32_t)lane;  // the host keeps tiles1 * 64 below 2^32
  const bool whole = v < a.nvec1;
  const bool part = v == a.nvec1 && a.tail1 != 0;
  if (whole || part) {
    VecU<DT> x[kXRanks];
#pragma unroll
    for (int k = 0; k < kXRanks; ++k) {
      if (k < n) {
        x[k].v = (u32x4){0u, 0u, 0u, 0u};
        if (whole) {
          x[k].v = load_in(a.in[k], v, a.aligned_in);
        } else {
#pragma unroll
          for (int e = 0; e < VE; ++e)  // static indices: the vectors stay in registers
            if ((uint32_t)e < a.tail1) vec_set<DT>(x[k], e, ((const S*)a.in[k])[(size_t)v * VE + e]);
        }
      }
    }
    A acc[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[e] = chain_first<DT, OP>(Elem<DT>::load(vec_get<DT>(x[0], e)));
#pragma unroll
    for (int k = 1; k < kXRanks; ++k) {
      if (k < n) {
#pragma unroll
        for (int e = 0; e < VE; ++e) acc[e] = chain_next<DT, OP>(acc[e], Elem<DT>::load(vec_get<DT>(x[k], e)));
      }
    }
    VecU<DT> r;
    r.v = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < VE; ++e) vec_set<DT>(r, e, Elem<DT>::store(chain_last<DT, OP>(acc[e], n)));
    if (a.my_flags) {
      // a staged shard: other wavefronts (of any rank) read it while this kernel runs, so it is
      // written through, whole vectors only (the staging buffer is padded to 16 bytes)
      store_vec_coherent(&((u32x4*)a.out1)[v], r.v);
    } else if (whole) {
      u32x4_unaligned* o = &((u32x4_unaligned*)a.out1)[v];
      if (a.stream_out) __builtin_nontemporal_store(r.v, o);
      else *o = r.v;
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e)
        if ((uint32_t)e < a.tail1) ((S*)a.out1)[(size_t)v * VE + e] = vec_get<DT>(r, e);
    }
  }
}

// Chunk c of every shard: lane q waits for owner q's flag; false when an owner did not publish in time.
__device__ __forceinline__ bool xrank_wait_chunk(const XRankArgs& a, uint32_t c, int n) {
  const int lane = threadIdx.x;
  const uint32_t t = c * kXChunkTiles;  // the chunk exists for owner q if its first tile does
  bool ok = true;
  // lane q takes owner q's entries (a select per owner: no per-lane indexing of the argument block)
  uint32_t my_full = 0, my_last = 0;
  const uint32_t* my_flag = nullptr;
#pragma unroll
  for (int q = 0; q < kXRanks; ++q) {
    if (lane == q && q < n) {
      my_full = a.full2[q];
      my_last = a.last2[q];
      my_flag = a.shard_flags[q];
    }
  }
  if (my_flag && (t < my_full || (t == my_full && my_last != 0))) {
    ok = wait_flag32(my_flag + c, a.tile_epoch, a.sync.limit_ticks);
    if (!ok) report_late(a.sync.status, lane, a.tile_epoch);
  }
  // the data is read past the caches, so no invalidate is needed (and none per chunk is paid)
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  return __builtin_amdgcn_ballot_w64(!ok) == 0;
}

// Tile t of every shard: the wavefront moves the (up to) n tiles with all loads in flight before
// the first store.
__device__ __forceinline__ void xrank_gather_tiles(const XRankArgs& a, uint32_t t, int n) {
  const int lane = threadIdx.x;
  const size_t off = (size_t)t * kXTileBytes;
  u32x4 x[kXRanks];
  uint32_t len[kXRanks];
#pragma unroll
  for (int q = 0; q < kXRanks; ++q) {
    len[q] = 0;
    x[q] = (u32x4){0u, 0u, 0u, 0u};
    if (q < n) {
      len[q] = t < a.full2[q] ? kXTileBytes : (t == a.full2[q] ? a.last2[q] : 0u);
      // whole vectors, and the one that holds the last bytes (the staging buffer is padded)
      if ((uint32_t)lane < ((len[q] + 15u) >> 4)) x[q] = load_vec_coherent(&((const u32x4*)(a.shard_src[q] + off))[lane]);
    }
  }
#pragma unroll
  for (int q = 0; q < kXRanks; ++q) {
    if (q < n) {
      const uint32_t nv = len[q] >> 4;
      char* dst = a.shard_dst[q] + off;
      if ((uint32_t)lane < nv) __builtin_nontemporal_store(x[q], &((u32x4_unaligned*)dst)[lane]);
      const uint32_t rem = len[q] & 15u;
      if ((uint32_t)lane == nv && rem) {
#pragma unroll
        for (int b = 0; b < 16; ++b)
          if ((uint32_t)b < rem) dst[(nv << 4) + b] = (char)(x[q][b >> 2] >> ((b & 3) * 8));
      }
    }
  }
}

template <int DT, int OP>
__global__ __launch_bounds__(kWave) void xrank_reduce_kernel(const XRankArgs a) {
  const int n = a.sync.n;
  if (xsync_begin(a.sync)) {
    if (!a.aligned_in) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");  // misaligned inputs go through the caches
    if (!a.my_flags) {
      for (uint32_t tile = blockIdx.x; tile < a.tiles1; tile += gridDim.x) xrank_reduce_tile<DT, OP>(a, tile, n);
    } else {
      // allreduce: chunk by chunk; phase 1 publishes, phase 2 waits
      const uint32_t chunks1 = (a.tiles1 + kXChunkTiles - 1) / kXChunkTiles;
      for (uint32_t c = blockIdx.x; c < chunks1; c += gridDim.x) {
        for (uint32_t k = 0; k < kXChunkTiles; ++k)
          if (c * kXChunkTiles + k < a.tiles1) xrank_reduce_tile<DT, OP>(a, c * kXChunkTiles + k, n);
        // the chunk has reached memory before its flag can be seen: its stores are written through,
        // so waiting for them is enough
        wait_own_stores();
        if (threadIdx.x == 0) __hip_atomic_store(a.my_flags + c, a.tile_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      const uint32_t chunks2 = (a.tiles2 + kXChunkTiles - 1) / kXChunkTiles;
      for (uint32_t c = blockIdx.x; c < chunks2; c += gridDim.x) {
        if (!xrank_wait_chunk(a, c, n)) continue;
        for (uint32_t k = 0; k < kXChunkTiles; ++k)
          if (c * kXChunkTiles + k < a.tiles2) xrank_gather_tiles(a, c * kXChunkTiles + k, n);
      }
    }
  }
  xsync_end(a.sync, gridDim.x);
}

}  // namespace
