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
//            output for a reduce_scatter -- and publishes one flag per 1 KiB tile
//   phase 2  (allreduce) tile by tile, all finished shards are copied from the owners' staging
//            buffers into the caller's tensor; a tile waits for its owner's flag only
//   end      (reduce_scatter) xsync_end: nobody's kernel completes before all ranks are done reading
//
// which is the two-shot allreduce of the reference's large path (reduce-scatter through scratch,
// then all-gather: src/gpu/allreduce.h:306-533) without its nine launches.  The allreduce needs no
// closing wait: a rank's tensor is read by phase 1 of the shard owners only, tile (q, t) of it is
// overwritten by this rank's phase 2 only after owner q has published flag t, and this rank's
// kernel ends only when it has copied -- hence seen the flag of -- every tile of every owner.
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

// All extents are 32-bit and precomputed by the host: the device does no uniform 64-bit compares.
struct XRankArgs {
  const char* in[kXRanks];            // phase 1 inputs in rank order, already at this rank's shard
  char* out1;                         // phase 1 output
  uint32_t* my_flags;                 // phase 1 publishes my_flags[t] = tile_epoch (null: no flags)
  uint32_t nvec1;                     // phase 1: whole vectors ...
  uint32_t tail1;                     // ... and elements after them (< elements per vector)
  uint32_t tiles1;                    // tiles that cover both
  uint32_t tile_epoch;
  // phase 2: shard q of the message is copied from shard_src[q] to shard_dst[q], tile t of it once
  // shard_flags[q][t] has reached tile_epoch
  const char* shard_src[kXRanks];
  const uint32_t* shard_flags[kXRanks];
  char* shard_dst[kXRanks];
  uint32_t full2[kXRanks];            // whole tiles of shard q
  uint32_t last2[kXRanks];            // bytes of the partial tile after them (0: none)
  uint32_t tiles2;                    // tiles of the longest shard; 0 = no phase 2
  uint32_t stream_out;                // write out1 past the caches (large reduce_scatter outputs)
  XSync sync;
};

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
          x[k].v = __builtin_nontemporal_load(&((const u32x4_unaligned*)a.in[k])[v]);
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
    if (whole) {
      u32x4_unaligned* o = &((u32x4_unaligned*)a.out1)[v];
      if (a.stream_out) __builtin_nontemporal_store(r.v, o);
      else *o = r.v;
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e)
        if ((uint32_t)e < a.tail1) ((S*)a.out1)[(size_t)v * VE + e] = vec_get<DT>(r, e);
    }
  }
  if (a.my_flags) {
    // the tile is written back before its flag can be seen
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    if (lane == 0) __hip_atomic_store(a.my_flags + tile, a.tile_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Tile t of every shard: lane q waits for owner q's flag, then the wavefront moves the (up to) n
// tiles with all loads in flight before the first store.
__device__ __forceinline__ void xrank_gather_tiles(const XRankArgs& a, uint32_t t, int n) {
  const int lane = threadIdx.x;
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
    ok = wait_flag32(my_flag + t, a.tile_epoch, a.sync.limit_ticks);
    if (!ok) report_late(a.sync.status, lane, a.tile_epoch);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
  if (__builtin_amdgcn_ballot_w64(!ok) != 0) return;
  const size_t off = (size_t)t * kXTileBytes;
  u32x4 x[kXRanks];
  uint32_t len[kXRanks];
#pragma unroll
  for (int q = 0; q < kXRanks; ++q) {
    len[q] = 0;
    if (q < n) {
      len[q] = t < a.full2[q] ? kXTileBytes : (t == a.full2[q] ? a.last2[q] : 0u);
      x[q] = (u32x4){0u, 0u, 0u, 0u};
      if ((uint32_t)lane < (len[q] >> 4)) x[q] = __builtin_nontemporal_load(&((const u32x4*)(a.shard_src[q] + off))[lane]);
    }
  }
#pragma unroll
  for (int q = 0; q < kXRanks; ++q) {
    if (q < n) {
      const uint32_t nv = len[q] >> 4;
      if ((uint32_t)lane < nv) __builtin_nontemporal_store(x[q], &((u32x4_unaligned*)(a.shard_dst[q] + off))[lane]);
      const uint32_t rem = len[q] & 15u;
      if ((uint32_t)lane < rem) (a.shard_dst[q] + off)[(nv << 4) + lane] = (a.shard_src[q] + off)[(nv << 4) + lane];
    }
  }
}

template <int DT, int OP>
__global__ __launch_bounds__(kWave) void xrank_reduce_kernel(const XRankArgs a) {
  const int n = a.sync.n;
  if (xsync_begin(a.sync)) {
    for (uint32_t tile = blockIdx.x; tile < a.tiles1; tile += gridDim.x) xrank_reduce_tile<DT, OP>(a, tile, n);
    for (uint32_t t = blockIdx.x; t < a.tiles2; t += gridDim.x) xrank_gather_tiles(a, t, n);
  }
  xsync_end(a.sync, gridDim.x);
}

}  // namespace
