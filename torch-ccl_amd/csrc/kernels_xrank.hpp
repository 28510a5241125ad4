// One-launch reductions between rank processes that read the peers' tensors in place.
//
// With several processes on one GPU every kernel launch of a process waits for its turn at the
// dispatcher, so a collective made of several launches (barrier, reduce, barrier, gather, barrier)
// costs as many turns per rank.  This kernel is the whole collective in one launch:
//
//   begin    every rank's input is complete (xsync_begin: the launch itself says "my stream has
//            reached the collective"; all workgroups wait for all ranks' words)
//   reduce   this rank reduces ITS shard of all ranks' tensors (ascending-rank chain, as
//            reduce_vec_kernel) and writes it to the caller's output (reduce_scatter) or, written
//            through, into the same shard of EVERY rank's tensor (allreduce: the peers' mappings
//            are writable, as the temp buffers are that the reference's gather step stores into,
//            src/gpu/allreduce.h:470-487)
//   end      xsync_end: nobody's kernel completes before all ranks are done reading (and, for the
//            allreduce, writing)
//
// The allreduce moves n reads and n writes per element of a shard -- S bytes in, S bytes out per
// rank for a message of S bytes -- where the reference's two-shot large path (reduce-scatter
// through scratch, then all-gather: src/gpu/allreduce.h:306-533) moves (n + 1) reads and 2 writes
// per element in two phases with a rank synchronisation between them.  While the collective runs
// only the owner of a shard touches that shard of any tensor (each lane reads the n values of a
// vector before it writes them), so no flags are needed between the ranks.
//
// The grid is persistent and small enough that the launches of all ranks are resident together
// (waiting workgroups hold their slots).  All waits are bounded.
#pragma once

#include "kernels_common.hpp"
#include "kernels_fused.hpp"
#include "kernels_sync.hpp"

namespace {

constexpr int kXRanks = kLeanSyncRanks;
constexpr uint32_t kXTileBytes = kWave * 16;  // 1 KiB: one vector per lane

// All extents are 32-bit and precomputed by the host: the device does no uniform 64-bit compares.
struct XRankArgs {
  const char* in[kXRanks];            // inputs in rank order, already at this rank's shard
  char* out1;                         // reduce_scatter: the output
  uint32_t nvec1;                     // whole vectors ...
  uint32_t tail1;                     // ... and elements after them (< elements per vector)
  uint32_t tiles1;                    // tiles that cover both
  uint32_t stream_out;                // write out1 past the caches (large reduce_scatter outputs)
  uint32_t aligned_in;                // every in[k] is 8-byte aligned: read past the caches
  uint32_t push;                      // allreduce: write the result over in[k] of every rank k instead of out1
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
    if (a.push) {
      // the finished shard goes straight into every rank's tensor, written through: the owners read
      // it with kernels that start after this one has published its closing epoch
#pragma unroll
      for (int k = 0; k < kXRanks; ++k) {
        if (k < n) {
          if (whole) {
            store_vec_through(const_cast<char*>(a.in[k]) + (size_t)v * 16, r.v);
          } else {
#pragma unroll
            for (int e = 0; e < VE; ++e)
              if ((uint32_t)e < a.tail1)
                __hip_atomic_store(&((S*)const_cast<char*>(a.in[k]))[(size_t)v * VE + e], vec_get<DT>(r, e), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          }
        }
      }
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

template <int DT, int OP>
__global__ __launch_bounds__(kWave) void xrank_reduce_kernel(const XRankArgs a) {
  const int n = a.sync.n;
  if (xsync_begin(a.sync)) {
    if (!a.aligned_in) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");  // misaligned inputs go through the caches
    for (uint32_t tile = blockIdx.x; tile < a.tiles1; tile += gridDim.x) xrank_reduce_tile<DT, OP>(a, tile, n);
  }
  xsync_end(a.sync, gridDim.x);
}

}  // namespace
