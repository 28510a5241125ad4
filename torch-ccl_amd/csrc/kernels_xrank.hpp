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
  uint32_t no_invalidate;             // with aligned_in == 0: the caches are clean already (a kernel boundary lies behind the ranks' barrier)
  // The addresses of the ranks' tensors from device memory instead (null: in[] above holds them):
  // in_table[k] + in_off, as the barrier kernel in front of this launch has resolved them from the
  // ranks' offers.  A null entry: the launch does nothing but take part in the closing wait.
  const uint64_t* in_table;
  uint64_t in_off;
  // Or exchanged by this launch itself (the one-launch form with offers): this rank's offer goes into
  // offer[rank] before its ready flag, and every wavefront resolves the peers' offers against
  // `imports` after the opening wait (in_off applies as above).
  uint64_t* offer[kXRanks];
  uint64_t mine[4];
  const mccl_import_table_t* imports;
  uint64_t my_buffer;
  XSync sync;
};

// Lane l's vector of tile `tile` of a peer's tensor.  8-byte aligned tensors (always, for whole
// tensors out of an allocator) are read past the caches in one streaming access (load_tile_coherent);
// others as an ordinary unaligned load after a cache invalidate (aligned_in == 0 makes the kernel
// invalidate once per workgroup).
__device__ __forceinline__ u32x4 load_in(const char* base, uint32_t tile, uint32_t aligned, uint32_t lane) {
  const char* tb = base + (size_t)tile * kXTileBytes;  // uniform
  if (aligned) return load_tile_coherent(tb, lane * 16u);
  return __builtin_nontemporal_load(&((const u32x4_unaligned*)tb)[lane]);
}

// Where the ranks' tensors are: from the argument block, or from device memory (in_table).  Only
// ever indexed with constants, so that it lives in scalar registers.
struct XIns {
  const char* p[kXRanks];
};

// in[k] for a k known at run time only (a select per rank: no dynamic indexing)
__device__ __forceinline__ const char* pick_in(const XIns& in, int k) {
  const char* p = in.p[0];
#pragma unroll
  for (int q = 1; q < kXRanks; ++q)
    if (k == q) p = in.p[q];
  return p;
}

template <int DT, int NS>
__device__ __forceinline__ void xrank_load_tile(const XRankArgs& a, const XIns& in, const Wave& w, uint32_t tile, int n, uint32_t aligned, VecU<DT> (&x)[kXRanks]) {
  const uint32_t v = tile * kWave + w.lane;  // the host keeps tiles1 * 64 below 2^32
  if (v < a.nvec1) {
#pragma unroll
    for (int k = 0; k < kXRanks; ++k) {
      if (NS ? k < NS : k < n) x[k].v = load_in(in.p[k], tile, aligned, w.lane);
    }
  }
}

// Reduces the loaded vectors of a tile (ascending-rank chain) and stores the result.
template <int DT, int OP, int NS>
__device__ __forceinline__ void xrank_finish_tile(const XRankArgs& a, const XIns& in, const Wave& w, uint32_t tile, int n, uint32_t aligned, const VecU<DT> (&x)[kXRanks]) {
  using A = typename Elem<DT>::acc_t;
  constexpr int VE = vec_elems<DT>();
  const uint32_t v = tile * kWave + w.lane;
  if (v < a.nvec1) {
    A acc[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[e] = chain_first<DT, OP>(Elem<DT>::load(vec_get<DT>(x[0], e)));
#pragma unroll
    for (int k = 1; k < kXRanks; ++k) {
      if (NS ? k < NS : k < n) {
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
        if (NS ? k < NS : k < n) {
          char* tb = const_cast<char*>(in.p[k]) + (size_t)tile * kXTileBytes;  // uniform
          if (aligned) store_tile_through(tb, w.lane * 16u, r.v);
          else store_vec_through(tb + w.lane * 16u, r.v);
        }
      }
    } else {
      u32x4_unaligned* o = &((u32x4_unaligned*)a.out1)[v];
      if (a.stream_out) store_vec_stream((u32x4*)o, r.v);
      else *o = r.v;
    }
  }
}

// The elements after the last whole vector (fewer than a vector holds): lane e takes element e.
template <int DT, int OP>
__device__ __forceinline__ void xrank_tail(const XRankArgs& a, const XIns& in, const Wave& w, int n) {
  using S = typename Elem<DT>::store_t;
  using A = typename Elem<DT>::acc_t;
  constexpr int VE = vec_elems<DT>();
  if (w.lane < a.tail1) {
    const size_t i = (size_t)a.nvec1 * VE + w.lane;
    A acc = chain_first<DT, OP>(Elem<DT>::load(__hip_atomic_load(&((const S*)in.p[0])[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)));
    for (int k = 1; k < n; ++k) {
      const S* src = (const S*)pick_in(in, k);
      acc = chain_next<DT, OP>(acc, Elem<DT>::load(__hip_atomic_load(&src[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)));
    }
    const S r = Elem<DT>::store(chain_last<DT, OP>(acc, n));
    if (a.push) {
      for (int k = 0; k < n; ++k) __hip_atomic_store(&((S*)const_cast<char*>(pick_in(in, k)))[i], r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    } else {
      ((S*)a.out1)[i] = r;
    }
  }
}

// The grid is persistent: wavefront i of c walks tiles i, i + c, ...  The loads of its
// next tile are in flight while it reduces and stores the current one (two register sets, used
// alternately): without that all wavefronts, released together by the opening wait, alternate
// between a phase of loads and a phase of stores in step, and the memory pipeline runs dry
// between the phases.
template <int DT, int OP, int NS>
__device__ __forceinline__ void xrank_walk(const XRankArgs& a, const XIns& in, const Wave& w, int n, uint32_t aligned) {
  const uint32_t T = a.tiles1, G = w.count;
  uint32_t t0 = w.index;
  if (t0 < T) {
    VecU<DT> x0[kXRanks], x1[kXRanks];
    xrank_load_tile<DT, NS>(a, in, w, t0, n, aligned, x0);
    for (;;) {
      const uint32_t t1 = t0 + G;
      if (t1 < T) xrank_load_tile<DT, NS>(a, in, w, t1, n, aligned, x1);
      xrank_finish_tile<DT, OP, NS>(a, in, w, t0, n, aligned, x0);
      if (t1 >= T) break;
      t0 = t1 + G;
      if (t0 < T) xrank_load_tile<DT, NS>(a, in, w, t0, n, aligned, x0);
      xrank_finish_tile<DT, OP, NS>(a, in, w, t1, n, aligned, x1);
      if (t0 >= T) break;
    }
  }
}

// INDIRECT 1: the tensors' addresses come from the table in device memory that the kernel in front of
// this one has written (a kernel of its own, so that the common form starts exactly as before: a
// wavefront of one tile lives for a few microseconds, and a chain of selects in front of its loads
// showed as 15 % of the shard reduction's time).  Read with scalar loads, like the arguments; a table
// entry of a rank that takes part must not be null.
// INDIRECT 2: the launch exchanges the offers itself -- the one-launch form, whose opening wait is
// the barrier: lane r of every wavefront resolves rank r's offer once the wait has passed and the
// addresses are broadcast into scalar registers.
template <int DT, int OP, int WPG, int INDIRECT>
__global__ __launch_bounds__(kWave * WPG) void xrank_reduce_kernel(const XRankArgs a) {
  const int n = a.sync.n;
  const Wave w = this_wave<WPG>();
  XIns in;
  bool resolved = true;
  if constexpr (INDIRECT == 1) {
    const auto* table = (const __attribute__((address_space(4))) uint64_t*)a.in_table;
#pragma unroll
    for (int k = 0; k < kXRanks; ++k) {
      const uint64_t p = table[k];
      if (k < n) resolved = resolved && p != 0;
      in.p[k] = (const char*)(p + a.in_off);
    }
  } else if constexpr (INDIRECT == 2) {
    if (blockIdx.x == 0 && threadIdx.x == 0) publish_offer(a.offer[a.sync.rank], a.mine);  // before xsync_begin stores this rank's flag
  } else {
#pragma unroll
    for (int k = 0; k < kXRanks; ++k) in.p[k] = a.in[k];
  }
  bool begun = resolved && xsync_begin(a.sync);
  uint32_t aligned = a.aligned_in;
  if constexpr (INDIRECT == 2) {
    if (begun) {
      uint64_t where = a.my_buffer;
      const int r = (int)w.lane;
      if (r < n && r != a.sync.rank) {
        where = resolve_offer(a.offer[r], a.imports, r);
        if (!where) report_late(a.sync.status, r, MCCL_STATUS_UNMAPPED);
      }
      begun = __builtin_amdgcn_ballot_w64(r < n && where == 0) == 0;
      where += a.in_off;
      // (only now is it known where the tensors lie: 8-byte aligned ones -- whole tensors out of an
      // allocator always are -- are read past the caches in one streaming access each and need no
      // invalidate, which with several processes on the GPU is everybody's loss)
      aligned = __builtin_amdgcn_ballot_w64(r < n && (where & 7u) != 0) == 0 ? 1u : 0u;
#pragma unroll
      for (int k = 0; k < kXRanks; ++k) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)where, k);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(where >> 32), k);
        in.p[k] = (const char*)(((uint64_t)hi << 32) | lo);
      }
    } else {
#pragma unroll
      for (int k = 0; k < kXRanks; ++k) in.p[k] = nullptr;
    }
  }
  if (begun) {
    if (!aligned && !a.no_invalidate) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");  // misaligned inputs go through the caches
    if (n == kXRanks) xrank_walk<DT, OP, kXRanks>(a, in, w, n, aligned);
    else xrank_walk<DT, OP, 0>(a, in, w, n, aligned);
    if (a.tail1 && w.index == w.count - 1) xrank_tail<DT, OP>(a, in, w, n);
  }
  xsync_end(a.sync, gridDim.x, a.push != 0);
}

}  // namespace
