// N-buffer reduction kernels (allreduce local-reduce, reduce_scatter shard reduction, coalesced
// reductions).  What they replace in the reference: the N-peer sum of
// src/gpu/allreduce_small.h:289-361, the five data kernels of src/gpu/allreduce.h:306-533 and the
// ccl::allreduce / ccl::reduce_scatter call sites of src/gpu/dpcpp_ccl.cpp:781-788, 1002-1008.
#pragma once

#include "kernels_common.hpp"

namespace {

// One reduction of a launch, fully described by the host so that a wavefront needs one
// scalar load to start and 32-bit uniform arithmetic only:
//   elements [0, head)                      peeled, element-wise (out not yet 128-byte aligned)
//   vectors  [0, nvec) at byte offset head*es   the vector body
//   elements [head + nvec*VE, +tail)        peeled, element-wise
struct ReduceJob {
  char* out;
  size_t in_off;   // byte offset applied to every input pointer
  size_t nvec;     // 16-byte vectors in the body
  uint32_t head;   // elements before the body (< 128): the body starts on a cache line of out
  uint32_t tail;   // elements after the body (< 16)
};

// Kernel arguments.  reduce_n: one job.  reduce_scatter: one job per shard, same pointers,
// different byte offsets.  reduce_multi (OWN == true kernels): job j reads the n pointers
// starting at ptr[job_ptr0[j]].
constexpr uint32_t kFlagStreamOut = 1u;  // write the output with streaming (write-through) stores

struct ReduceArgs {
  const char* ptr[MCCL_MAX_RANKS];
  ReduceJob job[kMaxJobs];
  int job_ptr0[kMaxJobs];
  int n;
  uint32_t flags;
};

// The same for the common call: one job, at most kLeanRanks inputs.  104 bytes instead of 2.8 KB:
// the launch path of the runtime gets measurably slower above ~104 bytes of kernel arguments
// (2.6 -> 3.6 us per back-to-back launch), which is most of the cost of a small message.
constexpr int kLeanRanks = 8;
struct LeanReduceArgs {
  const char* ptr[kLeanRanks];
  ReduceJob job[1];
  int n;
  uint32_t flags;
};
static_assert(sizeof(LeanReduceArgs) <= 104, "lean kernel arguments must stay below the launch-cost step");

// Element-wise reduction of one element (used for peeled heads/tails and the misaligned path).
template <int DT, int OP, typename ARGS>
__device__ __forceinline__ void reduce_one(const ARGS& a, int p0, int n, size_t in_off,
                                           char* out, size_t idx) {
  using S = typename Elem<DT>::store_t;
  using A = typename Elem<DT>::acc_t;
  A acc = chain_first<DT, OP>(Elem<DT>::load(((const S*)(a.ptr[p0] + in_off))[idx]));
  for (int k = 1; k < n; ++k)
    acc = chain_next<DT, OP>(acc, Elem<DT>::load(((const S*)(a.ptr[p0 + k] + in_off))[idx]));
  acc = chain_last<DT, OP>(acc, n);
  ((S*)out)[idx] = Elem<DT>::store(acc);
}

// Loads one 16-byte vector; GUARD adds the bounds check of the last, partial tile.  The vector body
// is aligned on the output; an input that is not congruent with it mod 16 is read at whatever
// alignment its elements have (global loads may be unaligned on this target: the hardware splits
// them), hence the under-aligned pointer type.  Aligned inputs get the same instruction.

template <bool GUARD>
__device__ __forceinline__ u32x4 load_vec(const u32x4_unaligned* p, size_t v, size_t nvec) {
  if constexpr (GUARD) {
    if (v >= nvec) return (u32x4){0u, 0u, 0u, 0u};
  }
  return __builtin_nontemporal_load(&p[v]);  // streamed once: keep it out of the caches
}

// Streaming 16-byte store for large outputs: written through at agent scope (`sc1`), which on
// this part is the fastest way past the caches for a stream that nobody re-reads soon (8 reads :
// 1 write at 64 MiB per stream: plain 82 %, `nt` 85 %, `sc1` 86.8 % of the HBM peak).  Written as
// an instruction because the hint has to survive: the compiler drops the non-temporal hint of
// __builtin_nontemporal_store on the unguarded path of the tile loop.  The compiler does not know
// that this is a store of more than 8 bytes, after which the data registers must not be
// overwritten in the next cycle (it would schedule the hazard's wait state itself for a store it
// knows), so the wait states are part of the instruction sequence.  The operands are vector
// registers only: no scalar-to-vector-memory hazard can arise.  Stores the compiler cannot see in
// its vmcnt bookkeeping only ever make its waits stricter (loads return in order among
// themselves).
__device__ __forceinline__ void store_vec_stream(u32x4* p, u32x4 x) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(x) : "memory");
}

// One tile of BLOCK*U vectors: every lane loads its U vectors from all n inputs, runs the
// ascending-rank chain in registers and streams the result out.
// NT > 0: rank count known at compile time, all NT*U loads in flight before the first add.
// NT == 0: runtime rank count, groups of 8 ranks.
template <int DT, int OP, int NT, int U, int BLOCK, bool GUARD, typename ARGS>
__device__ __forceinline__ void reduce_tile(const ARGS& a, int p0, size_t in_byte_off,
                                            u32x4* ov, size_t v0, size_t nvec, int n, bool stream_out) {
  using A = typename Elem<DT>::acc_t;
  using S = typename Elem<DT>::store_t;
  constexpr int VE = vec_elems<DT>();
  A acc[U][VE];

  if constexpr (NT > 0) {
    VecU<DT> x[NT][U];
#pragma unroll
    for (int k = 0; k < NT; ++k) {
      const u32x4_unaligned* iv = (const u32x4_unaligned*)(a.ptr[p0 + k] + in_byte_off);
#pragma unroll
      for (int u = 0; u < U; ++u) x[k][u].v = load_vec<GUARD>(iv, v0 + (size_t)u * BLOCK, nvec);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < VE; ++e) acc[u][e] = chain_first<DT, OP>(Elem<DT>::load(vec_get<DT>(x[0][u], e)));
#pragma unroll
      for (int k = 1; k < NT; ++k)
#pragma unroll
        for (int e = 0; e < VE; ++e)
          acc[u][e] = chain_next<DT, OP>(acc[u][e], Elem<DT>::load(vec_get<DT>(x[k][u], e)));
    }
  } else {
    // runtime rank count: groups of up to eight ranks, so that up to eight ranks have all their
    // loads in flight before the first add, like the compile-time rank counts
    constexpr int G = 8;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < VE; ++e) acc[u][e] = (A)0;  // overwritten by rank 0's element
    for (int kb = 0; kb < n; kb += G) {
      VecU<DT> x[G][U];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        if (kb + g < n) {
          const u32x4_unaligned* iv = (const u32x4_unaligned*)(a.ptr[p0 + kb + g] + in_byte_off);
#pragma unroll
          for (int u = 0; u < U; ++u) x[g][u].v = load_vec<GUARD>(iv, v0 + (size_t)u * BLOCK, nvec);
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        if (kb + g < n) {
#pragma unroll
          for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < VE; ++e) {
              const A xv = Elem<DT>::load(vec_get<DT>(x[g][u], e));
              if (g == 0 && kb == 0) acc[u][e] = chain_first<DT, OP>(xv);
              else acc[u][e] = chain_next<DT, OP>(acc[u][e], xv);
            }
        }
      }
    }
  }

#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t v = v0 + (size_t)u * BLOCK;
    if (!GUARD || v < nvec) {
      VecU<DT> r;
      if constexpr (sizeof(S) == 1) r.v = (u32x4){0u, 0u, 0u, 0u};  // vec_set ors the bytes in
#pragma unroll
      for (int e = 0; e < VE; ++e) vec_set<DT>(r, e, Elem<DT>::store(chain_last<DT, OP>(acc[u][e], n)));
      // large outputs are streamed past the caches; small ones stay cacheable for their consumer
      if (stream_out) store_vec_stream(&ov[v], r.v);
      else ov[v] = r.v;
    }
  }
}

// Vector kernel.  The host aligns the vector body on the output; inputs need element alignment
// only.  The output may be exactly one of the inputs: a lane reads
// element i of every input before it writes element i, and no other lane touches i.
// OWN: each job has its own n pointers (coalesced reductions); otherwise all jobs share
// ptr[0..n) and the pointer loads do not wait for the job record.
template <int DT, int OP, int NT, int U, int BLOCK, bool OWN, typename ARGS>
__global__ __launch_bounds__(BLOCK) void reduce_vec_kernel(const ARGS a) {
  using S = typename Elem<DT>::store_t;
  constexpr int VE = vec_elems<DT>();
  const int jid = blockIdx.y;
  int p0 = 0;
  if constexpr (OWN) p0 = a.job_ptr0[jid];
  const int n = (NT > 0) ? NT : a.n;
  const bool stream_out = (a.flags & kFlagStreamOut) != 0;
  char* out = a.job[jid].out;
  const size_t in_off = a.job[jid].in_off;
  const size_t nvec = a.job[jid].nvec;
  const uint32_t head = a.job[jid].head;
  const uint32_t tail = a.job[jid].tail;

  if (blockIdx.x == 0) {
    const uint32_t t = threadIdx.x;
    // head < 128 and tail < 16 elements: a couple of strides of the workgroup at most
    for (uint32_t i = t; i < head + tail; i += BLOCK)
      reduce_one<DT, OP>(a, p0, n, in_off, out, i < head ? (size_t)i : (size_t)head + nvec * VE + (i - head));
  }

  const size_t body_off = (size_t)head * sizeof(S);  // bytes
  u32x4* ov = (u32x4*)(out + body_off);
  constexpr uint32_t TILE = (uint32_t)BLOCK * U;
  // the host keeps nvec / TILE below 2^32
  const uint32_t full_tiles = (uint32_t)(nvec / TILE);
  const uint32_t partial = (uint32_t)(nvec % TILE) ? 1u : 0u;

  uint32_t tile = blockIdx.x;
  for (; tile < full_tiles; tile += gridDim.x)
    reduce_tile<DT, OP, NT, U, BLOCK, false>(a, p0, in_off + body_off, ov, (size_t)tile * TILE + threadIdx.x, nvec, n, stream_out);
  if (tile == full_tiles && partial)  // the one partial tile; exactly one workgroup reaches it
    reduce_tile<DT, OP, NT, U, BLOCK, true>(a, p0, in_off + body_off, ov, (size_t)tile * TILE + threadIdx.x, nvec, n, stream_out);
}

}  // namespace
