// One-launch small allreduce across rank processes: copy-in, cross-rank flags and the N-peer
// reduction in a single kernel, the structure of the reference's small allreduce
// (src/gpu/allreduce_small.h:166-361: copy into the IPC-visible buffer, rank barrier, sum of the N
// peer buffers).  Where the reference synchronises the whole grid and then all ranks, this kernel
// synchronises tile by tile: the wavefront that owns tile t of rank r
//   1. copies its 1 KiB of the caller's tensor into rank r's staging buffer,
//   2. publishes flag[r][t] = epoch (release),
//   3. waits until flag[q][t] has reached the epoch for every peer q (acquire, bounded),
//   4. reads tile t of every peer's staging buffer, runs the ascending-rank chain (its own
//      contribution comes from the registers of step 1) and writes the caller's output.
// A wavefront depends on the wavefronts of the same tile in the peers' launches only, so no grid
// has to be resident as a whole, and a launch needs no second kernel and no host round trip.
// Sixteen wavefronts (16 KiB of message) share a workgroup, for no other reason than that a
// workgroup sits on one compute unit: the wavefronts that wait for a late rank then hold
// bytes / 16 KiB compute units per rank instead of being spread over all of them, and whatever the
// late rank still has to run in front of its own launch finds whole compute units free.  A caller
// that limits the compute units further gets up to four tiles per wavefront: all copied in and
// published first, then waited for and reduced one after the other.
// Visibility inside the kernel is per access: the staging tile is written through to memory and
// waited for before its flag is stored, and the peers' tiles are read past the caches, so no
// cache-wide write-back or invalidate is paid per tile.
//
// The epoch that tags a launch's flags, and with it the choice between the two alternating sets of
// staging buffers and flags, comes from the host -- or, for launches that are replayed from a HIP
// graph (where kernel arguments are frozen at capture), from a word of this rank's own device
// memory that the launch itself advances: every wavefront reads it when it starts, the last one out
// stores the next value.  This is the reference's triple-buffer index advanced per call
// (`buffer_index`, src/gpu/allreduce_small.h:118, 139), kept where a replayed launch can reach it.  All ranks run
// the same sequence of such launches, so their words agree without ever being exchanged.
#pragma once

#include "kernels_common.hpp"
#include "kernels_sync.hpp"

namespace {

constexpr int kFusedRanks = 8;

struct FusedArgs {
  const char* in;             // this rank's contribution (element-aligned)
  char* out;                  // result; may be `in`
  char* stage[kFusedRanks];   // staging buffer of every rank (16-byte aligned), this process's mappings
  uint32_t* flag[kFusedRanks];  // per-tile flags of every rank
  uint64_t nvec;              // whole 16-byte vectors of the message
  uint64_t limit_ticks;
  uint32_t* status;
  uint32_t tail;              // elements after the last whole vector (< elements per vector)
  uint32_t epoch;
  uint32_t tiles;             // 1 KiB tiles of the message: wavefronts with work
  int n;
  int rank;
  // Device-resident epoch (null: `epoch` above is used): state[0] = number of launches completed on
  // these buffers, state[kFusedStateCounter] = wavefronts of the running launch that are done.  The
  // launch uses epoch state[0] + 1 and the buffer set (epoch & 1): set 1 lies stage_stride bytes /
  // flag_stride words behind set 0, which is what stage[] and flag[] then point at.
  uint32_t* state;
  uint32_t stage_stride;
  uint32_t flag_stride;
  // Bisecting switches (MCCL_FUSED_WORK_ONLY / MCCL_FUSED_SYNC_ONLY): the launch without its rank
  // waits, or with nothing but them -- for timing what each part costs, never for results.
  uint32_t mode;
};

constexpr int kFusedStateCounter = 16;  // 32-bit words: on a cache line of its own

constexpr int kFusedWavesPerGroup = 16;

// A launch limited to few workgroups gives a wavefront up to this many tiles.
constexpr int kFusedMaxTilesPerWave = 4;

// A wavefront of a launch with a device-resident epoch is done: the last one of the launch stores
// the epoch the launch ran with, which is what the next launch on these buffers starts from.  Every
// wavefront has read the word before it gets here, so the store cannot overtake a reader.
__device__ __forceinline__ void fused_wave_done(const FusedArgs& a, uint32_t epoch, uint32_t waves, int lane) {
  if (!a.state || lane != 0) return;
  uint32_t* counter = a.state + kFusedStateCounter;
  if (__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == waves) {
    __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(a.state, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int DT, int OP>
__global__ __launch_bounds__(kWave * kFusedWavesPerGroup) void allreduce_fused_kernel(const FusedArgs a) {
  using S = typename Elem<DT>::store_t;
  using A = typename Elem<DT>::acc_t;
  constexpr int VE = vec_elems<DT>();
  const uint32_t wave = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const uint32_t waves = gridDim.x * (blockDim.x / kWave);
  const int lane = threadIdx.x % kWave;
  uint32_t epoch = a.epoch;
  uint32_t stage_off = 0, flag_off = 0;  // which of the two buffer sets
  if (a.state) {
    epoch = __builtin_amdgcn_readfirstlane(__hip_atomic_load(a.state, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) + 1u;
    stage_off = (epoch & 1u) * a.stage_stride;
    flag_off = (epoch & 1u) * a.flag_stride;
  }
  if (wave >= a.tiles) {  // (the wavefronts of a workgroup never meet at a barrier)
    fused_wave_done(a, epoch, waves, lane);
    return;
  }
  // this wavefront's tiles: wave, wave + waves, ... (the host launches enough wavefronts for
  // kFusedMaxTilesPerWave to cover the message)

  // 1. copy-in of all of them
  VecU<DT> mine[kFusedMaxTilesPerWave];
#pragma unroll
  for (int j = 0; j < kFusedMaxTilesPerWave; ++j) {
    const uint32_t tile = wave + (uint32_t)j * waves;
    if (tile >= a.tiles) break;
    const uint64_t v = (uint64_t)tile * kWave + lane;
    const bool whole = v < a.nvec;
    const bool part = v == a.nvec && a.tail != 0;  // the one vector that is not whole
    mine[j].v = (u32x4){0u, 0u, 0u, 0u};
    if (a.mode & MCCL_FUSED_SYNC_ONLY) continue;
    if (whole) {
      mine[j].v = __builtin_nontemporal_load(&((const u32x4_unaligned*)a.in)[v]);
    } else if (part) {
      for (uint32_t e = 0; e < a.tail; ++e) vec_set<DT>(mine[j], (int)e, ((const S*)a.in)[v * VE + e]);
    }
    if (whole || part) store_vec_coherent(&((u32x4*)(a.stage[a.rank] + stage_off))[v], mine[j].v);  // written through
  }
  // 2. publish: the tiles have reached memory before their flags can be seen
  wait_own_stores();
#pragma unroll
  for (int j = 0; j < kFusedMaxTilesPerWave; ++j) {
    const uint32_t tile = wave + (uint32_t)j * waves;
    if (tile >= a.tiles) break;
    if (lane == 0) __hip_atomic_store(a.flag[a.rank] + flag_off + tile, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
#pragma unroll
  for (int j = 0; j < kFusedMaxTilesPerWave; ++j) {
    const uint32_t tile = wave + (uint32_t)j * waves;
    if (tile >= a.tiles) break;
    const uint64_t v = (uint64_t)tile * kWave + lane;
    const bool whole = v < a.nvec;
    const bool part = v == a.nvec && a.tail != 0;
    // 3. wait for the same tile of every peer
    bool ok = true;
    if (lane < a.n && lane != a.rank && !(a.mode & MCCL_FUSED_WORK_ONLY)) {
      ok = wait_flag32(a.flag[lane] + flag_off + tile, epoch, a.limit_ticks);
      if (!ok) report_late(a.status, lane, epoch);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the loads below stay below the wait
    // tiles whose peers did not arrive are left alone (the failure is reported through `status`)
    if (__builtin_amdgcn_ballot_w64(!ok) != 0) {
      fused_wave_done(a, epoch, waves, lane);
      return;
    }
    if (!(whole || part) || (a.mode & MCCL_FUSED_SYNC_ONLY)) continue;

    // 4. the N-peer reduction, ascending rank order; all peer loads are issued before the first add
    VecU<DT> x[kFusedRanks];
#pragma unroll
    for (int k = 0; k < kFusedRanks; ++k) {
      if (k < a.n) {
        if (k == a.rank) x[k].v = mine[j].v;
        else x[k].v = load_vec_coherent(&((const u32x4*)(a.stage[k] + stage_off))[v]);  // past the caches: written by another rank just now
      }
    }
    A acc[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[e] = chain_first<DT, OP>(Elem<DT>::load(vec_get<DT>(x[0], e)));
#pragma unroll
    for (int k = 1; k < kFusedRanks; ++k) {
      if (k < a.n) {
#pragma unroll
        for (int e = 0; e < VE; ++e) acc[e] = chain_next<DT, OP>(acc[e], Elem<DT>::load(vec_get<DT>(x[k], e)));
      }
    }
    VecU<DT> r;
    r.v = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < VE; ++e) vec_set<DT>(r, e, Elem<DT>::store(chain_last<DT, OP>(acc[e], a.n)));
    if (whole) {
      ((u32x4_unaligned*)a.out)[v] = r.v;
    } else {
      for (uint32_t e = 0; e < a.tail; ++e) ((S*)a.out)[v * VE + e] = vec_get<DT>(r, (int)e);
    }
  }
  fused_wave_done(a, epoch, waves, lane);
}

}  // namespace
