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

// Polls *word until it is at least `epoch` (64-bit, monotonic).  Returns false at the time limit.
__device__ __forceinline__ bool wait_flag64(const uint64_t* word, uint64_t epoch, uint64_t limit_ticks) {
  const uint64_t t0 = wall_clock64();
  while (__hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) < epoch) {
    if (wall_clock64() - t0 > limit_ticks) return false;
    __builtin_amdgcn_s_sleep(1);
  }
  return true;
}

__device__ __forceinline__ void report_late(uint32_t* status, int late_rank, uint32_t epoch_lo) {
  if (!status) return;
  __hip_atomic_store(status + 1, epoch_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(status, (uint32_t)(late_rank + 1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

template <typename ARGS>
__global__ __launch_bounds__(kWave) void rank_barrier_kernel(const ARGS a) {
  const int lane = threadIdx.x;
  if (lane == 0) __hip_atomic_store(a.flag[a.rank], a.epoch, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  if (lane < a.n && lane != a.rank) {
    if (!wait_flag64(a.flag[lane], a.epoch, a.limit_ticks)) report_late(a.status, lane, (uint32_t)a.epoch);
  }
}

}  // namespace
