// Launch dispatch of the reduction kernels: shape x argument block x rank-count specialisation x
// op for one element type.  Each element type is compiled as a translation unit of its own
// (mccl_reduce_dtype.hip, built once per type), which is what keeps the build parallel.
#pragma once

#include "kernels_fused.hpp"
#include "kernels_reduce.hpp"
#include "kernels_xrank.hpp"

namespace {

enum Shape { kShapeSmall, kShapeStream, kShapePersistent };

// Geometry of a launch.
struct Geometry {
  Shape shape;
  unsigned grid_x;
  int block;
  unsigned lds;   // dynamic LDS reservation (occupancy cap), bytes
  bool own_ptrs;  // jobs carry their own pointer sets (coalesced reductions)
  bool stream_out;  // write the output with streaming (write-through) stores
};

template <int DT, int OP, int NT, bool OWN, typename ARGS>
hipError_t launch_vec_args(const ARGS& a, const Geometry& g, int njobs, hipStream_t s) {
  const dim3 grid(g.grid_x, njobs, 1);
  if (g.shape == kShapePersistent)
    hipLaunchKernelGGL((reduce_vec_kernel<DT, OP, NT, kUnrollPersistent, kBlockPersistent, OWN, ARGS>), grid,
                       dim3(kBlockPersistent), 0, s, a);
  else
    hipLaunchKernelGGL((reduce_vec_kernel<DT, OP, NT, 1, kWave, OWN, ARGS>), grid, dim3(kWave), g.lds, s, a);
  return hipGetLastError();
}

// One job over at most kLeanRanks shared pointers travels in the 104-byte argument block.
template <int DT, int OP, int NT, bool OWN>
hipError_t launch_vec(const ReduceArgs& a, const Geometry& g, int njobs, hipStream_t s) {
  if constexpr (!OWN) {
    if (njobs == 1 && a.n <= kLeanRanks) {
      LeanReduceArgs lean;
      for (int k = 0; k < kLeanRanks; ++k) lean.ptr[k] = k < a.n ? a.ptr[k] : nullptr;
      lean.job[0] = a.job[0];
      lean.n = a.n;
      lean.flags = a.flags;
      return launch_vec_args<DT, OP, NT, false, LeanReduceArgs>(lean, g, 1, s);
    }
  }
  return launch_vec_args<DT, OP, NT, OWN, ReduceArgs>(a, g, njobs, s);
}

template <int DT, int OP>
hipError_t launch_op(const ReduceArgs& a, const Geometry& g, int njobs, hipStream_t s) {
  if (g.own_ptrs) return launch_vec<DT, OP, 0, true>(a, g, njobs, s);
  if constexpr (OP == MCCL_SUM || OP == MCCL_AVG) {  // the ops of gradient reductions
    switch (a.n) {
      case 2: return launch_vec<DT, OP, 2, false>(a, g, njobs, s);
      case 4: return launch_vec<DT, OP, 4, false>(a, g, njobs, s);
      case 8: return launch_vec<DT, OP, 8, false>(a, g, njobs, s);
      default: break;
    }
  }
  return launch_vec<DT, OP, 0, false>(a, g, njobs, s);
}

template <int DT>
hipError_t launch_dtype(const ReduceArgs& a, int op, const Geometry& g, int njobs, hipStream_t s) {
  switch (op) {
    case MCCL_SUM: return launch_op<DT, MCCL_SUM>(a, g, njobs, s);
    case MCCL_PROD: return launch_op<DT, MCCL_PROD>(a, g, njobs, s);
    case MCCL_MIN: return launch_op<DT, MCCL_MIN>(a, g, njobs, s);
    case MCCL_MAX: return launch_op<DT, MCCL_MAX>(a, g, njobs, s);
    case MCCL_AVG:
      if constexpr (Elem<DT>::kIsFloat) return launch_op<DT, MCCL_AVG>(a, g, njobs, s);
      else return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
  }
}

// The one-launch small allreduce: `groups` workgroups of up to sixteen wavefronts.
template <int DT>
hipError_t launch_fused_dtype(const FusedArgs& a, int op, unsigned groups, hipStream_t s) {
  if (groups < 1 || a.tiles < 1) return hipErrorInvalidValue;
  const unsigned waves = a.tiles < (unsigned)kFusedWavesPerGroup ? a.tiles : (unsigned)kFusedWavesPerGroup;
  const dim3 grid(groups, 1, 1), block(kWave * waves);
  switch (op) {
    case MCCL_SUM: hipLaunchKernelGGL((allreduce_fused_kernel<DT, MCCL_SUM>), grid, block, 0, s, a); break;
    case MCCL_PROD: hipLaunchKernelGGL((allreduce_fused_kernel<DT, MCCL_PROD>), grid, block, 0, s, a); break;
    case MCCL_MIN: hipLaunchKernelGGL((allreduce_fused_kernel<DT, MCCL_MIN>), grid, block, 0, s, a); break;
    case MCCL_MAX: hipLaunchKernelGGL((allreduce_fused_kernel<DT, MCCL_MAX>), grid, block, 0, s, a); break;
    case MCCL_AVG:
      if constexpr (Elem<DT>::kIsFloat) {
        hipLaunchKernelGGL((allreduce_fused_kernel<DT, MCCL_AVG>), grid, block, 0, s, a);
        break;
      } else {
        return hipErrorInvalidValue;
      }
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// Workgroups of `kernel` (of `block` work-items) a launch that waits for `ranks` launches at its
// start may have: this rank's share of HALF of what the kernel's register use lets the GPU hold at
// once.  The other half is room for whatever a late rank still has to run before it can join -- a
// budget equal to the whole residency (which a fixed 4096 wavefronts once was, for a kernel of 114
// registers) lets seven waiting ranks fill every slot.
template <typename K>
unsigned blocks_per_cu(K kernel, int block) {
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block, 0) != hipSuccess || per_cu < 1) {
    (void)hipGetLastError();
    per_cu = 1;
  }
  return (unsigned)per_cu;
}
inline unsigned waiting_share(unsigned per_cu, unsigned cus, unsigned ranks) {
  const uint64_t share = (uint64_t)per_cu * cus / 2u / (ranks ? ranks : 1u);
  return share ? (unsigned)share : 1u;
}

// The one-launch cross-rank reduction (reduce_scatter, in-place allreduce): grid of `groups`
// workgroups, single wavefronts or (packed) kPackedWaves wavefronts each.  waiting_ranks > 0: the
// launch waits for its peers at its start, so its grid is cut to this rank's share of the GPU
// (the kernel walks its tiles with whatever grid it gets).
template <int DT, int OP, int WPG>
hipError_t launch_xrank_kernel(const XRankArgs& a, unsigned groups, unsigned lds, unsigned cus, unsigned waiting_ranks, hipStream_t s) {
  if (a.in_table) {
    // addresses from device memory: behind a barrier kernel only (no opening wait, single wavefronts)
    if constexpr (WPG == 1) {
      if (waiting_ranks) return hipErrorInvalidValue;
      hipLaunchKernelGGL((xrank_reduce_kernel<DT, OP, 1, 1>), dim3(groups, 1, 1), dim3(kWave), lds, s, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidValue;
    }
  }
  if (a.imports) {
    // the launch exchanges the offers itself: the one-launch form on few compute units (packed)
    if constexpr (WPG == kPackedWaves) {
      if (!waiting_ranks) return hipErrorInvalidValue;
      static const unsigned per_cu = blocks_per_cu(xrank_reduce_kernel<DT, OP, kPackedWaves, 2>, kWave * kPackedWaves);
      const unsigned cap = waiting_share(per_cu, cus, waiting_ranks);
      if (groups > cap) groups = cap;
      hipLaunchKernelGGL((xrank_reduce_kernel<DT, OP, kPackedWaves, 2>), dim3(groups, 1, 1), dim3(kWave * kPackedWaves), lds, s, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidValue;
    }
  }
  if (waiting_ranks) {
    static const unsigned per_cu = blocks_per_cu(xrank_reduce_kernel<DT, OP, WPG, 0>, kWave * WPG);  // asked once per kernel
    const unsigned cap = waiting_share(per_cu, cus, waiting_ranks);
    if (groups > cap) groups = cap;
  }
  hipLaunchKernelGGL((xrank_reduce_kernel<DT, OP, WPG, 0>), dim3(groups, 1, 1), dim3(kWave * WPG), lds, s, a);
  return hipGetLastError();
}

template <int DT, int WPG>
hipError_t launch_xrank_packing(const XRankArgs& a, int op, unsigned groups, unsigned lds, unsigned cus, unsigned waiting_ranks, hipStream_t s) {
  switch (op) {
    case MCCL_SUM: return launch_xrank_kernel<DT, MCCL_SUM, WPG>(a, groups, lds, cus, waiting_ranks, s);
    case MCCL_PROD: return launch_xrank_kernel<DT, MCCL_PROD, WPG>(a, groups, lds, cus, waiting_ranks, s);
    case MCCL_MIN: return launch_xrank_kernel<DT, MCCL_MIN, WPG>(a, groups, lds, cus, waiting_ranks, s);
    case MCCL_MAX: return launch_xrank_kernel<DT, MCCL_MAX, WPG>(a, groups, lds, cus, waiting_ranks, s);
    case MCCL_AVG:
      if constexpr (Elem<DT>::kIsFloat) return launch_xrank_kernel<DT, MCCL_AVG, WPG>(a, groups, lds, cus, waiting_ranks, s);
      else return hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
  }
}

template <int DT>
hipError_t launch_xrank_dtype(const XRankArgs& a, int op, unsigned groups, int packed, unsigned lds, unsigned cus, unsigned waiting_ranks, hipStream_t s) {
  return packed ? launch_xrank_packing<DT, kPackedWaves>(a, op, groups, lds, cus, waiting_ranks, s)
                : launch_xrank_packing<DT, 1>(a, op, groups, lds, cus, waiting_ranks, s);
}

}  // namespace

// Entry points of the per-type translation units.  Plain types only: the argument block and the
// geometry live in unnamed namespaces and are therefore distinct types in every translation unit
// (with one layout).  `reduce_args` points at a ReduceArgs.
#define MCCL_REDUCE_ENTRY_ARGS                                                                 \
  const void *reduce_args, int op, int shape, unsigned grid_x, unsigned lds, int own_ptrs, int njobs, \
      hipStream_t stream
extern "C" {
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt0(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt1(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt2(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt3(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt4(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt5(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt6(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt7(MCCL_REDUCE_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_reduce_dt8(MCCL_REDUCE_ENTRY_ARGS);
}
// `fused_args` points at a FusedArgs.
#define MCCL_FUSED_ENTRY_ARGS const void *fused_args, int op, unsigned groups, hipStream_t stream
extern "C" {
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt0(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt1(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt2(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt3(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt4(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt5(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt6(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt7(MCCL_FUSED_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_fused_dt8(MCCL_FUSED_ENTRY_ARGS);
// `xrank_args` points at an XRankArgs; lds = dynamic LDS bytes reserved per workgroup (residency cap);
// waiting_ranks > 0: the launch waits for that many ranks' launches and is cut to its share of `cus` compute units
#define MCCL_XRANK_ENTRY_ARGS \
  const void *xrank_args, int op, unsigned groups, int packed, unsigned lds, unsigned cus, unsigned waiting_ranks, hipStream_t stream
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt0(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt1(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt2(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt3(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt4(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt5(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt6(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt7(MCCL_XRANK_ENTRY_ARGS);
__attribute__((visibility("hidden"))) hipError_t mccl_launch_xrank_dt8(MCCL_XRANK_ENTRY_ARGS);
}
