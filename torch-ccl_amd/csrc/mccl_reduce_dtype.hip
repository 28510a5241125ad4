// One element type of the reduction kernels per translation unit: compiled once for every
// mccl_dtype_t code with -DMCCL_REDUCE_DT=<code> (see build.py), linked into libmi355ccl.so.
#include <hip/hip_runtime.h>

#include "mccl.h"

#include "reduce_launch.hpp"

#ifndef MCCL_REDUCE_DT
#error "compile with -DMCCL_REDUCE_DT=<mccl_dtype_t code>"
#endif

#define MCCL_PASTE2(a, b) a##b
#define MCCL_PASTE(a, b) MCCL_PASTE2(a, b)

extern "C" hipError_t MCCL_PASTE(mccl_launch_reduce_dt, MCCL_REDUCE_DT)(MCCL_REDUCE_ENTRY_ARGS) {
  Geometry g;
  g.shape = (Shape)shape;
  g.grid_x = grid_x;
  g.block = shape == kShapePersistent ? kBlockPersistent : kWave;
  g.lds = lds;
  g.own_ptrs = own_ptrs != 0;
  g.stream_out = false;  // travels in the argument block's flags
  return launch_dtype<MCCL_REDUCE_DT>(*static_cast<const ReduceArgs*>(reduce_args), op, g, njobs, stream);
}

extern "C" hipError_t MCCL_PASTE(mccl_launch_fused_dt, MCCL_REDUCE_DT)(MCCL_FUSED_ENTRY_ARGS) {
  return launch_fused_dtype<MCCL_REDUCE_DT>(*static_cast<const FusedArgs*>(fused_args), op, groups, stream);
}

extern "C" hipError_t MCCL_PASTE(mccl_launch_xrank_dt, MCCL_REDUCE_DT)(MCCL_XRANK_ENTRY_ARGS) {
  return launch_xrank_dtype<MCCL_REDUCE_DT>(*static_cast<const XRankArgs*>(xrank_args), op, groups, packed, lds, cus, waiting_ranks, stream);
}
