// libmi355ccl: launch planning and the C ABI declared in include/mccl.h.  The device code is in
// kernels_common.hpp (element types, the reduction chain), kernels_reduce.hpp, kernels_copy.hpp
// and kernels_moe.hpp.
//
// Everything here is HBM-bandwidth bound.  Design rules:
//   * one 16-byte vector per lane per input, so a wavefront reads 1 KiB contiguous from
//     each of the N inputs; all N (x unroll) loads of a tile are issued before the first
//     add so the memory system sees N*U independent requests per lane;
//   * accumulation is a sequential ascending-rank chain held in registers (fp32 for
//     f16/bf16), one round-to-nearest-even on store;
//   * large outputs are written with streaming stores (written through past the caches at
//     agent scope): worth 2-5 % against plain stores, most on multi-GiB footprints; small
//     outputs stay cacheable for their consumer;
//   * inputs are read with non-temporal loads: nothing is reused, and on this part the
//     streaming hint alone is worth about 12 % of bandwidth;
//   * launch shapes (same kernel code, different geometry):
//       small      one wavefront per workgroup, one vector per lane, grid covers the
//                  message: a 256 KiB message lands on all 256 CUs in one launch;
//       stream     the same geometry plus a dynamic-LDS reservation that caps residency at
//                  W wavefronts per CU, W chosen so that about 64 KiB of loads are in
//                  flight per CU.  The hardware dispatcher hands out tiles in address
//                  order, so the set of live tiles is a compact window that sweeps the
//                  buffers; with more resident wavefronts the window widens, DRAM pages
//                  are re-opened more often and bandwidth drops (measured: 84-87 % of peak
//                  at W = 7-8 for eight inputs against 75 % uncapped);
//       persistent a fixed grid proportional to the CU count walking tiles grid-stride.
//                  Slower than "stream" on large messages (the workgroups drift apart and
//                  the live window smears) but a few percent ahead while the whole working
//                  set fits the 256 MB Infinity Cache, which is where AUTO uses it;
//   * misaligned heads/tails are peeled element-wise inside the same launch up to the first
//     128-byte boundary of the output (whole cache lines per tile); inputs that are not
//     congruent with the output mod 16 are read with unaligned vector loads (the hardware
//     splits them).
//
// What each kernel replaces in the reference (intel/torch-ccl):
//   reduce_vec_kernel : the N-peer sum of src/gpu/allreduce_small.h:289-361,
//       the five data kernels of src/gpu/allreduce.h:306-533, ccl::allreduce /
//       ccl::reduce_scatter call sites in src/gpu/dpcpp_ccl.cpp:781-788, 1002-1008
//   rank_barrier_kernel : the one-thread sync kernels between the data kernels of
//       src/gpu/allreduce.h:731-769, 835-877
//   allreduce_fused_kernel : the whole small allreduce of src/gpu/allreduce_small.h:166-361
//       (copy-in, rank barrier, N-peer sum in one launch)
//   copy_segments_kernel : ccl::allgatherv / ccl::alltoall(v) data movement
//       (src/gpu/dpcpp_ccl.cpp:1176-1182, 1403-1455) and the pack/unpack copy_ loops
//       (src/gpu/dpcpp_ccl.cpp:1505-1538)
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <mutex>
#include <vector>

#include "mccl.h"

#include "kernels_common.hpp"
#include "kernels_copy.hpp"
#include "kernels_moe.hpp"
#include "kernels_sync.hpp"
#include "reduce_launch.hpp"

namespace {

// ------------------------------------------------------------------------------------------
// error plumbing
// ------------------------------------------------------------------------------------------
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(expr)                                                                   \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess)                                                               \
      return fail(MCCL_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),  \
                  __FILE__, __LINE__);                                                  \
  } while (0)

// ------------------------------------------------------------------------------------------
// tuning state and per-device facts
// ------------------------------------------------------------------------------------------
constexpr unsigned kMaxGridX = 1u << 24;  // larger messages wrap through the grid-stride loop
// Chunk counters are 32 bits wide and advance by the grid size: the limit leaves room for the
// last step past the end.
constexpr uint64_t kMaxChunks = 0xf0000000ull;
constexpr size_t kLdsPerCu = 160 * 1024;  // gfx950
constexpr int kBatchedSegs = 256;  // segments of an all-to-all collected before they are handed to the launcher
constexpr int kMaxWavesPerCu = 32;

// tunables (mccl_set_tuning); defaults come from sweeps on MI355X.  Read by every launch and
// written by whoever sweeps them, possibly from another thread: relaxed atomics.
constexpr long long kTuneDefault[MCCL_TUNE_COUNT_] = {
    /* PERSISTENT_BLOCKS_PER_CU */ 8,
    /* STREAM_WAVES_PER_CU      */ 0,
    /* SMALL_MAX_BYTES          */ 4 << 20,
    /* COPY_WAVES_PER_CU        */ 24,
    /* STREAM_MIN_TOTAL_BYTES   */ 112ll << 20,
    /* COMBINE_PIECES_PER_WAVE  */ 2,
    /* COMBINE_WAVES_PER_CU     */ 0,
    /* XRANK_WAVES_ALL_RANKS    */ 4096,
    /* COPY_VECTORS_PER_LANE    */ 1,  // neither 2 nor 4: chosen by size
    /* COPY_STREAM_STORES       */ 3,  // neither 1 nor 2: chosen by size
    /* COPY_LARGE_MIN_BYTES     */ 1ll << 30,
    /* GATHER_WAVES_PER_CU      */ 28,
    /* XRANK_CACHED_LOADS       */ 2,
    /* XRANK_FRESH_WAVES_PER_CU */ 32,
    /* XRANK_FRESH_MAX_WAVES    */ 0,
};
constexpr int kCopyUnrollLarge = 2;   // vectors per lane per chunk of large copies
constexpr int kCopyStreamLarge = 1;   // store flavour of large copies: 1 = written through (sc1), 2 = non-temporal
struct TuneTable {
  std::atomic<long long> v[MCCL_TUNE_COUNT_];
  TuneTable() {
    for (int i = 0; i < MCCL_TUNE_COUNT_; ++i) v[i].store(kTuneDefault[i], std::memory_order_relaxed);
  }
  long long operator[](int knob) const { return v[knob].load(std::memory_order_relaxed); }
  void set(int knob, long long value) { v[knob].store(value, std::memory_order_relaxed); }
};
TuneTable g_tune;

// Dynamic-LDS bytes that limit residency to `waves` single-wavefront workgroups per CU
// (0 = no reservation needed).
unsigned lds_for_waves(long long waves) {
  if (waves >= kMaxWavesPerCu) return 0;
  if (waves < 1) waves = 1;
  size_t b = (kLdsPerCu / (size_t)waves) & ~(size_t)511;
  if (b > 64 * 1024) b = 64 * 1024;
  return (unsigned)b;
}

struct DeviceFacts {
  int cus = 0;
};
DeviceFacts g_facts[64];
std::once_flag g_facts_once[64];

int device_cus(int* cus_out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(MCCL_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  hipError_t err = hipSuccess;
  std::call_once(g_facts_once[dev], [&]() {
    int cus = 0;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    g_facts[dev].cus = cus > 0 ? cus : 256;
  });
  if (err != hipSuccess) return fail(MCCL_ERR_HIP, "hipDeviceGetAttribute failed: %s", hipGetErrorString(err));
  *cus_out = g_facts[dev].cus;
  return MCCL_OK;
}

// ------------------------------------------------------------------------------------------
// host-side launch helpers
// ------------------------------------------------------------------------------------------
bool valid_dtype(int dt) { return dt >= MCCL_U8 && dt <= MCCL_BF16; }
bool valid_op(int op) { return op == MCCL_SUM || op == MCCL_AVG || op == MCCL_PROD || op == MCCL_MIN || op == MCCL_MAX; }
bool float_dtype(int dt) { return dt == MCCL_F16 || dt == MCCL_F32 || dt == MCCL_F64 || dt == MCCL_BF16; }

size_t dtype_size(int dt) {
  switch (dt) {
    case MCCL_U8: case MCCL_I8: return 1;
    case MCCL_I16: case MCCL_F16: case MCCL_BF16: return 2;
    case MCCL_I32: case MCCL_F32: return 4;
    case MCCL_I64: case MCCL_F64: return 8;
    default: return 0;
  }
}

hipError_t launch_any(const ReduceArgs& a, int dtype, int op, const Geometry& g, int njobs, hipStream_t s) {
  const int own = g.own_ptrs ? 1 : 0;
  switch (dtype) {
    case MCCL_U8: return mccl_launch_reduce_dt0(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_I8: return mccl_launch_reduce_dt1(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_I16: return mccl_launch_reduce_dt2(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_I32: return mccl_launch_reduce_dt3(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_I64: return mccl_launch_reduce_dt4(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_F16: return mccl_launch_reduce_dt5(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_F32: return mccl_launch_reduce_dt6(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_F64: return mccl_launch_reduce_dt7(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    case MCCL_BF16: return mccl_launch_reduce_dt8(&a, op, g.shape, g.grid_x, g.lds, own, njobs, s);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_fused_any(const FusedArgs& a, int dtype, int op, unsigned groups, hipStream_t s) {
  switch (dtype) {
    case MCCL_U8: return mccl_launch_fused_dt0(&a, op, groups, s);
    case MCCL_I8: return mccl_launch_fused_dt1(&a, op, groups, s);
    case MCCL_I16: return mccl_launch_fused_dt2(&a, op, groups, s);
    case MCCL_I32: return mccl_launch_fused_dt3(&a, op, groups, s);
    case MCCL_I64: return mccl_launch_fused_dt4(&a, op, groups, s);
    case MCCL_F16: return mccl_launch_fused_dt5(&a, op, groups, s);
    case MCCL_F32: return mccl_launch_fused_dt6(&a, op, groups, s);
    case MCCL_F64: return mccl_launch_fused_dt7(&a, op, groups, s);
    case MCCL_BF16: return mccl_launch_fused_dt8(&a, op, groups, s);
    default: return hipErrorInvalidValue;
  }
}

// waiting_ranks > 0: the launch waits for that many ranks' launches at its start and is cut to its
// share of the GPU's residency (reduce_launch.hpp: waiting_share).
hipError_t launch_xrank_any(const XRankArgs& a, int dtype, int op, unsigned groups, int packed, unsigned lds, unsigned waiting_ranks, hipStream_t s) {
  int cus_i = 0;
  if (device_cus(&cus_i) != MCCL_OK) return hipErrorInvalidDevice;
  const unsigned cus = (unsigned)cus_i;
  switch (dtype) {
    case MCCL_U8: return mccl_launch_xrank_dt0(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_I8: return mccl_launch_xrank_dt1(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_I16: return mccl_launch_xrank_dt2(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_I32: return mccl_launch_xrank_dt3(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_I64: return mccl_launch_xrank_dt4(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_F16: return mccl_launch_xrank_dt5(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_F32: return mccl_launch_xrank_dt6(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_F64: return mccl_launch_xrank_dt7(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    case MCCL_BF16: return mccl_launch_xrank_dt8(&a, op, groups, packed, lds, cus, waiting_ranks, s);
    default: return hipErrorInvalidValue;
  }
}

// Ticks of the 100 MHz wall clock a device-side wait may last; 0 asks for the default of 10 s.
constexpr uint64_t kTicksPerUs = 100;
uint64_t wait_limit_ticks(uint64_t timeout_us) {
  if (timeout_us == 0) timeout_us = 10ull * 1000 * 1000;
  if (timeout_us > 3600ull * 1000 * 1000) timeout_us = 3600ull * 1000 * 1000;
  return timeout_us * kTicksPerUs;
}

// Loads one wavefront keeps in flight per tile: all ranks up to eight (compile-time rank counts
// and the generic path alike, which loads in groups of eight).
int loads_in_flight(int n, int /*op*/, bool /*own_ptrs*/) { return n < 8 ? n : 8; }

// Resident wavefronts per CU of the stream shape.  Enough loads in flight to cover the memory
// latency at full bandwidth (about 14 MB over the chip), and no more: every further wavefront
// widens the window of live tiles and costs DRAM page locality.  Measured optima on MI355X
// (bf16, 64 MiB per rank; % of the HBM peak at the optimum / two wavefronts off it):
//   loads in flight   SUM, AVG, PROD          MIN, MAX (compare + select per element: more ALU
//                                             work per byte wants more wavefronts to hide it)
//   8                 8   (87 / 84)           12  (83 / 78 at 9, 74 at 8)
//   7                 10  (86 / 80 at 7)      12
//   6                 11  (85 / 81 at 8)      14
//   5                 12  (84 / 79 at 9)      14  (85 / 80 at 12)
//   4                 14  (85 / 80 at 9)      14  (86 / 77 at 12)
//   3 or fewer        no cap (85 against 81 at 14 wavefronts for three loads)
long long stream_waves(int n, int op, bool own_ptrs) {
  if (g_tune[MCCL_TUNE_STREAM_WAVES_PER_CU] > 0) return g_tune[MCCL_TUNE_STREAM_WAVES_PER_CU];
  const int loads = loads_in_flight(n, op, own_ptrs);
  if (loads <= 3) return kMaxWavesPerCu;
  if (op == MCCL_MIN || op == MCCL_MAX) return loads >= 7 ? 12 : 14;
  switch (loads) {
    case 8: return 8;
    case 7: return 10;
    case 6: return 11;
    case 5: return 12;
    default: return 14;
  }
}

// Geometry of a vector launch over njobs jobs whose largest has max_count elements.
int plan_vec(size_t max_count, int njobs, int n, int dtype, int op, int variant, bool own_ptrs,
             Geometry* g) {
  int cus = 0;
  int rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  const size_t es = dtype_size(dtype);
  const size_t nvec = max_count / (16 / es) + 1;
  // Measured crossovers on MI355X.  Up to a few MiB per rank a launch is latency-bound: one
  // wavefront per tile, cacheable output.  From about 112 MiB of traffic per launch the capped
  // in-order stream with a streamed (written-through) output wins by 3-15 %.  In between, four or
  // more ranks do best with the persistent grid and a cacheable output (the working set sits in
  // the Infinity Cache, where a streamed output costs up to 20 %); with fewer ranks the output is
  // a third or more of the traffic and streaming it pays from 8 MiB per rank on.
  const size_t per_rank = max_count * es;
  const size_t total = per_rank * (size_t)(n + 1) * (size_t)njobs;
  const bool small_msg = per_rank <= (size_t)g_tune[MCCL_TUNE_SMALL_MAX_BYTES];
  const bool large_msg = total >= (size_t)g_tune[MCCL_TUNE_STREAM_MIN_TOTAL_BYTES];
  // MIN / MAX of two ranks: a wavefront of the stream shape has two loads in flight and then a
  // compare, a NaN test and a select per element, which at full residency leaves the memory
  // pipeline short (78-80 % of peak against 84 % for SUM).  Two vectors per lane, i.e. the
  // persistent kernel on a grid of 64 workgroups per CU, brings it to 83.7 %.
  const bool two_rank_minmax = variant == MCCL_VARIANT_AUTO && n == 2 && (op == MCCL_MIN || op == MCCL_MAX);
  Shape shape;
  switch (variant) {
    case MCCL_VARIANT_SMALL: shape = kShapeSmall; break;
    case MCCL_VARIANT_PERSISTENT: shape = kShapePersistent; break;
    case MCCL_VARIANT_STREAM: shape = kShapeStream; break;
    case MCCL_VARIANT_AUTO:
      if (small_msg) shape = kShapeSmall;
      else if (large_msg) shape = two_rank_minmax ? kShapePersistent : kShapeStream;
      else shape = n >= 4 ? kShapePersistent : kShapeSmall;
      break;
    default: return fail(MCCL_ERR_INVALID_ARG, "unknown variant %d", variant);
  }
  g->stream_out = !small_msg && (large_msg || n < 4);
  g->shape = shape;
  g->lds = 0;
  g->own_ptrs = own_ptrs;
  if (shape == kShapePersistent) {
    const size_t tile = (size_t)kBlockPersistent * kUnrollPersistent;
    size_t tiles = (nvec + tile - 1) / tile;
    const size_t per_cu = (two_rank_minmax && large_msg) ? 64 : (size_t)g_tune[MCCL_TUNE_PERSISTENT_BLOCKS_PER_CU];
    size_t want = (size_t)cus * per_cu / (size_t)njobs;
    if (want < 1) want = 1;
    if (tiles > want) tiles = want;
    g->grid_x = (unsigned)(tiles ? tiles : 1);
    g->block = kBlockPersistent;
  } else {
    size_t tiles = (nvec + kWave - 1) / kWave;
    if (tiles > kMaxGridX) tiles = kMaxGridX;
    g->grid_x = (unsigned)(tiles ? tiles : 1);
    g->block = kWave;
    if (shape == kShapeStream) g->lds = lds_for_waves(stream_waves(n, op, own_ptrs));
  }
  return MCCL_OK;
}

// A reduction as the entry points describe it, before the host splits it for the kernels.
struct JobSpec {
  char* out;
  size_t in_off;
  size_t count;
  int ptr0;
};

// Launch one batch of jobs.  a.ptr / a.n are populated; specs describe the jobs.  The vector
// body of a job starts at the first 128-byte boundary of its output (full cache lines per
// tile); inputs need element alignment only.
int launch_jobs(ReduceArgs& a, const JobSpec* specs, int njobs, int dtype, int op, int variant,
                bool own_ptrs, hipStream_t s) {
  const size_t es = dtype_size(dtype);
  const size_t ve = 16 / es;
  int nv = 0;
  size_t vmax = 0;
  for (int j = 0; j < njobs; ++j) {
    const JobSpec& sp = specs[j];
    if (sp.count == 0) continue;
    const uintptr_t o = (uintptr_t)sp.out;
    if (o % es) return fail(MCCL_ERR_INVALID_ARG, "output pointer not aligned to the element size");
    for (int k = 0; k < a.n; ++k) {
      const uintptr_t p = (uintptr_t)(a.ptr[sp.ptr0 + k] + sp.in_off);
      if (p % es) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d not aligned to the element size", k);
    }
    size_t head = ((128u - (unsigned)(o & 127u)) & 127u) / es;  // the body starts on a cache line of out
    if (head > sp.count) head = sp.count;
    const size_t nvec = (sp.count - head) / ve;
    if (nvec / kWave > kMaxChunks) return fail(MCCL_ERR_INVALID_ARG, "message too large");
    ReduceJob& jb = a.job[nv];
    jb.out = sp.out;
    jb.in_off = sp.in_off;
    jb.nvec = nvec;
    jb.head = (uint32_t)head;
    jb.tail = (uint32_t)(sp.count - head - nvec * ve);
    a.job_ptr0[nv] = sp.ptr0;
    ++nv;
    if (sp.count > vmax) vmax = sp.count;
  }
  // An output may be exactly the input range its own job reads from one rank (in place); any
  // other overlap with something this launch reads or writes would race between wavefronts.
  // Checked with a sort and one sweep over the byte ranges (jobs x (ranks + 1) of them), not pair
  // by pair: a coalesced launch of 64 buckets from 64 ranks has 4160 ranges.
  {
    struct Range {
      uintptr_t lo, hi;
      int job, rank;  // rank < 0: the job's output
    };
    static thread_local std::vector<Range> ranges;
    ranges.clear();
    for (int j = 0; j < nv; ++j) {
      const size_t bytes = (a.job[j].head + a.job[j].nvec * ve + a.job[j].tail) * es;
      const uintptr_t o0 = (uintptr_t)a.job[j].out;
      ranges.push_back(Range{o0, o0 + bytes, j, -1});
      for (int k = 0; k < a.n; ++k) {
        const uintptr_t p0 = (uintptr_t)(a.ptr[a.job_ptr0[j] + k] + a.job[j].in_off);
        if (p0 != o0) ranges.push_back(Range{p0, p0 + bytes, j, k});  // p0 == o0: in place, allowed
      }
    }
    std::sort(ranges.begin(), ranges.end(), [](const Range& x, const Range& y) { return x.lo < y.lo; });
    const Range* far_any = nullptr;  // the earlier range that reaches farthest
    const Range* far_out = nullptr;  // the earlier output that reaches farthest
    for (const Range& r : ranges) {
      const Range* hit = nullptr;
      if (r.rank < 0) {
        if (far_any && far_any->hi > r.lo) hit = far_any;
      } else if (far_out && far_out->hi > r.lo) {
        hit = far_out;
      }
      if (hit) {
        const Range& out_r = r.rank < 0 ? r : *hit;
        const Range& other = r.rank < 0 ? *hit : r;
        if (other.rank < 0) return fail(MCCL_ERR_INVALID_ARG, "outputs %d and %d overlap", out_r.job, other.job);
        return fail(MCCL_ERR_INVALID_ARG, "output %d partially overlaps input %d of reduction %d", out_r.job, other.rank, other.job);
      }
      if (!far_any || r.hi > far_any->hi) far_any = &r;
      if (r.rank < 0 && (!far_out || r.hi > far_out->hi)) far_out = &r;
    }
  }
  if (nv) {
    Geometry g;
    int rc = plan_vec(vmax, nv, a.n, dtype, op, variant, own_ptrs, &g);
    if (rc != MCCL_OK) return rc;
    // outputs of launches that move more than the Infinity Cache holds are streamed past the
    // caches (2-5 % of bandwidth); smaller ones stay cacheable for whoever reads them next
    a.flags = g.stream_out ? kFlagStreamOut : 0u;
    hipError_t e = launch_any(a, dtype, op, g, nv, s);
    if (e != hipSuccess) return fail(MCCL_ERR_HIP, "reduce kernel launch failed: %s", hipGetErrorString(e));
  }
  return MCCL_OK;
}

int check_reduce_args_no_ptr(int n, int dtype, int op);

int check_reduce_args(const void* const* in, int n, int dtype, int op) {
  if (!in) return fail(MCCL_ERR_INVALID_ARG, "input pointer table is null");
  return check_reduce_args_no_ptr(n, dtype, op);
}

int check_reduce_args_no_ptr(int n, int dtype, int op) {
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  if (!valid_dtype(dtype)) return fail(MCCL_ERR_INVALID_ARG, "unknown dtype code %d", dtype);
  if (!valid_op(op)) return fail(MCCL_ERR_INVALID_ARG, "unknown reduce op code %d", op);
  if (op == MCCL_AVG && !float_dtype(dtype)) return fail(MCCL_ERR_UNSUPPORTED, "AVG is defined for floating-point types only");
  return MCCL_OK;
}

int launch_copy(const mccl_segment_t* segs, int nseg, hipStream_t s) {
  size_t total_bytes = 0;
  for (int k = 0; k < nseg; ++k) {  // refusals first, before anything is enqueued
    if (segs[k].bytes && (!segs[k].src || !segs[k].dst)) return fail(MCCL_ERR_INVALID_ARG, "segment %d has a null pointer", k);
    total_bytes += segs[k].bytes;
  }
  int cus = 0;
  int rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  // Geometry of the call: vectors per lane per chunk and the flavour of the full-chunk stores.
  // Tunable for sweeps; the defaults follow the total size.  Measured on MI355X (C5: 64 segments,
  // 3.5 GiB moved; a 512 MiB single-segment copy), % of the HBM peak of 2 x bytes moved:
  //   2 vectors per lane, nt stores:  C5 81.6 at 24 wavefronts per CU (80.8 at 28, 77.7 at 20), copy 83.5
  //   2 vectors per lane, sc1 stores: C5 83.7 at 24 (82.8 at 20, 78.6 at 28),                  copy 82.9
  //   4 vectors per lane (4 KiB per wavefront): 81.5 / 81.6 at 16 wavefronts, lower everywhere else
  // so chunks stay at 2 KiB, 24 wavefronts are resident per CU, and calls that move 1 GiB or more
  // write their full chunks through past the caches.
  long long unroll = g_tune[MCCL_TUNE_COPY_VECTORS_PER_LANE];
  if (unroll != 2 && unroll != 4) unroll = total_bytes >= (size_t)g_tune[MCCL_TUNE_COPY_LARGE_MIN_BYTES] ? kCopyUnrollLarge : kCopyUnroll;
  long long stream_store = g_tune[MCCL_TUNE_COPY_STREAM_STORES];
  if (stream_store != 1 && stream_store != 2) stream_store = total_bytes >= (size_t)g_tune[MCCL_TUNE_COPY_LARGE_MIN_BYTES] ? kCopyStreamLarge : 2;
  const size_t chunk_bytes = (size_t)kWave * 16 * (size_t)unroll;
  int i = 0;
  while (i < nseg) {
    CopyArgs a;
    int m = 0;
    uint64_t chunks = 0;
    a.chunk_prefix[0] = 0;
    while (i < nseg && m < kMaxSegs) {
      const mccl_segment_t& sg = segs[i];
      if (sg.bytes == 0) { ++i; continue; }
      const uintptr_t dp = (uintptr_t)sg.dst;
      CopySeg cs;
      cs.src = (const char*)sg.src;
      cs.dst = (char*)sg.dst;
      cs.pad_ = 0;
      size_t head = (128u - (unsigned)(dp & 127u)) & 127u;  // the body starts on a cache line of dst
      if (head > sg.bytes) head = sg.bytes;
      const size_t body = sg.bytes - head;
      const uint64_t nfull = body / chunk_bytes;
      cs.head = (uint32_t)head;
      cs.last = (uint32_t)(body % chunk_bytes);
      uint64_t c = nfull + (cs.last ? 1 : 0);
      if (c == 0) c = 1;  // head only: chunk 0 still has to run
      if (nfull > 0xf0000000ull || chunks + c > kMaxChunks) {
        if (m == 0) return fail(MCCL_ERR_INVALID_ARG, "segment %d too large", i);
        break;
      }
      cs.nfull = (uint32_t)nfull;
      a.seg[m] = cs;
      chunks += c;
      a.chunk_prefix[++m] = (uint32_t)chunks;
      ++i;
    }
    if (m == 0) break;
    a.nseg = m;
    uint64_t grid = chunks;
    if (grid > kMaxGridX) grid = kMaxGridX;
    // small copies are latency bound: no residency cap below 4 chunks per CU
    const unsigned lds = (chunks > (uint64_t)cus * 4) ? lds_for_waves(g_tune[MCCL_TUNE_COPY_WAVES_PER_CU]) : 0;
    const dim3 g3((unsigned)grid), b3(kWave);
    if (unroll == 4) {
      if (stream_store == 1) hipLaunchKernelGGL((copy_segments_kernel<4, true>), g3, b3, lds, s, a);
      else hipLaunchKernelGGL((copy_segments_kernel<4, false>), g3, b3, lds, s, a);
    } else {
      if (stream_store == 1) hipLaunchKernelGGL((copy_segments_kernel<2, true>), g3, b3, lds, s, a);
      else hipLaunchKernelGGL((copy_segments_kernel<2, false>), g3, b3, lds, s, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MCCL_ERR_HIP, "copy kernel launch failed: %s", hipGetErrorString(e));
  }
  return MCCL_OK;
}

// Launches gather segments in batches of kMaxSegs.
struct GatherSpec {
  const void* src;
  size_t src_rows;
  const int64_t* idx;
  void* dst;
  size_t nrows;
};

int launch_gather(const GatherSpec* specs, int nspec, size_t row_bytes, hipStream_t s) {
  if (row_bytes == 0) return MCCL_OK;
  if (row_bytes > 0x7fffffffull) return fail(MCCL_ERR_INVALID_ARG, "row of %zu bytes is too long", row_bytes);
  const uint32_t ppr = (uint32_t)((row_bytes + kCopyChunk - 1) / kCopyChunk);
  // Rows that are not a whole number of 2 KiB pieces are moved as 2 KiB windows of the
  // destination (several small rows, or the end of one row and the start of the next, per
  // wavefront): one piece of one row per wavefront leaves lanes idle (1 KiB rows: 4.6 TB/s against
  // 7.0 this way).  Needs rows and buffers that are multiples of 16 bytes.
  bool flat = row_bytes % kCopyChunk != 0 && row_bytes % 16 == 0;
  for (int k = 0; flat && k < nspec; ++k)
    if (specs[k].nrows && (((((uintptr_t)specs[k].src) | ((uintptr_t)specs[k].dst)) & 15u) ||
                           (uint64_t)specs[k].nrows * (row_bytes / 16) >= 0xffffffffull))
      flat = false;
  int i = 0;
  while (i < nspec) {
    GatherArgs a;
    int m = 0;
    uint64_t chunks = 0;
    a.chunk_prefix[0] = 0;
    while (i < nspec && m < kMaxSegs) {
      const GatherSpec& g = specs[i];
      if (g.nrows == 0) { ++i; continue; }
      if (!g.src || !g.idx || !g.dst) return fail(MCCL_ERR_INVALID_ARG, "gather segment %d has a null pointer", i);
      if (g.nrows > 0xffffffffull || g.src_rows > 0xffffffffull)
        return fail(MCCL_ERR_INVALID_ARG, "gather segment %d has too many rows", i);
      if ((uintptr_t)g.idx % 8) return fail(MCCL_ERR_INVALID_ARG, "row index table %d is not 8-byte aligned", i);
      const uint64_t c = flat ? ((uint64_t)g.nrows * row_bytes + kCopyChunk - 1) / kCopyChunk
                              : (uint64_t)g.nrows * ppr;
      if (chunks + c > kMaxChunks) {
        if (m == 0) return fail(MCCL_ERR_INVALID_ARG, "gather segment %d too large", i);
        break;
      }
      a.seg[m] = GatherSeg{(const char*)g.src, g.idx, (char*)g.dst, (uint32_t)g.nrows, (uint32_t)g.src_rows};
      chunks += c;
      a.chunk_prefix[++m] = (uint32_t)chunks;
      ++i;
    }
    if (m == 0) break;
    a.nseg = m;
    a.row_bytes = (uint32_t)row_bytes;
    a.pieces_per_row = ppr;
    a.flat = flat ? 1u : 0u;
    int cus = 0;
    int rc = device_cus(&cus);
    if (rc != MCCL_OK) return rc;
    uint64_t grid = chunks;
    if (grid > kMaxGridX) grid = kMaxGridX;
    const unsigned lds = (chunks > (uint64_t)cus * 4) ? lds_for_waves(g_tune[MCCL_TUNE_GATHER_WAVES_PER_CU]) : 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)grid), dim3(kWave), lds, s, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MCCL_ERR_HIP, "gather kernel launch failed: %s", hipGetErrorString(e));
  }
  return MCCL_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------
extern "C" {

int mccl_version(void) { return 150; }

const char* mccl_last_error(void) { return g_err; }

size_t mccl_dtype_size(int dtype) { return dtype_size(dtype); }

int mccl_set_tuning(int knob, long long value) {
  if (knob < 0 || knob >= MCCL_TUNE_COUNT_) return fail(MCCL_ERR_INVALID_ARG, "unknown tuning knob %d", knob);
  g_tune.set(knob, value > 0 ? value : kTuneDefault[knob]);
  return MCCL_OK;
}

long long mccl_get_tuning(int knob) {
  if (knob < 0 || knob >= MCCL_TUNE_COUNT_) return -1;
  return g_tune[knob];
}

int mccl_query_launch(size_t count, int n, int dtype, int op, int variant, int* block_size,
                      int* lds_bytes) {
  int rc = check_reduce_args_no_ptr(n, dtype, op);
  if (rc != MCCL_OK) return rc;
  Geometry g;
  rc = plan_vec(count, 1, n, dtype, op, variant, false, &g);
  if (rc != MCCL_OK) return rc;
  if (block_size) *block_size = g.block;
  if (lds_bytes) *lds_bytes = (int)g.lds;
  return (int)g.grid_x;
}

int mccl_placement_check(const void* const* in, int n, size_t bytes) {
  if (!in || n < 2 || n > MCCL_MAX_RANKS) return 0;
  if (bytes < (256u << 20)) return 0;  // smaller messages have not shown the effect
  // Measured on MI355X (8 inputs, bare streaming kernel and the library's): equal spacings of
  // 256 MiB and more that are whole multiples of 2 MiB -- 256 MiB, 512 MiB, 1 GiB, and the
  // "size + 2 MiB" a caching allocator gives equal tensors of 1 GiB and more -- run at 76-81 % of
  // the HBM peak where the same buffers a further 4 KiB apart per rank run at 85-87 %.  Irregular
  // placements have not collided.
  const intptr_t d = (intptr_t)((const char*)in[1] - (const char*)in[0]);
  const uintptr_t ad = (uintptr_t)(d < 0 ? -d : d);
  if (ad < (256u << 20) || ad % (2u << 20)) return 0;
  for (int k = 2; k < n; ++k)
    if ((intptr_t)((const char*)in[k] - (const char*)in[k - 1]) != d) return 0;
  return 1;
}

int mccl_reduce_n(const void* const* in, int n, void* out, size_t count, int dtype, int op,
                  int variant, void* stream) {
  int rc = check_reduce_args(in, n, dtype, op);
  if (rc != MCCL_OK) return rc;
  if (variant < MCCL_VARIANT_AUTO || variant > MCCL_VARIANT_STREAM) return fail(MCCL_ERR_INVALID_ARG, "unknown variant %d", variant);
  if (count == 0) return MCCL_OK;
  if (!out) return fail(MCCL_ERR_INVALID_ARG, "output pointer is null");
  ReduceArgs a;
  memset(&a, 0, sizeof(a));
  for (int k = 0; k < n; ++k) {
    if (!in[k]) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d is null", k);
    a.ptr[k] = (const char*)in[k];
  }
  a.n = n;
  const JobSpec spec{(char*)out, 0, count, 0};
  return launch_jobs(a, &spec, 1, dtype, op, variant, false, (hipStream_t)stream);
}

int mccl_reduce_scatter_n(const void* const* in, int n, void* const* out, size_t shard_count,
                          int shard_first, int shard_num, int dtype, int op, void* stream) {
  int rc = check_reduce_args(in, n, dtype, op);
  if (rc != MCCL_OK) return rc;
  if (shard_first < 0 || shard_num < 0) return fail(MCCL_ERR_INVALID_ARG, "negative shard range");
  if (shard_num == 0 || shard_count == 0) return MCCL_OK;
  if (!out) return fail(MCCL_ERR_INVALID_ARG, "output pointer table is null");
  const size_t es = dtype_size(dtype);
  ReduceArgs a;
  memset(&a, 0, sizeof(a));
  for (int k = 0; k < n; ++k) {
    if (!in[k]) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d is null", k);
    a.ptr[k] = (const char*)in[k];
  }
  a.n = n;
  for (int s0 = 0; s0 < shard_num; s0 += kMaxJobs) {
    const int m = (shard_num - s0 < kMaxJobs) ? shard_num - s0 : kMaxJobs;
    JobSpec specs[kMaxJobs];
    for (int j = 0; j < m; ++j) {
      if (!out[s0 + j]) return fail(MCCL_ERR_INVALID_ARG, "output pointer %d is null", s0 + j);
      specs[j] = JobSpec{(char*)out[s0 + j], (size_t)(shard_first + s0 + j) * shard_count * es, shard_count, 0};
    }
    rc = launch_jobs(a, specs, m, dtype, op, MCCL_VARIANT_AUTO, false, (hipStream_t)stream);
    if (rc != MCCL_OK) return rc;
  }
  return MCCL_OK;
}

int mccl_reduce_multi(const void* const* in, int n, void* const* out, const size_t* counts,
                      int nbuf, int dtype, int op, void* stream) {
  int rc = check_reduce_args(in, n, dtype, op);
  if (rc != MCCL_OK) return rc;
  if (nbuf < 0) return fail(MCCL_ERR_INVALID_ARG, "negative buffer count");
  if (nbuf == 0) return MCCL_OK;
  if (!out || !counts) return fail(MCCL_ERR_INVALID_ARG, "output or count table is null");
  int per_launch = MCCL_MAX_RANKS / n;
  if (per_launch > kMaxJobs) per_launch = kMaxJobs;
  for (int b0 = 0; b0 < nbuf; b0 += per_launch) {
    const int m = (nbuf - b0 < per_launch) ? nbuf - b0 : per_launch;
    ReduceArgs a;
    memset(&a, 0, sizeof(a));
    a.n = n;
    JobSpec specs[kMaxJobs];
    for (int j = 0; j < m; ++j) {
      for (int k = 0; k < n; ++k) {
        const void* p = in[(size_t)(b0 + j) * n + k];
        if (!p && counts[b0 + j]) return fail(MCCL_ERR_INVALID_ARG, "input pointer (%d,%d) is null", b0 + j, k);
        a.ptr[j * n + k] = (const char*)p;
      }
      if (!out[b0 + j] && counts[b0 + j]) return fail(MCCL_ERR_INVALID_ARG, "output pointer %d is null", b0 + j);
      specs[j] = JobSpec{(char*)out[b0 + j], 0, counts[b0 + j], j * n};
    }
    rc = launch_jobs(a, specs, m, dtype, op, MCCL_VARIANT_AUTO, true, (hipStream_t)stream);
    if (rc != MCCL_OK) return rc;
  }
  return MCCL_OK;
}

int mccl_rank_barrier(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us,
                      void* status, void* stream) {
  if (!flags) return fail(MCCL_ERR_INVALID_ARG, "flag pointer table is null");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  if (rank < 0 || rank >= n) return fail(MCCL_ERR_INVALID_ARG, "rank %d outside [0, %d)", rank, n);
  if ((uintptr_t)status % 4) return fail(MCCL_ERR_INVALID_ARG, "status word is not 4-byte aligned");
  for (int r = 0; r < n; ++r) {
    if (!flags[r]) return fail(MCCL_ERR_INVALID_ARG, "flag pointer %d is null", r);
    if ((uintptr_t)flags[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "flag pointer %d is not 8-byte aligned", r);
  }
  hipStream_t s = (hipStream_t)stream;
  if (n <= kLeanSyncRanks) {
    LeanBarrierArgs a;
    memset(&a, 0, sizeof(a));
    for (int r = 0; r < n; ++r) a.flag[r] = (uint64_t*)flags[r];
    a.epoch = epoch;
    a.limit_ticks = wait_limit_ticks(timeout_us);
    a.status = (uint32_t*)status;
    a.n = n;
    a.rank = rank;
    hipLaunchKernelGGL(rank_barrier_kernel<LeanBarrierArgs>, dim3(1), dim3(kWave), 0, s, a);
  } else {
    BarrierArgs a;
    memset(&a, 0, sizeof(a));
    for (int r = 0; r < n; ++r) a.flag[r] = (uint64_t*)flags[r];
    a.epoch = epoch;
    a.limit_ticks = wait_limit_ticks(timeout_us);
    a.status = (uint32_t*)status;
    a.n = n;
    a.rank = rank;
    hipLaunchKernelGGL(rank_barrier_kernel<BarrierArgs>, dim3(1), dim3(kWave), 0, s, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "barrier kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

int mccl_rank_barrier_offers(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us, void* status,
                             const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                             const mccl_import_table_t* imports, void* resolved, void* stream) {
  if (!flags || !offers) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer table is null");
  if (n < 1 || n > MCCL_OFFER_RANKS) return fail(MCCL_ERR_UNSUPPORTED, "a barrier with offers takes 1 to %d ranks, got %d", MCCL_OFFER_RANKS, n);
  if (rank < 0 || rank >= n) return fail(MCCL_ERR_INVALID_ARG, "rank %d outside [0, %d)", rank, n);
  if ((uintptr_t)status % 4) return fail(MCCL_ERR_INVALID_ARG, "status word is not 4-byte aligned");
  if (!mine || !imports || !resolved) return fail(MCCL_ERR_INVALID_ARG, "offer, import table or output table is null");
  if ((uintptr_t)imports % 8 || (uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "import table or output table is not 8-byte aligned");
  if (mine->entry != MCCL_OFFER_STAGED && mine->entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "offer names entry %u of %d", mine->entry, MCCL_OFFER_ENTRIES);
  OfferBarrierArgs a;
  memset(&a, 0, sizeof(a));
  for (int r = 0; r < n; ++r) {
    if (!flags[r] || !offers[r]) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer %d is null", r);
    if ((uintptr_t)flags[r] % 8 || (uintptr_t)offers[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer %d is not 8-byte aligned", r);
    a.flag[r] = (uint64_t*)flags[r];
    a.offer[r] = (uint64_t*)offers[r];
  }
  a.epoch = epoch;
  a.limit_ticks = wait_limit_ticks(timeout_us);
  a.status = (uint32_t*)status;
  a.mine[0] = (uint64_t)mine->entry | ((uint64_t)mine->slot << 32);
  a.mine[1] = mine->generation;
  a.mine[2] = mine->offset;
  a.mine[3] = mine->bytes;
  a.my_buffer = (uint64_t)(uintptr_t)my_buffer;
  a.imports = imports;
  a.resolved = (uint64_t*)resolved;
  a.n = n;
  a.rank = rank;
  hipLaunchKernelGGL(rank_barrier_offers_kernel, dim3(1), dim3(kWave), 0, (hipStream_t)stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "barrier kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

int mccl_rank_barrier_offers_each(void* const* flags, int n, int rank, uint64_t epoch, uint64_t timeout_us, void* status,
                                  const mccl_offer_t* mine, const uint64_t* expect_bytes, const void* my_source,
                                  void* const* offers, const mccl_import_table_t* imports, void* resolved, void* stream) {
  if (!flags || !offers) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer table is null");
  if (n < 1 || n > MCCL_OFFER_RANKS) return fail(MCCL_ERR_UNSUPPORTED, "a barrier with offers takes 1 to %d ranks, got %d", MCCL_OFFER_RANKS, n);
  if (rank < 0 || rank >= n) return fail(MCCL_ERR_INVALID_ARG, "rank %d outside [0, %d)", rank, n);
  if ((uintptr_t)status % 4) return fail(MCCL_ERR_INVALID_ARG, "status word is not 4-byte aligned");
  if (!mine || !expect_bytes || !imports || !resolved) return fail(MCCL_ERR_INVALID_ARG, "offers, expected lengths, import table or output table is null");
  if ((uintptr_t)imports % 8 || (uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "import table or output table is not 8-byte aligned");
  OfferEachArgs a;
  memset(&a, 0, sizeof(a));
  for (int r = 0; r < n; ++r) {
    if (!flags[r] || !offers[r]) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer %d is null", r);
    if ((uintptr_t)flags[r] % 8 || (uintptr_t)offers[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "flag or offer pointer %d is not 8-byte aligned", r);
    const mccl_offer_t& o = mine[r];
    if (o.entry != MCCL_OFFER_STAGED && o.entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "offer %d names entry %u of %d", r, o.entry, MCCL_OFFER_ENTRIES);
    if (o.entry == MCCL_OFFER_STAGED && o.slot >= MCCL_OFFER_SLOTS) return fail(MCCL_ERR_INVALID_ARG, "offer %d names staging buffer %u of %d", r, o.slot, MCCL_OFFER_SLOTS);
    a.flag[r] = (uint64_t*)flags[r];
    a.row[r] = (uint64_t*)offers[r];
    a.mine[r][0] = (uint64_t)o.entry | ((uint64_t)o.slot << 32);
    a.mine[r][1] = o.generation;
    a.mine[r][2] = o.offset;
    a.mine[r][3] = o.bytes;
    a.expect[r] = expect_bytes[r];
  }
  a.epoch = epoch;
  a.limit_ticks = wait_limit_ticks(timeout_us);
  a.status = (uint32_t*)status;
  a.my_source = (uint64_t)(uintptr_t)my_source;
  a.imports = imports;
  a.resolved = (uint64_t*)resolved;
  a.n = n;
  a.rank = rank;
  hipLaunchKernelGGL(rank_barrier_offers_each_kernel, dim3(1), dim3(kWave), 0, (hipStream_t)stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "barrier kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

int mccl_import_table_update(mccl_import_table_t* table, const mccl_import_update_t* updates, int n, void* stream) {
  if (n == 0) return MCCL_OK;
  if (!table || !updates) return fail(MCCL_ERR_INVALID_ARG, "table or update list is null");
  if ((uintptr_t)table % 8) return fail(MCCL_ERR_INVALID_ARG, "import table is not 8-byte aligned");
  if (n < 0 || n > MCCL_IMPORT_UPDATES) return fail(MCCL_ERR_INVALID_ARG, "%d updates in one call, at most %d", n, MCCL_IMPORT_UPDATES);
  ImportUpdateArgs a;
  memset(&a, 0, sizeof(a));
  a.table = table;
  a.n = n;
  for (int i = 0; i < n; ++i) {
    const mccl_import_update_t& u = updates[i];
    if (u.rank >= MCCL_OFFER_RANKS) return fail(MCCL_ERR_INVALID_ARG, "update %d names rank %u of %d", i, u.rank, MCCL_OFFER_RANKS);
    if (u.entry != MCCL_OFFER_STAGED && u.entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "update %d names entry %u of %d", i, u.entry, MCCL_OFFER_ENTRIES);
    if (u.entry == MCCL_OFFER_STAGED && u.slot >= MCCL_OFFER_SLOTS) return fail(MCCL_ERR_INVALID_ARG, "update %d names staging buffer %u of %d", i, u.slot, MCCL_OFFER_SLOTS);
    for (int j = 0; j < i; ++j)
      if (updates[j].rank == u.rank && updates[j].entry == u.entry && (u.entry != MCCL_OFFER_STAGED || updates[j].slot == u.slot))
        return fail(MCCL_ERR_INVALID_ARG, "updates %d and %d name the same entry", j, i);
    a.update[i] = u;
  }
  hipLaunchKernelGGL(import_table_update_kernel, dim3(1), dim3(kWave), 0, (hipStream_t)stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "table update launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // extern "C"

namespace {

// Both forms of the one-launch small allreduce: the epoch from the host (state == null), or kept in
// `state` on the device and advanced by the launch itself.
int allreduce_fused_impl(const void* in, void* out, size_t count, int dtype, int op, void* const* stage,
                         void* const* tile_flags, int n, int rank, uint32_t epoch, void* state, size_t stage_stride,
                         size_t flags_stride, uint64_t timeout_us, void* status, unsigned max_compute_units, unsigned mode,
                         void* stream) {
  int rc = check_reduce_args_no_ptr(n, dtype, op);
  if (mode & ~(MCCL_FUSED_WORK_ONLY | MCCL_FUSED_SYNC_ONLY)) return fail(MCCL_ERR_INVALID_ARG, "unknown flags 0x%x", mode);
  if (mode == (MCCL_FUSED_WORK_ONLY | MCCL_FUSED_SYNC_ONLY)) return fail(MCCL_ERR_INVALID_ARG, "work-only and sync-only exclude each other");
  if (rc != MCCL_OK) return rc;
  if (n > MCCL_FUSED_MAX_RANKS) return fail(MCCL_ERR_UNSUPPORTED, "the one-launch allreduce takes at most %d ranks, got %d", MCCL_FUSED_MAX_RANKS, n);
  if (rank < 0 || rank >= n) return fail(MCCL_ERR_INVALID_ARG, "rank %d outside [0, %d)", rank, n);
  if (!stage || !tile_flags) return fail(MCCL_ERR_INVALID_ARG, "staging or flag pointer table is null");
  if ((uintptr_t)status % 4) return fail(MCCL_ERR_INVALID_ARG, "status word is not 4-byte aligned");
  const size_t es = dtype_size(dtype);
  for (int r = 0; r < n; ++r) {
    if (!stage[r] || !tile_flags[r]) return fail(MCCL_ERR_INVALID_ARG, "staging or flag pointer %d is null", r);
    if ((uintptr_t)stage[r] % 16) return fail(MCCL_ERR_INVALID_ARG, "staging buffer %d is not 16-byte aligned", r);
    if ((uintptr_t)tile_flags[r] % 4) return fail(MCCL_ERR_INVALID_ARG, "flag array %d is not 4-byte aligned", r);
  }
  const size_t ve = 16 / es;
  const size_t nvec = count / ve;
  const size_t tiles = (nvec + (count % ve ? 1 : 0) + kWave - 1) / kWave;
  if (state) {
    if ((uintptr_t)state % 64) return fail(MCCL_ERR_INVALID_ARG, "the epoch state is not 64-byte aligned");
    if (stage_stride % 16 || stage_stride > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "the staging sets must lie a multiple of 16 bytes (below 4 GiB) apart");
    if (flags_stride % 4 || flags_stride > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "the flag sets must lie a multiple of 4 bytes (below 4 GiB) apart");
    if (count * es > stage_stride || tiles * 4 > flags_stride) return fail(MCCL_ERR_INVALID_ARG, "the message does not fit between the two buffer sets");
  }
  if (count == 0) return MCCL_OK;  // on every rank alike: no launch, the epoch stays
  if (!in || !out) return fail(MCCL_ERR_INVALID_ARG, "input or output pointer is null");
  if ((uintptr_t)in % es || (uintptr_t)out % es) return fail(MCCL_ERR_INVALID_ARG, "input or output pointer not aligned to the element size");
  if (in != out) {
    const uintptr_t i0 = (uintptr_t)in, o0 = (uintptr_t)out;
    if (i0 < o0 + count * es && o0 < i0 + count * es) return fail(MCCL_ERR_INVALID_ARG, "output partially overlaps the input");
  }
  if (tiles > kMaxGridX) return fail(MCCL_ERR_INVALID_ARG, "message too large for the one-launch allreduce");
  // one wavefront per tile, sixteen to a workgroup; with a limit on the workgroups a wavefront
  // takes up to kFusedMaxTilesPerWave tiles
  size_t groups = (tiles + kFusedWavesPerGroup - 1) / kFusedWavesPerGroup;
  if (max_compute_units && groups > max_compute_units) {
    groups = max_compute_units;
    if (tiles > groups * kFusedWavesPerGroup * kFusedMaxTilesPerWave)
      return fail(MCCL_ERR_INVALID_ARG, "a one-launch allreduce on %u compute units takes at most %zu bytes, got %zu", max_compute_units,
                  groups * kFusedWavesPerGroup * kFusedMaxTilesPerWave * (size_t)MCCL_FUSED_TILE_BYTES, count * es);
  }
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  a.in = (const char*)in;
  a.out = (char*)out;
  for (int r = 0; r < n; ++r) {
    a.stage[r] = (char*)stage[r];
    a.flag[r] = (uint32_t*)tile_flags[r];
  }
  a.nvec = nvec;
  a.limit_ticks = wait_limit_ticks(timeout_us);
  a.status = (uint32_t*)status;
  a.tail = (uint32_t)(count % ve);
  a.epoch = epoch;
  a.tiles = (uint32_t)tiles;
  a.n = n;
  a.rank = rank;
  a.state = (uint32_t*)state;
  a.stage_stride = (uint32_t)stage_stride;
  a.flag_stride = (uint32_t)(flags_stride / 4);
  a.mode = mode;
  hipError_t e = launch_fused_any(a, dtype, op, (unsigned)groups, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "fused allreduce launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_allreduce_fused(const void* in, void* out, size_t count, int dtype, int op,
                         void* const* stage, void* const* tile_flags, int n, int rank, uint32_t epoch,
                         uint64_t timeout_us, void* status, unsigned max_compute_units, void* stream) {
  return allreduce_fused_impl(in, out, count, dtype, op, stage, tile_flags, n, rank, epoch, nullptr, 0, 0, timeout_us, status,
                              max_compute_units, 0u, stream);
}

int mccl_allreduce_fused_replayable(const void* in, void* out, size_t count, int dtype, int op,
                                    void* const* stage, void* const* tile_flags, size_t stage_stride, size_t flags_stride,
                                    void* state, int n, int rank, uint64_t timeout_us, void* status,
                                    unsigned max_compute_units, unsigned flags, void* stream) {
  if (!state) return fail(MCCL_ERR_INVALID_ARG, "the epoch state is null");
  return allreduce_fused_impl(in, out, count, dtype, op, stage, tile_flags, n, rank, 0, state, stage_stride, flags_stride,
                              timeout_us, status, max_compute_units, flags, stream);
}

}  // extern "C"

namespace {

// Workgroups (single wavefronts) of a launch that waits for its peers inside the kernel: all
// ranks' launches must be resident at once, so each gets its share of a fixed budget.
// A launch that waits for its peers gets its share of the wavefronts all ranks may hold together;
// one that does not wait (the caller has ordered the ranks) can never keep a peer's launch out and
// takes the whole budget.
unsigned xrank_grid(uint64_t tiles, int n, bool waits = true) {
  uint64_t cap = (uint64_t)g_tune[MCCL_TUNE_XRANK_WAVES_ALL_RANKS] / (uint64_t)(waits ? n : 1);
  if (cap < 1) cap = 1;
  if (tiles < 1) tiles = 1;
  return (unsigned)(tiles < cap ? tiles : cap);
}

// The shape of a cross-rank launch: single wavefronts spread over the GPU, or -- when the caller
// limits the compute units the launch may hold while it waits -- that many workgroups of
// kPackedWaves wavefronts at most (and never more wavefronts than the budget above allows).
// `lds`: dynamic LDS reserved per workgroup, which caps how many are resident on a compute unit.
struct XShape {
  unsigned groups;
  int packed;
  unsigned lds;
};
// fresh_tiles: a launch that does not wait at its start may be given one workgroup per so many tiles
// instead of a persistent grid (fresh workgroups move more bytes per second than a grid's walk, and
// nothing has to be resident together with anything); 0 for kernels that gain nothing from it.
// Measured behind the closing count, 8 x 64 MiB, one process: the shard reduction 94.5 us with one
// tile per workgroup against 106 us as a grid of 4096 wavefronts, the push 97.5 us with two tiles
// per workgroup (both loads in flight before the sixteen stores) against 104 us; the in-place
// allreduce is level (74 against 73-75 % of the HBM peak) and keeps the grid.
XShape xrank_shape(uint64_t tiles, const mccl_xsync_t* sy, bool waits = true, unsigned fresh_tiles = 0) {
  if (sy->max_compute_units == 0) {
    if (!waits && fresh_tiles) {
      uint64_t cap = (uint64_t)g_tune[MCCL_TUNE_XRANK_FRESH_MAX_WAVES];
      if (cap < 1 || cap > kMaxGridX) cap = kMaxGridX;
      uint64_t want = (tiles + fresh_tiles - 1) / fresh_tiles;
      if (want < 1) want = 1;
      int cus = 0;
      const bool large = device_cus(&cus) == MCCL_OK && want > (uint64_t)cus * 4;  // small launches are latency bound: no cap
      return XShape{(unsigned)(want < cap ? want : cap), 0, large ? lds_for_waves(g_tune[MCCL_TUNE_XRANK_FRESH_WAVES_PER_CU]) : 0u};
    }
    return XShape{xrank_grid(tiles, sy->n, waits), 0, 0u};
  }
  const uint64_t waves = xrank_grid(tiles, sy->n, waits);
  uint64_t groups = (waves + kPackedWaves - 1) / kPackedWaves;
  if (groups > sy->max_compute_units) groups = sy->max_compute_units;
  return XShape{(unsigned)groups, 1, 0u};
}

int fill_xsync(const mccl_xsync_t* sy, XSync* x) {
  if (!sy) return fail(MCCL_ERR_INVALID_ARG, "sync descriptor is null");
  if (sy->n < 1 || sy->n > kXRanks) return fail(MCCL_ERR_UNSUPPORTED, "one-launch collectives take 1 to %d ranks, got %d", kXRanks, sy->n);
  if (sy->rank < 0 || sy->rank >= sy->n) return fail(MCCL_ERR_INVALID_ARG, "rank %d outside [0, %d)", sy->rank, sy->n);
  memset(x, 0, sizeof(*x));
  x->n = sy->n;
  x->rank = sy->rank;
  // ready_epoch 0: the caller has ordered the start of the ranks itself (a barrier kernel in front,
  // host barriers): no opening wait; done_epoch 0: no closing wait
  if (sy->ready_epoch == 0 && sy->done_epoch == 0) return MCCL_OK;
  if (!sy->words) return fail(MCCL_ERR_INVALID_ARG, "sync word table is null");
  if (sy->done_epoch != 0 && sy->done_epoch <= sy->ready_epoch) return fail(MCCL_ERR_INVALID_ARG, "done_epoch must be 0 or above ready_epoch");
  if (sy->done_epoch != 0 && !sy->done_counter) return fail(MCCL_ERR_INVALID_ARG, "a closing wait needs a done counter");
  if ((uintptr_t)sy->done_counter % 64) return fail(MCCL_ERR_INVALID_ARG, "the done counters are not 64-byte aligned");
  if ((uintptr_t)sy->status % 4) return fail(MCCL_ERR_INVALID_ARG, "status word is not 4-byte aligned");
  for (int r = 0; r < sy->n; ++r) {
    if (!sy->words[r]) return fail(MCCL_ERR_INVALID_ARG, "sync word %d is null", r);
    if ((uintptr_t)sy->words[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "sync word %d is not 8-byte aligned", r);
    x->word[r] = (uint64_t*)sy->words[r];
  }
  x->ready_epoch = sy->ready_epoch;
  x->done_epoch = sy->done_epoch;
  x->done_count = (uint32_t*)sy->done_counter;
  x->limit_ticks = wait_limit_ticks(sy->timeout_us);
  x->status = (uint32_t*)sy->status;
  return MCCL_OK;
}

// How the peers' tensors are read (MCCL_TUNE_XRANK_CACHED_LOADS).
void apply_cached_loads(XRankArgs* a) {
  const long long mode = g_tune[MCCL_TUNE_XRANK_CACHED_LOADS];
  if (mode == 1) {
    a->aligned_in = 0;
  } else if (mode == 2 && a->sync.ready_epoch == 0) {
    a->aligned_in = 0;
    a->no_invalidate = 1;
  }
}

// The in-place allreduce with its tensors' addresses from the host (tensors) or from device memory
// (resolved: read by the kernel when it starts).
struct OfferExchange {  // the launch exchanges the ranks' offers itself
  const mccl_offer_t* mine;
  const void* my_buffer;
  void* const* offers;
  const mccl_import_table_t* imports;
};

int allreduce_sync_impl(void* const* tensors, const void* resolved, const OfferExchange* ox, size_t count, int dtype, int op,
                        const mccl_xsync_t* sync, void* stream) {
  XRankArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  rc = check_reduce_args_no_ptr(a.sync.n, dtype, op);
  if (rc != MCCL_OK) return rc;
  if (a.sync.ready_epoch != 0 && a.sync.done_epoch == 0)
    return fail(MCCL_ERR_INVALID_ARG, "the in-place allreduce needs a closing wait (done_epoch) when it has an opening one");
  const int n = a.sync.n, me = a.sync.rank;
  const size_t es = dtype_size(dtype);
  if (tensors) {
    for (int r = 0; r < n; ++r) {
      if (count && !tensors[r]) return fail(MCCL_ERR_INVALID_ARG, "tensor pointer %d is null", r);
      if ((uintptr_t)tensors[r] % es) return fail(MCCL_ERR_INVALID_ARG, "tensor %d not aligned to the element size", r);
    }
    // two ranks' tensors may be the same memory (one process playing several ranks), never partly so
    for (int r = 0; r < n && count; ++r)
      for (int q = r + 1; q < n; ++q) {
        const uintptr_t a0 = (uintptr_t)tensors[r], b0 = (uintptr_t)tensors[q];
        if (a0 != b0 && a0 < b0 + count * es && b0 < a0 + count * es)
          return fail(MCCL_ERR_INVALID_ARG, "tensors %d and %d partially overlap", r, q);
      }
  }
  const size_t shard = mccl_allreduce_sync_shard(count, n);
  const size_t lo = (size_t)me * shard < count ? (size_t)me * shard : count;
  const size_t n_me = lo + shard < count ? shard : count - lo;
  const size_t ve = 16 / es;
  if ((uint64_t)shard * es / 16 + kWave > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "message too large");
  a.aligned_in = 1;
  if (tensors) {
    for (int k = 0; k < n; ++k) {
      a.in[k] = (const char*)tensors[k] + lo * es;
      if (n_me && ((uintptr_t)a.in[k] & 7u)) a.aligned_in = 0;
    }
  } else if (resolved) {
    // where the tensors lie is not known here: any alignment, read through the caches (the barrier
    // in front has ordered the ranks, so the caches start clean)
    a.in_table = (const uint64_t*)resolved;
    a.in_off = lo * es;
    a.aligned_in = 0;
    a.no_invalidate = 1;
  } else {
    // the same, the offers exchanged by this launch: the peers' data was complete before their
    // launches began, but lines of it may sit in this launch's caches from before: one invalidate
    // per workgroup after the opening wait (aligned_in 0 without no_invalidate)
    for (int r = 0; r < n; ++r) {
      if (!ox->offers[r]) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is null", r);
      if ((uintptr_t)ox->offers[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is not 8-byte aligned", r);
      a.offer[r] = (uint64_t*)ox->offers[r];
    }
    a.mine[0] = (uint64_t)ox->mine->entry | ((uint64_t)ox->mine->slot << 32);
    a.mine[1] = ox->mine->generation;
    a.mine[2] = ox->mine->offset;
    a.mine[3] = ox->mine->bytes;
    a.imports = ox->imports;
    a.my_buffer = (uint64_t)(uintptr_t)ox->my_buffer;
    a.in_off = lo * es;
    a.aligned_in = 0;
  }
  a.push = 1;
  a.nvec1 = (uint32_t)(n_me / ve);
  a.tail1 = (uint32_t)(n_me % ve);
  a.tiles1 = (uint32_t)((n_me / ve + (n_me % ve ? 1 : 0) + kWave - 1) / kWave);
  apply_cached_loads(&a);
  const XShape shape = xrank_shape(a.tiles1, sync, a.sync.ready_epoch != 0);
  hipError_t e = launch_xrank_any(a, dtype, op, shape.groups, shape.packed, shape.lds, a.sync.ready_epoch != 0 ? (unsigned)a.sync.n : 0u, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "allreduce kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

// src_rank / resolved: the sources come from a table in device memory (mccl_copy_segments_sync_resolved).
int copy_segments_sync_impl(const mccl_segment_t* segs, const int* src_rank, const void* resolved, int nseg, unsigned flags,
                            const mccl_xsync_t* sync, void* stream) {
  SyncCopyArgs a;
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  a.src_table = (const uint64_t*)resolved;
  memset(a.src_rank, 0xff, sizeof(a.src_rank));
  if (nseg < 0 || nseg > kMaxSegs) return fail(MCCL_ERR_INVALID_ARG, "a one-launch copy takes 0 to %d segments, got %d", kMaxSegs, nseg);
  if (nseg && !segs) return fail(MCCL_ERR_INVALID_ARG, "segment table is null");
  int m = 0;
  uint64_t chunks = 0;
  a.copy.chunk_prefix[0] = 0;
  for (int i = 0; i < nseg; ++i) {
    const mccl_segment_t& sg = segs[i];
    if (sg.bytes == 0) continue;
    const int from = src_rank ? src_rank[i] : -1;
    if (from >= a.sync.n) return fail(MCCL_ERR_INVALID_ARG, "segment %d reads from rank %d of %d", i, from, a.sync.n);
    if ((from < 0 && !sg.src) || !sg.dst) return fail(MCCL_ERR_INVALID_ARG, "segment %d has a null pointer", i);
    a.src_rank[m] = (int8_t)(from < 0 ? -1 : from);
    const uintptr_t dp = (uintptr_t)sg.dst;
    CopySeg cs;
    cs.src = (const char*)sg.src;
    cs.dst = (char*)sg.dst;
    cs.pad_ = 0;
    size_t head = (128u - (unsigned)(dp & 127u)) & 127u;
    if (head > sg.bytes) head = sg.bytes;
    const size_t body = sg.bytes - head;
    const uint64_t nfull = body / kCopyChunk;
    cs.head = (uint32_t)head;
    cs.last = (uint32_t)(body % kCopyChunk);
    uint64_t c = nfull + (cs.last ? 1 : 0);
    if (c == 0) c = 1;
    if (nfull > 0xf0000000ull || chunks + c > kMaxChunks) return fail(MCCL_ERR_INVALID_ARG, "segment %d too large for a one-launch copy", i);
    cs.nfull = (uint32_t)nfull;
    a.copy.seg[m] = cs;
    chunks += c;
    a.copy.chunk_prefix[++m] = (uint32_t)chunks;
  }
  a.copy.nseg = m;  // may be 0: the launch still takes part in the waits
  // Full chunks of 8-byte aligned sources are read past the caches; whatever else there is (heads,
  // partial chunks, misaligned sources) is read through them, after an invalidate per workgroup.
  a.invalidate = 0;
  a.shared = (flags & MCCL_COPY_SHARED_SOURCES) ? 1u : 0u;
  for (int k = 0; k < m; ++k) {
    const CopySeg& cs = a.copy.seg[k];
    if (cs.head || cs.last || (((uintptr_t)cs.src + cs.head) & 7u)) a.invalidate = 1;
  }
  const XShape shape = xrank_shape(chunks, sync);  // (a copy gains nothing from more wavefronts than its share, waits or not)
  unsigned grid = shape.groups;
  if (flags & ~MCCL_COPY_SHARED_SOURCES) return fail(MCCL_ERR_INVALID_ARG, "unknown copy flags 0x%x", flags);
  int cus = 0;
  rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  if (resolved) {
    if (shape.packed) return fail(MCCL_ERR_INVALID_ARG, "a copy over resolved addresses runs as single wavefronts (max_compute_units 0)");
    // the plain copy's launch (launch_copy): a workgroup per chunk, its residency cap, its choice of stores
    // (two chunks per workgroup from 128 MiB on: every workgroup counts itself out with an atomic, sixteen
    // counters take about 7 ns per atomic each, and at one 2 KiB chunk per workgroup that count, not the
    // copy, set the pace -- 188 us against 146 us for eight pieces of 56 MiB, the plain copy 142 us)
    const uint64_t per_group = chunks >= (1u << 16) ? 2 : 1;
    grid = (unsigned)std::min<uint64_t>(std::max<uint64_t>((chunks + per_group - 1) / per_group, 1), kMaxGridX);
    const unsigned lds = (chunks > (uint64_t)cus * 4) ? lds_for_waves(g_tune[MCCL_TUNE_COPY_WAVES_PER_CU]) : 0;
    long long stream_store = g_tune[MCCL_TUNE_COPY_STREAM_STORES];
    if (stream_store != 1 && stream_store != 2) stream_store = chunks * kCopyChunk >= (uint64_t)g_tune[MCCL_TUNE_COPY_LARGE_MIN_BYTES] ? kCopyStreamLarge : 2;
    if (stream_store == 1) hipLaunchKernelGGL(copy_segments_resolved_kernel<true>, dim3(grid), dim3(kWave), lds, (hipStream_t)stream, a);
    else hipLaunchKernelGGL(copy_segments_resolved_kernel<false>, dim3(grid), dim3(kWave), lds, (hipStream_t)stream, a);
  } else if (shape.packed) {
    static const unsigned per_cu = blocks_per_cu(copy_segments_sync_kernel<kPackedWaves>, kWave * kPackedWaves);
    if (a.sync.ready_epoch != 0) grid = std::min(grid, waiting_share(per_cu, (unsigned)cus, (unsigned)a.sync.n));
    hipLaunchKernelGGL(copy_segments_sync_kernel<kPackedWaves>, dim3(grid), dim3(kWave * kPackedWaves), 0, (hipStream_t)stream, a);
  } else {
    static const unsigned per_cu = blocks_per_cu(copy_segments_sync_kernel<1>, kWave);
    if (a.sync.ready_epoch != 0) grid = std::min(grid, waiting_share(per_cu, (unsigned)cus, (unsigned)a.sync.n));
    hipLaunchKernelGGL(copy_segments_sync_kernel<1>, dim3(grid), dim3(kWave), 0, (hipStream_t)stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "copy kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_copy_segments_sync(const mccl_segment_t* segs, int nseg, unsigned flags, const mccl_xsync_t* sync, void* stream) {
  return copy_segments_sync_impl(segs, nullptr, nullptr, nseg, flags, sync, stream);
}


int mccl_copy_segments_sync_resolved(const mccl_segment_t* segs, const int* src_rank, int nseg, const void* resolved,
                                     unsigned flags, const mccl_xsync_t* sync, void* stream) {
  if (!resolved) return fail(MCCL_ERR_INVALID_ARG, "address table is null");
  if ((uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "address table is not 8-byte aligned");
  if (nseg > 0 && !src_rank) return fail(MCCL_ERR_INVALID_ARG, "source rank table is null");
  if (sync && (sync->ready_epoch != 0 || sync->done_epoch == 0))
    return fail(MCCL_ERR_INVALID_ARG, "a launch over resolved addresses runs behind a barrier: ready_epoch 0, done_epoch set");
  return copy_segments_sync_impl(segs, src_rank, resolved, nseg, flags, sync, stream);
}

int mccl_fanout_sync(const void* src, void* const* dst, int ndst, size_t bytes, const mccl_xsync_t* sync, void* stream) {
  FanoutArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  if (ndst < 1 || ndst > kLeanSyncRanks) return fail(MCCL_ERR_UNSUPPORTED, "a push takes 1 to %d destinations, got %d", kLeanSyncRanks, ndst);
  if (!dst) return fail(MCCL_ERR_INVALID_ARG, "destination table is null");
  if (bytes / 16 > 0xf0000000ull) return fail(MCCL_ERR_INVALID_ARG, "message too large for one push");
  a.ndst = ndst;
  a.aligned = 1;
  if (bytes) {
    if (!src) return fail(MCCL_ERR_INVALID_ARG, "source pointer is null");
    int m = 0;
    for (int k = 0; k < ndst; ++k) {
      if (!dst[k]) return fail(MCCL_ERR_INVALID_ARG, "destination pointer %d is null", k);
      const uintptr_t s0 = (uintptr_t)src, d0 = (uintptr_t)dst[k];
      if (s0 == d0) continue;  // in place: this rank's contribution already sits in its own output
      if (s0 < d0 + bytes && d0 < s0 + bytes) return fail(MCCL_ERR_INVALID_ARG, "destination %d partially overlaps the source", k);
      if (d0 & 15u) a.aligned = 0;
      a.dst[m++] = (char*)dst[k];
    }
    a.ndst = m;
    a.src = (const char*)src;
    a.nvec = (uint32_t)(bytes / 16);
    a.tail = (uint32_t)(bytes % 16);
    a.tiles = (uint32_t)((bytes / 16 + kWave - 1) / kWave);
  }
  // (the last wavefront takes the tail: a launch of at least one)
  const XShape shape = xrank_shape(a.tiles, sync, a.sync.ready_epoch != 0, /*fresh_tiles=*/2);
  unsigned grid = shape.groups;
  int cus = 0;
  rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  if (shape.packed) {
    static const unsigned per_cu = blocks_per_cu(fanout_sync_kernel<kPackedWaves>, kWave * kPackedWaves);
    if (a.sync.ready_epoch != 0) grid = std::min(grid, waiting_share(per_cu, (unsigned)cus, (unsigned)a.sync.n));
    hipLaunchKernelGGL(fanout_sync_kernel<kPackedWaves>, dim3(grid), dim3(kWave * kPackedWaves), 0, (hipStream_t)stream, a);
  } else {
    static const unsigned per_cu = blocks_per_cu(fanout_sync_kernel<1>, kWave);
    if (a.sync.ready_epoch != 0) grid = std::min(grid, waiting_share(per_cu, (unsigned)cus, (unsigned)a.sync.n));
    hipLaunchKernelGGL(fanout_sync_kernel<1>, dim3(grid), dim3(kWave), shape.lds, (hipStream_t)stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "push kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

int mccl_reduce_sync(const void* const* in, void* out, size_t count, int dtype, int op,
                     const mccl_xsync_t* sync, void* stream) {
  XRankArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  rc = check_reduce_args(in, a.sync.n, dtype, op);
  if (rc != MCCL_OK) return rc;
  const size_t es = dtype_size(dtype);
  if (count) {
    if (!out) return fail(MCCL_ERR_INVALID_ARG, "output pointer is null");
    if ((uintptr_t)out % es) return fail(MCCL_ERR_INVALID_ARG, "output pointer not aligned to the element size");
    for (int k = 0; k < a.sync.n; ++k) {
      if (!in[k]) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d is null", k);
      if ((uintptr_t)in[k] % es) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d not aligned to the element size", k);
      a.in[k] = (const char*)in[k];
    }
  }
  // the output may be exactly one of the inputs (a lane reads element i of every input before it
  // writes element i); any other overlap would have one workgroup write what another still reads
  for (int k = 0; k < a.sync.n && count; ++k) {
    const uintptr_t i0 = (uintptr_t)in[k], o0 = (uintptr_t)out;
    if (i0 != o0 && i0 < o0 + count * es && o0 < i0 + count * es)
      return fail(MCCL_ERR_INVALID_ARG, "output partially overlaps input %d", k);
  }
  const size_t ve = 16 / es;
  const uint64_t vecs = count / ve + (count % ve ? 1 : 0);
  if (vecs + kWave > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "message too large");
  a.out1 = (char*)out;
  a.nvec1 = (uint32_t)(count / ve);
  a.tail1 = (uint32_t)(count % ve);
  a.tiles1 = (uint32_t)((vecs + kWave - 1) / kWave);
  a.stream_out = count * es >= (32u << 20) ? 1u : 0u;
  a.aligned_in = 1;
  for (int k = 0; k < a.sync.n; ++k)
    if (count && ((uintptr_t)in[k] & 7u)) a.aligned_in = 0;
  apply_cached_loads(&a);
  const XShape shape = xrank_shape(a.tiles1, sync, a.sync.ready_epoch != 0, /*fresh_tiles=*/1);
  hipError_t e = launch_xrank_any(a, dtype, op, shape.groups, shape.packed, shape.lds, a.sync.ready_epoch != 0 ? (unsigned)a.sync.n : 0u, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "reduce kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // extern "C"

namespace {

int check_offer_exchange(const OfferExchange& ox, int n) {
  if (!ox.mine || !ox.offers || !ox.imports) return fail(MCCL_ERR_INVALID_ARG, "offer, offer table or import table is null");
  if ((uintptr_t)ox.imports % 8) return fail(MCCL_ERR_INVALID_ARG, "import table is not 8-byte aligned");
  if (ox.mine->entry != MCCL_OFFER_STAGED && ox.mine->entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "offer names entry %u of %d", ox.mine->entry, MCCL_OFFER_ENTRIES);
  for (int r = 0; r < n; ++r) {
    if (!ox.offers[r]) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is null", r);
    if ((uintptr_t)ox.offers[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is not 8-byte aligned", r);
  }
  return MCCL_OK;
}

void offer_words(const mccl_offer_t& mine, uint64_t (&w)[4]) {
  w[0] = (uint64_t)mine.entry | ((uint64_t)mine.slot << 32);
  w[1] = mine.generation;
  w[2] = mine.offset;
  w[3] = mine.bytes;
}

int check_indirect_sync(const mccl_xsync_t* sync, bool one_launch) {
  if (!sync) return MCCL_OK;  // fill_xsync reports it
  if (one_launch) {
    if (sync->ready_epoch == 0 || sync->done_epoch == 0 || sync->max_compute_units == 0)
      return fail(MCCL_ERR_INVALID_ARG, "the one-launch form with offers needs ready_epoch, done_epoch and max_compute_units");
  } else if (sync->ready_epoch != 0 || sync->done_epoch == 0) {
    return fail(MCCL_ERR_INVALID_ARG, "a launch over resolved addresses runs behind a barrier: ready_epoch 0, done_epoch set");
  }
  return MCCL_OK;
}

// The shard reduction over addresses from the ranks' offers: `resolved` (behind the barrier that
// resolved them) or `ox` (the launch exchanges them itself).
int reduce_sync_indirect(const void* resolved, const OfferExchange* ox, size_t in_offset, void* out, size_t count, int dtype,
                         int op, const mccl_xsync_t* sync, void* stream) {
  XRankArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  rc = check_reduce_args_no_ptr(a.sync.n, dtype, op);
  if (rc != MCCL_OK) return rc;
  rc = check_indirect_sync(sync, ox != nullptr);
  if (rc != MCCL_OK) return rc;
  const size_t es = dtype_size(dtype);
  if (in_offset % es) return fail(MCCL_ERR_INVALID_ARG, "input offset not aligned to the element size");
  if (count) {
    if (!out) return fail(MCCL_ERR_INVALID_ARG, "output pointer is null");
    if ((uintptr_t)out % es) return fail(MCCL_ERR_INVALID_ARG, "output pointer not aligned to the element size");
  }
  const size_t ve = 16 / es;
  const uint64_t vecs = count / ve + (count % ve ? 1 : 0);
  if (vecs + kWave > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "message too large");
  a.out1 = (char*)out;
  a.nvec1 = (uint32_t)(count / ve);
  a.tail1 = (uint32_t)(count % ve);
  a.tiles1 = (uint32_t)((vecs + kWave - 1) / kWave);
  a.stream_out = count * es >= (32u << 20) ? 1u : 0u;
  a.in_off = in_offset;
  a.aligned_in = 0;  // where the inputs lie is not known here: any alignment, through the caches
  if (resolved) {
    a.in_table = (const uint64_t*)resolved;
    a.no_invalidate = 1;  // behind a kernel boundary: the caches start clean
  } else {
    rc = check_offer_exchange(*ox, a.sync.n);
    if (rc != MCCL_OK) return rc;
    for (int r = 0; r < a.sync.n; ++r) a.offer[r] = (uint64_t*)ox->offers[r];
    offer_words(*ox->mine, a.mine);
    a.imports = ox->imports;
    a.my_buffer = (uint64_t)(uintptr_t)ox->my_buffer;
  }
  const XShape shape = xrank_shape(a.tiles1, sync, a.sync.ready_epoch != 0, /*fresh_tiles=*/1);
  hipError_t e = launch_xrank_any(a, dtype, op, shape.groups, shape.packed, shape.lds, a.sync.ready_epoch != 0 ? (unsigned)a.sync.n : 0u, (hipStream_t)stream);
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "reduce kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

int fanout_sync_indirect(const void* src, const void* resolved, const OfferExchange* ox, size_t dst_offset, size_t bytes,
                         int skip_own, const mccl_xsync_t* sync, void* stream) {
  FanoutArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  rc = check_indirect_sync(sync, ox != nullptr);
  if (rc != MCCL_OK) return rc;
  if (bytes / 16 > 0xf0000000ull) return fail(MCCL_ERR_INVALID_ARG, "message too large for one push");
  if (bytes && !src) return fail(MCCL_ERR_INVALID_ARG, "source pointer is null");
  a.src = (const char*)src;
  a.nvec = (uint32_t)(bytes / 16);
  a.tail = (uint32_t)(bytes % 16);
  a.tiles = (uint32_t)((bytes / 16 + kWave - 1) / kWave);
  a.dst_off = dst_offset;
  a.dst_mask = (1u << a.sync.n) - 1u;
  if (skip_own) a.dst_mask &= ~(1u << a.sync.rank);
  if (resolved) {
    a.dst_table = (const uint64_t*)resolved;
  } else {
    rc = check_offer_exchange(*ox, a.sync.n);
    if (rc != MCCL_OK) return rc;
    for (int r = 0; r < a.sync.n; ++r) a.offer[r] = (uint64_t*)ox->offers[r];
    offer_words(*ox->mine, a.mine);
    a.imports = ox->imports;
    a.my_buffer = (uint64_t)(uintptr_t)ox->my_buffer;
  }
  const XShape shape = xrank_shape(a.tiles, sync, a.sync.ready_epoch != 0, /*fresh_tiles=*/2);
  unsigned grid = shape.groups;
  int cus = 0;
  rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  if (ox) {
    if (!shape.packed) return fail(MCCL_ERR_INVALID_ARG, "the one-launch push with offers runs packed (max_compute_units)");
    static const unsigned per_cu = blocks_per_cu(fanout_indirect_kernel<kPackedWaves, 2>, kWave * kPackedWaves);
    grid = std::min(grid, waiting_share(per_cu, (unsigned)cus, (unsigned)a.sync.n));
    hipLaunchKernelGGL((fanout_indirect_kernel<kPackedWaves, 2>), dim3(grid), dim3(kWave * kPackedWaves), 0, (hipStream_t)stream, a);
  } else {
    if (shape.packed) return fail(MCCL_ERR_INVALID_ARG, "a push over resolved addresses runs as single wavefronts (max_compute_units 0)");
    hipLaunchKernelGGL((fanout_indirect_kernel<1, 1>), dim3(grid), dim3(kWave), shape.lds, (hipStream_t)stream, a);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "push kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_reduce_sync_resolved(const void* resolved, size_t in_offset, void* out, size_t count, int dtype, int op,
                              const mccl_xsync_t* sync, void* stream) {
  if (!resolved) return fail(MCCL_ERR_INVALID_ARG, "address table is null");
  if ((uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "address table is not 8-byte aligned");
  return reduce_sync_indirect(resolved, nullptr, in_offset, out, count, dtype, op, sync, stream);
}

int mccl_reduce_sync_offers(size_t in_offset, void* out, size_t count, int dtype, int op, const mccl_xsync_t* sync,
                            const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                            const mccl_import_table_t* imports, void* stream) {
  const OfferExchange ox{mine, my_buffer, offers, imports};
  return reduce_sync_indirect(nullptr, &ox, in_offset, out, count, dtype, op, sync, stream);
}

int mccl_fanout_sync_resolved(const void* src, const void* resolved, size_t dst_offset, size_t bytes, int skip_own,
                              const mccl_xsync_t* sync, void* stream) {
  if (!resolved) return fail(MCCL_ERR_INVALID_ARG, "address table is null");
  if ((uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "address table is not 8-byte aligned");
  return fanout_sync_indirect(src, resolved, nullptr, dst_offset, bytes, skip_own, sync, stream);
}

int mccl_fanout_sync_offers(const void* src, size_t dst_offset, size_t bytes, int skip_own, const mccl_xsync_t* sync,
                            const mccl_offer_t* mine, const void* my_buffer, void* const* offers,
                            const mccl_import_table_t* imports, void* stream) {
  const OfferExchange ox{mine, my_buffer, offers, imports};
  return fanout_sync_indirect(src, nullptr, &ox, dst_offset, bytes, skip_own, sync, stream);
}

}  // extern "C"

namespace {

// The kernels' view of at most MCCL_OFFER_RANKS segments; src_is_offset[i]: segs[i].src is no address.
int fill_lean_copy(const mccl_segment_t* segs, const int* src_rank, int nseg, const char* what, LeanCopyArgs* out, int8_t* ranks, int n,
                   uint64_t* total_chunks) {
  if (nseg < 0 || nseg > MCCL_OFFER_RANKS) return fail(MCCL_ERR_INVALID_ARG, "%s: 0 to %d segments, got %d", what, MCCL_OFFER_RANKS, nseg);
  if (nseg && !segs) return fail(MCCL_ERR_INVALID_ARG, "%s: segment table is null", what);
  int m = 0;
  uint64_t chunks = 0;
  out->chunk_prefix[0] = 0;
  for (int i = 0; i < nseg; ++i) {
    const mccl_segment_t& sg = segs[i];
    if (sg.bytes == 0) continue;
    const int from = src_rank ? src_rank[i] : -1;
    if (from >= n) return fail(MCCL_ERR_INVALID_ARG, "%s: segment %d reads from rank %d of %d", what, i, from, n);
    if ((from < 0 && !sg.src) || !sg.dst) return fail(MCCL_ERR_INVALID_ARG, "%s: segment %d has a null pointer", what, i);
    CopySeg cs;
    cs.src = (const char*)sg.src;
    cs.dst = (char*)sg.dst;
    cs.pad_ = 0;
    size_t head = (128u - (unsigned)((uintptr_t)sg.dst & 127u)) & 127u;
    if (head > sg.bytes) head = sg.bytes;
    const size_t body = sg.bytes - head;
    const uint64_t nfull = body / kCopyChunk;
    cs.head = (uint32_t)head;
    cs.last = (uint32_t)(body % kCopyChunk);
    uint64_t c = nfull + (cs.last ? 1 : 0);
    if (c == 0) c = 1;
    if (nfull > 0xf0000000ull || chunks + c > kMaxChunks) return fail(MCCL_ERR_INVALID_ARG, "%s: segment %d too large for one launch", what, i);
    cs.nfull = (uint32_t)nfull;
    if (ranks) ranks[m] = (int8_t)(from < 0 ? -1 : from);
    out->seg[m] = cs;
    chunks += c;
    out->chunk_prefix[++m] = (uint32_t)chunks;
  }
  out->nseg = m;
  *total_chunks += chunks;
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_alltoall_sync_offers(const mccl_segment_t* stage, int nstage, const mccl_segment_t* pulls, const int* src_rank, int npull,
                              const mccl_xsync_t* sync, const mccl_offer_t* mine, const uint64_t* expect_bytes, const void* my_source,
                              void* const* offers, const mccl_import_table_t* imports, void* stream) {
  ExchangeArgs a;
  memset(&a, 0, sizeof(a));
  int rc = fill_xsync(sync, &a.sync);
  if (rc != MCCL_OK) return rc;
  rc = check_indirect_sync(sync, /*one_launch=*/true);
  if (rc != MCCL_OK) return rc;
  const int n = a.sync.n;
  if (n > MCCL_OFFER_RANKS) return fail(MCCL_ERR_UNSUPPORTED, "an all-to-all with offers takes 1 to %d ranks, got %d", MCCL_OFFER_RANKS, n);
  if (!mine || !expect_bytes || !offers || !imports) return fail(MCCL_ERR_INVALID_ARG, "offers, expected lengths, offer table or import table is null");
  if ((uintptr_t)imports % 8) return fail(MCCL_ERR_INVALID_ARG, "import table is not 8-byte aligned");
  if (npull > 0 && !src_rank) return fail(MCCL_ERR_INVALID_ARG, "source rank table is null");
  uint64_t chunks = 0;
  rc = fill_lean_copy(stage, nullptr, nstage, "copies into the outboxes", &a.stage, nullptr, n, &chunks);
  if (rc != MCCL_OK) return rc;
  memset(a.src_rank, 0xff, sizeof(a.src_rank));
  rc = fill_lean_copy(pulls, src_rank, npull, "pulls", &a.pull, a.src_rank, n, &chunks);
  if (rc != MCCL_OK) return rc;
  for (int r = 0; r < n; ++r) {
    if (!offers[r]) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is null", r);
    if ((uintptr_t)offers[r] % 8) return fail(MCCL_ERR_INVALID_ARG, "offer pointer %d is not 8-byte aligned", r);
    const mccl_offer_t& o = mine[r];
    if (o.entry != MCCL_OFFER_STAGED && o.entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "offer %d names entry %u of %d", r, o.entry, MCCL_OFFER_ENTRIES);
    if (o.entry == MCCL_OFFER_STAGED && o.slot >= MCCL_OFFER_SLOTS) return fail(MCCL_ERR_INVALID_ARG, "offer %d names staging buffer %u of %d", r, o.slot, MCCL_OFFER_SLOTS);
    a.row[r] = (uint64_t*)offers[r];
    offer_words(o, a.mine[r]);
    a.expect[r] = expect_bytes[r];
  }
  a.my_source = (uint64_t)(uintptr_t)my_source;
  a.imports = imports;
  for (int k = 0; k < a.pull.nseg; ++k) {
    const CopySeg& cs = a.pull.seg[k];
    if (cs.head || cs.last || (((uintptr_t)cs.src + cs.head) & 7u)) a.invalidate = 1;  // (src: an offset from an address the launch resolves)
  }
  a.staged_count = a.sync.done_count + kStagedCountWord;
  const XShape shape = xrank_shape(chunks, sync);
  if (!shape.packed) return fail(MCCL_ERR_INVALID_ARG, "the one-launch all-to-all with offers runs packed (max_compute_units)");
  int cus = 0;
  rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  static const unsigned per_cu = blocks_per_cu(exchange_offers_kernel<kPackedWaves>, kWave * kPackedWaves);
  const unsigned grid = std::min(shape.groups, waiting_share(per_cu, (unsigned)cus, (unsigned)n));
  hipLaunchKernelGGL(exchange_offers_kernel<kPackedWaves>, dim3(grid), dim3(kWave * kPackedWaves), 0, (hipStream_t)stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "all-to-all kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

size_t mccl_allreduce_sync_shard(size_t count, int n) {
  if (n < 1) return 0;
  const size_t per = (count + (size_t)n - 1) / (size_t)n;
  return (per + 63) / 64 * 64;
}

int mccl_allreduce_sync(void* const* tensors, size_t count, int dtype, int op, const mccl_xsync_t* sync, void* stream) {
  if (!tensors) return fail(MCCL_ERR_INVALID_ARG, "tensor table is null");
  return allreduce_sync_impl(tensors, nullptr, nullptr, count, dtype, op, sync, stream);
}

int mccl_allreduce_sync_resolved(const void* resolved, size_t count, int dtype, int op, const mccl_xsync_t* sync,
                                 void* stream) {
  if (!resolved) return fail(MCCL_ERR_INVALID_ARG, "address table is null");
  if ((uintptr_t)resolved % 8) return fail(MCCL_ERR_INVALID_ARG, "address table is not 8-byte aligned");
  if (sync && (sync->ready_epoch != 0 || sync->done_epoch == 0))
    return fail(MCCL_ERR_INVALID_ARG, "the allreduce over resolved addresses runs behind a barrier: ready_epoch 0, done_epoch set");
  return allreduce_sync_impl(nullptr, resolved, nullptr, count, dtype, op, sync, stream);
}

int mccl_allreduce_sync_offers(size_t count, int dtype, int op, const mccl_xsync_t* sync, const mccl_offer_t* mine,
                               const void* my_buffer, void* const* offers, const mccl_import_table_t* imports, void* stream) {
  if (!mine || !offers || !imports) return fail(MCCL_ERR_INVALID_ARG, "offer, offer table or import table is null");
  if ((uintptr_t)imports % 8) return fail(MCCL_ERR_INVALID_ARG, "import table is not 8-byte aligned");
  if (mine->entry != MCCL_OFFER_STAGED && mine->entry >= MCCL_OFFER_ENTRIES) return fail(MCCL_ERR_INVALID_ARG, "offer names entry %u of %d", mine->entry, MCCL_OFFER_ENTRIES);
  if (sync && (sync->ready_epoch == 0 || sync->done_epoch == 0 || sync->max_compute_units == 0))
    return fail(MCCL_ERR_INVALID_ARG, "the one-launch allreduce with offers needs ready_epoch, done_epoch and max_compute_units");
  const OfferExchange ox{mine, my_buffer, offers, imports};
  return allreduce_sync_impl(nullptr, nullptr, &ox, count, dtype, op, sync, stream);
}

int mccl_copy_segments(const mccl_segment_t* segs, int nseg, void* stream) {
  if (nseg < 0) return fail(MCCL_ERR_INVALID_ARG, "negative segment count");
  if (nseg == 0) return MCCL_OK;
  if (!segs) return fail(MCCL_ERR_INVALID_ARG, "segment table is null");
  return launch_copy(segs, nseg, (hipStream_t)stream);
}

int mccl_allgather_n(const void* const* in, int n, void* out, size_t bytes_per_rank, void* stream) {
  if (!in) return fail(MCCL_ERR_INVALID_ARG, "input pointer table is null");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  if (bytes_per_rank == 0) return MCCL_OK;
  if (!out) return fail(MCCL_ERR_INVALID_ARG, "output pointer is null");
  mccl_segment_t segs[MCCL_MAX_RANKS];
  for (int k = 0; k < n; ++k) {
    if (!in[k]) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d is null", k);
    segs[k].src = in[k];
    segs[k].dst = (char*)out + (size_t)k * bytes_per_rank;
    segs[k].bytes = bytes_per_rank;
  }
  return launch_copy(segs, n, (hipStream_t)stream);
}

int mccl_alltoallv_n(const void* const* in, void* const* out, int n, const int64_t* split_rows,
                     size_t row_bytes, void* stream) {
  if (!in || !out || !split_rows) return fail(MCCL_ERR_INVALID_ARG, "null table");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  for (int i = 0; i < n * n; ++i)
    if (split_rows[i] < 0) return fail(MCCL_ERR_INVALID_ARG, "negative split size");
  // All n x n segments, destination by destination (each output is written front to back), in as
  // few launches as the segment table allows: one for eight ranks.  One launch per destination
  // was 5x slower on a 1 MiB exchange (8 launches of 4-5 us), 2x at 56 MiB and still 18 % at
  // 448 MiB (every launch ends in a tail of half-empty CUs).
  mccl_segment_t segs[kBatchedSegs];
  size_t send_off[MCCL_MAX_RANKS];  // rows of rank r already addressed to lower destinations
  for (int r = 0; r < n; ++r) send_off[r] = 0;
  int m = 0;
  for (int d = 0; d < n; ++d) {
    size_t roff = 0;
    for (int r = 0; r < n; ++r) {
      const size_t rows = (size_t)split_rows[r * n + d];
      if (rows) {
        if (!in[r] || !out[d]) return fail(MCCL_ERR_INVALID_ARG, "null buffer for a non-empty segment");
        segs[m].src = (const char*)in[r] + send_off[r] * row_bytes;
        segs[m].dst = (char*)out[d] + roff * row_bytes;
        segs[m].bytes = rows * row_bytes;
        ++m;
      }
      roff += rows;
      send_off[r] += rows;
      if (m == kBatchedSegs || (m && d == n - 1 && r == n - 1)) {
        int rc = launch_copy(segs, m, (hipStream_t)stream);
        if (rc != MCCL_OK) return rc;
        m = 0;
      }
    }
  }
  return MCCL_OK;
}

int mccl_alltoallv_pull(const void* const* in, int n, void* out, const size_t* send_displ_bytes,
                        const size_t* recv_bytes, void* stream) {
  if (!in || !send_displ_bytes || !recv_bytes) return fail(MCCL_ERR_INVALID_ARG, "null table");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  mccl_segment_t segs[MCCL_MAX_RANKS];
  size_t off = 0;
  int m = 0;
  for (int r = 0; r < n; ++r) {
    if (recv_bytes[r]) {
      if (!in[r] || !out) return fail(MCCL_ERR_INVALID_ARG, "null buffer for a non-empty segment");
      segs[m].src = (const char*)in[r] + send_displ_bytes[r];
      segs[m].dst = (char*)out + off;
      segs[m].bytes = recv_bytes[r];
      ++m;
    }
    off += recv_bytes[r];
  }
  return launch_copy(segs, m, (hipStream_t)stream);
}

int mccl_pack(const void* const* src, const size_t* bytes, int n, void* dst, void* stream) {
  if (n < 0) return fail(MCCL_ERR_INVALID_ARG, "negative count");
  if (n == 0) return MCCL_OK;
  if (!src || !bytes) return fail(MCCL_ERR_INVALID_ARG, "null table");
  size_t total = 0;
  for (int i = 0; i < n; ++i) total += bytes[i];
  if (!total) return MCCL_OK;
  if (!dst) return fail(MCCL_ERR_INVALID_ARG, "destination pointer is null");
  size_t off = 0;
  for (int i0 = 0; i0 < n; i0 += kMaxSegs) {
    mccl_segment_t segs[kMaxSegs];
    const int m = (n - i0 < kMaxSegs) ? n - i0 : kMaxSegs;
    for (int i = 0; i < m; ++i) {
      segs[i].src = src[i0 + i];
      segs[i].dst = (char*)dst + off;
      segs[i].bytes = bytes[i0 + i];
      off += bytes[i0 + i];
    }
    int rc = launch_copy(segs, m, (hipStream_t)stream);
    if (rc != MCCL_OK) return rc;
  }
  return MCCL_OK;
}

int mccl_unpack(const void* src, void* const* dst, const size_t* bytes, int n, void* stream) {
  if (n < 0) return fail(MCCL_ERR_INVALID_ARG, "negative count");
  if (n == 0) return MCCL_OK;
  if (!dst || !bytes) return fail(MCCL_ERR_INVALID_ARG, "null table");
  size_t total = 0;
  for (int i = 0; i < n; ++i) total += bytes[i];
  if (!total) return MCCL_OK;
  if (!src) return fail(MCCL_ERR_INVALID_ARG, "source pointer is null");
  size_t off = 0;
  for (int i0 = 0; i0 < n; i0 += kMaxSegs) {
    mccl_segment_t segs[kMaxSegs];
    const int m = (n - i0 < kMaxSegs) ? n - i0 : kMaxSegs;
    for (int i = 0; i < m; ++i) {
      segs[i].src = (const char*)src + off;
      segs[i].dst = dst[i0 + i];
      segs[i].bytes = bytes[i0 + i];
      off += bytes[i0 + i];
    }
    int rc = launch_copy(segs, m, (hipStream_t)stream);
    if (rc != MCCL_OK) return rc;
  }
  return MCCL_OK;
}

int mccl_gather_rows(const void* src, size_t src_rows, const int64_t* row_index, size_t nrows,
                     size_t row_bytes, void* dst, void* stream) {
  if (nrows == 0 || row_bytes == 0) return MCCL_OK;
  GatherSpec g{src, src_rows, row_index, dst, nrows};
  return launch_gather(&g, 1, row_bytes, (hipStream_t)stream);
}

int mccl_moe_dispatch_n(const void* const* hidden, const size_t* hidden_rows,
                        const int64_t* const* row_index, void* const* out, int n,
                        const int64_t* split_rows, size_t row_bytes, void* stream) {
  if (!hidden || !hidden_rows || !row_index || !out || !split_rows) return fail(MCCL_ERR_INVALID_ARG, "null table");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  for (int i = 0; i < n * n; ++i)
    if (split_rows[i] < 0) return fail(MCCL_ERR_INVALID_ARG, "negative split size");
  // as mccl_alltoallv_n: destination by destination, in as few launches as the segment table allows
  GatherSpec specs[kBatchedSegs];
  size_t send_off[MCCL_MAX_RANKS];
  for (int r = 0; r < n; ++r) send_off[r] = 0;
  int m = 0;
  for (int d = 0; d < n; ++d) {
    size_t roff = 0;
    for (int r = 0; r < n; ++r) {
      const size_t rows = (size_t)split_rows[r * n + d];
      if (rows) {
        if (!hidden[r] || !row_index[r] || !out[d]) return fail(MCCL_ERR_INVALID_ARG, "null buffer for a non-empty segment");
        specs[m++] = GatherSpec{hidden[r], hidden_rows[r], row_index[r] + send_off[r], (char*)out[d] + roff * row_bytes, rows};
      }
      roff += rows;
      send_off[r] += rows;
      if (m == kBatchedSegs || (m && d == n - 1 && r == n - 1)) {
        int rc = launch_gather(specs, m, row_bytes, (hipStream_t)stream);
        if (rc != MCCL_OK) return rc;
        m = 0;
      }
    }
  }
  return MCCL_OK;
}

}  // extern "C"

namespace {

int launch_route_counts(const int32_t* expert_ids, size_t npairs, int n_experts, uint32_t* counters, bool clear_first,
                        int64_t* counts, hipStream_t s) {
  if (n_experts < 1 || n_experts > kRouteMaxExperts)
    return fail(MCCL_ERR_INVALID_ARG, "expert count %d outside [1, %d]", n_experts, kRouteMaxExperts);
  if (!counts) return fail(MCCL_ERR_INVALID_ARG, "counts pointer is null");
  if (npairs && !expert_ids) return fail(MCCL_ERR_INVALID_ARG, "expert id pointer is null");
  if ((uintptr_t)expert_ids % 4 || (uintptr_t)counts % 8 || (uintptr_t)counters % 4)
    return fail(MCCL_ERR_INVALID_ARG, "expert ids, counters or counts not aligned to their element size");
  int cus = 0;
  int rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  const unsigned fin = (unsigned)((n_experts + kRouteBlock - 1) / kRouteBlock);
  if (clear_first) hipLaunchKernelGGL(route_clear_kernel, dim3(fin), dim3(kRouteBlock), 0, s, counters, (uint32_t)n_experts);
  if (npairs) {
    uint64_t grid = (npairs + (uint64_t)kRouteBlock * 8 - 1) / ((uint64_t)kRouteBlock * 8);  // about 8 pairs per lane
    if (grid > (uint64_t)cus * 4) grid = (uint64_t)cus * 4;
    hipLaunchKernelGGL(route_count_kernel, dim3((unsigned)grid), dim3(kRouteBlock), 0, s, expert_ids, (uint64_t)npairs,
                       (uint32_t)n_experts, counters);
  }
  hipLaunchKernelGGL(route_finish_kernel, dim3(fin), dim3(kRouteBlock), 0, s, counters, (uint32_t)n_experts, counts);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "route count launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_route_counts(const int32_t* expert_ids, size_t npairs, int n_experts, void* workspace, int64_t* counts,
                      void* stream) {
  if (!workspace) return fail(MCCL_ERR_INVALID_ARG, "workspace pointer is null");
  return launch_route_counts(expert_ids, npairs, n_experts, (uint32_t*)workspace, /*clear_first=*/true, counts,
                             (hipStream_t)stream);
}

}  // extern "C"

// The counters of mccl_route_counts_noalloc: one array per GPU the library runs on, held until the
// process ends.  The name is a host-side handle, not a device address: host code uses the pointer
// hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) uint32_t scratch[MCCL_ROUTE_MAX_EXPERTS];

namespace {

uint32_t* g_scratch_ptr[64];
hipError_t g_scratch_err[64];
std::once_flag g_scratch_once[64];

// Address of `scratch` on the current device (looked up once per device, with that device current).
int scratch_of_current_device(uint32_t** ptr) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(MCCL_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  std::call_once(g_scratch_once[dev], [dev]() {
    void* p = nullptr;
    g_scratch_err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
  });
  if (g_scratch_err[dev] != hipSuccess || !g_scratch_ptr[dev])
    return fail(MCCL_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(g_scratch_err[dev]));
  *ptr = g_scratch_ptr[dev];
  return MCCL_OK;
}

}  // namespace

extern "C" {

int mccl_route_counts_noalloc(const int32_t* expert_ids, size_t npairs, int n_experts, int64_t* counts,
                              void* stream) {
  if (n_experts > MCCL_ROUTE_MAX_EXPERTS)
    return fail(MCCL_ERR_INVALID_ARG, "%d experts exceed the %d counters the library holds; use mccl_route_counts with a workspace",
                n_experts, MCCL_ROUTE_MAX_EXPERTS);
  uint32_t* counters = nullptr;
  int rc = scratch_of_current_device(&counters);
  if (rc != MCCL_OK) return rc;
  // the array keeps whatever the last call left (zero after a complete call): cleared first anyway
  return launch_route_counts(expert_ids, npairs, n_experts, counters, /*clear_first=*/true, counts, (hipStream_t)stream);
}

int mccl_moe_combine(const void* const* x, const size_t* x_rows, int n, const int32_t* src_rank,
                     const int64_t* src_row, const float* weights, size_t tokens, int topk,
                     size_t hidden_elems, int dtype, void* y, void* stream) {
  if (!x || !x_rows) return fail(MCCL_ERR_INVALID_ARG, "null table");
  if (n < 1 || n > MCCL_MAX_RANKS) return fail(MCCL_ERR_INVALID_ARG, "rank count %d outside [1, %d]", n, MCCL_MAX_RANKS);
  if (dtype != MCCL_BF16 && dtype != MCCL_F16 && dtype != MCCL_F32)
    return fail(MCCL_ERR_UNSUPPORTED, "moe_combine is defined for bf16, f16 and f32");
  if (topk < 1 || topk > 64) return fail(MCCL_ERR_INVALID_ARG, "topk %d outside [1, 64]", topk);
  if (tokens == 0 || hidden_elems == 0) return MCCL_OK;
  if (!src_rank || !src_row || !weights || !y) return fail(MCCL_ERR_INVALID_ARG, "null pointer");
  const size_t row_bytes = hidden_elems * dtype_size(dtype);
  if (row_bytes % 16) return fail(MCCL_ERR_UNSUPPORTED, "moe_combine needs rows that are a multiple of 16 bytes");
  if ((uintptr_t)y & 15u) return fail(MCCL_ERR_INVALID_ARG, "output is not 16-byte aligned");
  if (((uintptr_t)src_rank & 3u) || ((uintptr_t)src_row & 7u) || ((uintptr_t)weights & 3u))
    return fail(MCCL_ERR_INVALID_ARG, "index or weight table is misaligned");
  CombineArgs a;
  memset(&a, 0, sizeof(a));
  for (int r = 0; r < n; ++r) {
    if (x_rows[r] && !x[r]) return fail(MCCL_ERR_INVALID_ARG, "input pointer %d is null", r);
    if ((uintptr_t)x[r] & 15u) return fail(MCCL_ERR_INVALID_ARG, "input %d is not 16-byte aligned", r);
    if (x_rows[r] > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "input %d has too many rows", r);
    a.x[r] = (const char*)x[r];
    a.x_rows[r] = (uint32_t)x_rows[r];
  }
  const size_t row_vecs = row_bytes / 16;
  const size_t ppr = (row_vecs + kWave - 1) / kWave;
  if (tokens * ppr > kMaxChunks || row_vecs > 0xffffffffull) return fail(MCCL_ERR_INVALID_ARG, "message too large");
  a.src_rank = src_rank;
  a.src_row = src_row;
  a.w = weights;
  a.y = (char*)y;
  a.tokens = (uint32_t)tokens;
  a.topk = (uint32_t)topk;
  a.row_vecs = (uint32_t)row_vecs;
  a.pieces_per_row = (uint32_t)ppr;
  size_t ppw = (size_t)g_tune[MCCL_TUNE_COMBINE_PIECES_PER_WAVE];
  if (ppw < 1) ppw = 1;
  if (ppw > ppr) ppw = ppr;
  a.pieces_per_wave = (uint32_t)ppw;
  a.waves_per_row = (uint32_t)((ppr + ppw - 1) / ppw);
  a.n = n;
  int cus = 0;
  int rc = device_cus(&cus);
  if (rc != MCCL_OK) return rc;
  // One wavefront per chunk of a row, no residency cap (5.7 TB/s uncapped, 5.1 at 8 wavefronts
  // per CU).  Top-k up to 2, 4 and 8 are kernels of their own: with fewer row buffers a
  // wavefront needs fewer registers and more of them are resident (top-2 at 4096-wide rows 63 ->
  // 67 % of the HBM peak, top-4 at 5120 68 -> 74 %, top-1 47 -> 63 %); four row buffers deep
  // instead of two for top-2 changed nothing and cost top-1 seven points.  Measured and not adopted: a persistent grid whose wavefronts look up the next
  // chunk's routing entries while they stream the current rows (the knob below; 3-8 % slower at
  // every grid size, so the lookup is not what bounds the kernel), and one contiguous range of
  // tokens per XCD so that the wavefronts sharing routing entries meet in one L2 (9 % slower).
  uint64_t grid = (uint64_t)tokens * a.waves_per_row;
  if (grid > kMaxGridX) grid = kMaxGridX;
  if (topk <= 8 && g_tune[MCCL_TUNE_COMBINE_WAVES_PER_CU] > 0) {
    const uint64_t persistent = (uint64_t)cus * (uint64_t)g_tune[MCCL_TUNE_COMBINE_WAVES_PER_CU];
    if (grid > persistent) grid = persistent;
  }
  const unsigned lds = 0;
  hipStream_t s = (hipStream_t)stream;
  const dim3 g3((unsigned)grid), b3(kWave);
  const int group = topk <= 2 ? 2 : topk <= 4 ? 4 : topk <= 8 ? 8 : 0;
#define MCCL_LAUNCH_COMBINE(DT)                                                                     \
  switch (group) {                                                                                  \
    case 2: hipLaunchKernelGGL((moe_combine_kernel<DT, 2>), g3, b3, lds, s, a); break;              \
    case 4: hipLaunchKernelGGL((moe_combine_kernel<DT, 4>), g3, b3, lds, s, a); break;              \
    case 8: hipLaunchKernelGGL((moe_combine_kernel<DT, 8>), g3, b3, lds, s, a); break;              \
    default: hipLaunchKernelGGL((moe_combine_kernel<DT, 0>), g3, b3, lds, s, a); break;             \
  }
  switch (dtype) {
    case MCCL_BF16: MCCL_LAUNCH_COMBINE(MCCL_BF16); break;
    case MCCL_F16: MCCL_LAUNCH_COMBINE(MCCL_F16); break;
    default: MCCL_LAUNCH_COMBINE(MCCL_F32); break;
  }
#undef MCCL_LAUNCH_COMBINE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MCCL_ERR_HIP, "combine kernel launch failed: %s", hipGetErrorString(e));
  return MCCL_OK;
}

}  // extern "C"
