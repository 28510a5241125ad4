// What the translation units of the c10d backend share and nobody else sees: constants, the layout
// of a rank's arena and of the shared-memory control block, small helpers.
#pragma once
#include "process_group_ccl.hpp"

#include <ATen/hip/impl/HIPCachingAllocatorMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/record_function.h>
#include <c10/core/DeviceGuard.h>
#include <fcntl.h>
#include <sched.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <thread>

#include "mccl.h"

namespace mccl_pg {


constexpr int kMaxWorld = MCCL_MAX_RANKS;
constexpr int kTableMax = 2 * kMaxWorld + 8;
constexpr size_t kStageMin = 2u << 20;   // first staging allocation
constexpr size_t kStageMaxDefault = 1u << 30;  // one staging window; keeps every IPC allocation < 2 GiB
// Rank r's staging buffer starts (r mod 16) x 4 KiB into its allocation.  Equal-sized allocations
// tend to sit a power of two apart, and rank buffers at such a spacing make every wavefront of the
// reduction hit the same DRAM banks with all its loads (6-20 % of bandwidth on large messages).
constexpr size_t kStageStagger = 4096;
constexpr size_t kStageStaggerSlots = 16;
inline size_t stageOffset(int rank) { return (size_t)(rank % (int)kStageStaggerSlots) * kStageStagger; }
constexpr uint32_t kMagic = 0x4d43434c;  // "MCCL"
// Collectives staging at most this many bytes run on the caller's stream: the host waits for the
// copy-in in any case, there is no kernel long enough to be worth overlapping, and the
// cross-stream event dependency alone costs more than the kernel.
constexpr size_t kInlineStreamMax = 1u << 20;
// Allreduce messages of at least this many bytes, in groups of at least kTwoShotMinRanks, use
// the two-shot algorithm: every rank reduces only its 1/W shard of the staged inputs, then all
// ranks gather the W finished shards.  Per rank that moves about (4 + 1/W) S bytes instead of
// (W + 3) S; results are identical (same ascending-rank chain per element).  It is also the
// algorithm for W GPUs on xGMI, where each shard is reduced by the GPU that owns it.
constexpr size_t kTwoShotMinBytes = 4u << 20;
constexpr int kTwoShotMinRanks = 4;
// Device-synchronised groups: allreduces of at most this many bytes (and at most
// MCCL_FUSED_MAX_RANKS ranks) are one launch of mccl_allreduce_fused on the caller's stream.
constexpr size_t kFusedMaxBytes = 1u << 20;
// What a workgroup of the one-launch small allreduce covers at most (sixteen wavefronts, four
// 1 KiB tiles each) when the launch is limited to a number of compute units.
constexpr size_t kFusedBytesPerComputeUnit = 16u * 4u * MCCL_FUSED_TILE_BYTES;
constexpr unsigned kComputeUnits = 256;  // of an MI355X
// Tensors of at least this many bytes are offered to the peers in place (zero-copy) instead of
// being staged; an allocation must stay below 2 GiB to be shared between processes.
constexpr size_t kZeroCopyMinBytes = 1u << 20;
constexpr uint64_t kShareMaxAllocation = (2ull << 30) - (64u << 20);
constexpr int kMaxExports = 32;
constexpr int kEmptyShare = kMaxExports;  // "this rank's range is empty": nothing to map
// Layout of a rank's arena (device memory mapped by every peer at start-up).
constexpr size_t kArenaBarOff = 0;        // 64-bit barrier word
constexpr size_t kArenaFinalOff = 128;    // 64-bit departure word
constexpr size_t kArenaFusedFlagsOff = 4096;                 // two sets of tile flags, 8 KiB each
constexpr size_t kArenaFusedFlagsStride = 8192;
constexpr size_t kArenaFusedStageOff = 64u << 10;            // two staging buffers of 1 MiB, each
constexpr size_t kArenaFusedStageStride = kFusedMaxBytes + (64u << 10);  // followed by room for the rank stagger
constexpr size_t kArenaDoneCountOff = 24u << 10;  // MCCL_SYNC_COUNTER_BYTES of workgroup counters of the one-launch collectives
constexpr size_t kArenaFusedStateOff = 2048;  // MCCL_FUSED_STATE_BYTES: the device-resident epoch of the one-launch small allreduce
constexpr size_t kArenaOfferOff = 3072;       // two mccl_offer_t, 64 bytes apart: what this rank's tensor of a collective is
constexpr size_t kArenaOfferStride = 64;
constexpr size_t kArenaOfferRowOff = 3584;    // two rows of MCCL_OFFER_RANKS offers (all-to-all: one offer per reader), 256 bytes each
constexpr size_t kArenaOfferRowStride = MCCL_OFFER_RANKS * sizeof(mccl_offer_t);
constexpr size_t kArenaImportTableOff = 32u << 10;  // mccl_import_table_t: the peers' allocations as this rank has mapped them
constexpr size_t kArenaResolvedOff = 40u << 10;     // MCCL_OFFER_RANKS addresses: the ranks' tensors of the collective under way
constexpr size_t kArenaBytes = kArenaFusedStageOff + 2 * kArenaFusedStageStride;
static_assert(kArenaFusedStateOff + MCCL_FUSED_STATE_BYTES <= kArenaOfferOff && kArenaOfferOff + 2 * kArenaOfferStride <= kArenaFusedFlagsOff, "the offers lie between the epoch state and the flags");
static_assert(sizeof(mccl_offer_t) <= kArenaOfferStride, "an offer fits its slot");
static_assert(kArenaOfferOff + 2 * kArenaOfferStride <= kArenaOfferRowOff && kArenaOfferRowOff + 2 * kArenaOfferRowStride <= kArenaFusedFlagsOff, "the rows of offers lie between the offers and the flags");
// Outboxes of the all-to-all with standing offers: buffers of 2 MiB << level, level < kOutboxLevels.
constexpr size_t kOutboxMin = 2u << 20;
constexpr int kOutboxLevels = 10;  // up to 1 GiB: an allocation must stay below 2 GiB to be shared
inline int outboxLevel(size_t bytes) {
  int level = 0;
  while ((kOutboxMin << level) < bytes) ++level;
  return level;
}
static_assert(kArenaImportTableOff + sizeof(mccl_import_table_t) <= kArenaResolvedOff, "the import table ends before the resolved addresses");
static_assert(kArenaResolvedOff + MCCL_OFFER_RANKS * 8 <= kArenaFusedStageOff, "the resolved addresses end before the staging buffers");
static_assert(kMaxExports == MCCL_OFFER_ENTRIES, "an offer names an entry of the export table");
static_assert(kFusedMaxBytes / MCCL_FUSED_TILE_BYTES * 4 <= kArenaFusedFlagsStride, "tile flags must fit their slot");
static_assert(kArenaFusedFlagsOff + 2 * kArenaFusedFlagsStride <= kArenaDoneCountOff, "the flags end before the counters");
static_assert(kArenaDoneCountOff + MCCL_SYNC_COUNTER_BYTES <= kArenaImportTableOff, "the counters end before the import table");
static_assert(kArenaFusedStateOff + MCCL_FUSED_STATE_BYTES <= kArenaFusedFlagsOff, "the epoch state ends before the flags");

#define HIP_CHECK(expr)                                                                     \
  do {                                                                                      \
    hipError_t e_ = (expr);                                                                 \
    TORCH_CHECK(e_ == hipSuccess, "ccl backend: ", #expr, " failed: ", hipGetErrorString(e_)); \
  } while (0)

#define MCCL_CHECK(expr)                                                         \
  do {                                                                           \
    int rc_ = (expr);                                                            \
    TORCH_CHECK(rc_ == MCCL_OK, "ccl backend: ", #expr, ": ", mccl_last_error()); \
  } while (0)

inline bool envFlag(const char* name, bool dflt) {
  const char* v = std::getenv(name);
  if (!v || !*v) return dflt;
  return std::atoi(v) != 0;
}

// cclDatatypes of the reference (src/utils.cpp:46-58)
inline int dtypeCode(at::ScalarType t) {
  switch (t) {
    case at::kByte: return MCCL_U8;
    case at::kChar: return MCCL_I8;
    case at::kShort: return MCCL_I16;
    case at::kInt: return MCCL_I32;
    case at::kLong: return MCCL_I64;
    case at::kHalf: return MCCL_F16;
    case at::kFloat: return MCCL_F32;
    case at::kDouble: return MCCL_F64;
    case at::kBFloat16: return MCCL_BF16;
    case at::kBool: return MCCL_U8;
    default: TORCH_CHECK(false, "ccl backend: unsupported data type ", c10::toString(t));
  }
}

inline const char* reduceOpName(c10d::ReduceOp::RedOpType op) {
  switch (op) {
    case c10d::ReduceOp::SUM: return "SUM";
    case c10d::ReduceOp::AVG: return "AVG";
    case c10d::ReduceOp::PRODUCT: return "PRODUCT";
    case c10d::ReduceOp::MIN: return "MIN";
    case c10d::ReduceOp::MAX: return "MAX";
    case c10d::ReduceOp::BAND: return "BAND";
    case c10d::ReduceOp::BOR: return "BOR";
    case c10d::ReduceOp::BXOR: return "BXOR";
    case c10d::ReduceOp::PREMUL_SUM: return "PREMUL_SUM";
    default: return "UNUSED";
  }
}

// cclOps (src/utils.cpp:38-44) and the device allow-list (src/dispatch_stub.h:320-335).  AVG is
// accepted for floating-point tensors (the reference rejects it on device).
inline int opCode(const c10d::ReduceOp& op, at::ScalarType t) {
  switch (op.op_) {
    case c10d::ReduceOp::SUM: return MCCL_SUM;
    case c10d::ReduceOp::PRODUCT: return MCCL_PROD;
    case c10d::ReduceOp::MIN: return MCCL_MIN;
    case c10d::ReduceOp::MAX: return MCCL_MAX;
    case c10d::ReduceOp::AVG:
      TORCH_CHECK(at::isFloatingType(t), "Cannot use ReduceOp.AVG with integer tensors on CUDA");
      return MCCL_AVG;
    default:
      TORCH_CHECK(false, "Cannot use ReduceOp.", reduceOpName(op.op_), " with CUDA");
  }
}

inline void checkRank(int rank, int size) {
  if (!(rank >= 0 && rank < size)) throw std::invalid_argument("unexpected rank");
}

inline size_t nbytes(const at::Tensor& t) { return (size_t)t.numel() * t.element_size(); }

inline bool rangesOverlap(const void* a, size_t a_bytes, const void* b, size_t b_bytes) {
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a_bytes && b_bytes && a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

// A rank's small tensor (the output of reduce_scatter_tensor, the input of all_gather_into_tensor)
// against its large one of W slices: does it touch any slice but this rank's own?  In its own slice
// it is the in-place form; anywhere else the peers would read (or write) the large tensor in place
// while this rank writes (reads) the small one, so such a call is staged, where the copy-in comes
// first.
inline bool touchesForeignSlice(const void* small, size_t small_bytes, const void* large, size_t slice_bytes, int W, int me) {
  if (!rangesOverlap(small, small_bytes, large, slice_bytes * (size_t)W)) return false;
  const uintptr_t s0 = (uintptr_t)small, own = (uintptr_t)large + (size_t)me * slice_bytes;
  return !(s0 >= own && s0 + small_bytes <= own + slice_bytes);
}

inline size_t roundUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Device-to-device copy on the compute queue (the library's own segment copy): no DMA-engine
// round trip for small messages, full copy bandwidth for large ones.
inline void copyAsync(void* dst, const void* src, size_t bytes, hipStream_t s) {
  if (!bytes) return;
  mccl_segment_t seg{src, dst, bytes};
  int rc = mccl_copy_segments(&seg, 1, s);
  TORCH_CHECK(rc == MCCL_OK, "ccl backend: copy-in failed: ", mccl_last_error());
}


// ---------------------------------------------------------------------------------------------
// shared-memory control block
// ---------------------------------------------------------------------------------------------
constexpr int kRing = 4;  // ProcessGroupCCL::kP2PRing
constexpr size_t kP2PMinBytes = 64u << 10;

// One staging buffer of the sender and the message it currently holds.
struct P2PEntry {
  uint64_t gen;       // bumped whenever the sender replaces the buffer
  uint64_t ptr;       // the sender's address (threads of the same process use it directly)
  uint64_t capacity;
  uint64_t bytes;     // payload of the message
  hipIpcMemHandle_t handle;
};

// Mailbox of one ordered pair; lives in the sender's slot, indexed by destination.  Message k
// (from 1) travels in ring[(k - 1) % kRing]; the sender writes the entry and then `posted`, the
// receiver reads the entry after it has seen `posted` and writes `consumed` once its copy out of
// the buffer has finished.
struct alignas(64) P2PBox {
  std::atomic<uint64_t> posted;
  std::atomic<uint64_t> consumed;
  P2PEntry ring[kRing];
};

struct alignas(128) RankSlot {
  std::atomic<uint64_t> arrive;  // host barrier: epoch this rank has reached
  std::atomic<uint64_t> entered;  // collectives this rank's host thread has entered (device-synchronised groups)
  std::atomic<uint64_t> failed;  // non-zero once the rank gave up; peers stop waiting
  std::atomic<uint64_t> departed;  // non-zero once the rank's group object is being destroyed
  int64_t pid;
  // What the rank tells its peers for one collective: written before it arrives at the host
  // rendezvous of that collective, read by the peers after it.  Two records alternate, counted in
  // collectives that rendezvous: a rank can only be one rendezvous ahead of the slowest reader
  // (it cannot pass the next rendezvous before everybody has arrived there, i.e. is done reading).
  struct Published {
    uint64_t stage_gen;            // the staging buffer of the device slot this collective uses
    uint64_t stage_ptr;
    hipIpcMemHandle_t stage_handle;
    // zero-copy offer: entry of `exports` (< 0: cannot share; kEmptyShare: empty range), its
    // generation, and where the offered range starts inside the allocation
    int64_t share_entry;
    uint64_t share_gen;
    uint64_t share_off;
    int64_t table[kTableMax];      // per-collective scalars (split sizes, displacements)
  } pub[2];
  // device-side synchronisation: the rank's arena (flag words, fused-allreduce staging)
  uint64_t arena_ptr;
  hipIpcMemHandle_t arena_handle;
  // zero-copy: allocations of this rank the peers may map
  struct ExportEntry {
    std::atomic<uint64_t> gen;  // bumped whenever the entry changes or its allocation is freed
    // `gen` while the fields below describe a live allocation, 0 while they are being rewritten or
    // the allocation is gone: what a peer that reads the table on its own (no rendezvous) goes by
    std::atomic<uint64_t> live;
    uint64_t base;
    uint64_t size;
    hipIpcMemHandle_t handle;
  } exports[kMaxExports];
  // Standing offers: acked[o][e] = the generation of rank o's export entry e that THIS rank has
  // mapped, and the first collective of this rank whose kernels see that mapping.  Rank o offers
  // the entry to its peers' kernels only when every peer's ack says "mapped, from a collective not
  // later than this one".
  struct Ack {
    std::atomic<uint64_t> gen;
    std::atomic<uint64_t> from_seq;
  } acked[MCCL_OFFER_RANKS][kMaxExports];
  // All-to-all with standing offers.  outbox[d] is what this rank keeps for the pieces it sends rank d
  // when it cannot offer them in place: one buffer per size class (level), created when a piece first
  // needs it -- which rank d knows as well as this rank, because the length of the piece is the one
  // thing both of them know.  `ready` is written last.
  struct OutboxLevel {
    std::atomic<uint64_t> ready;
    uint64_t ptr;
    hipIpcMemHandle_t handle;
  };
  struct Outbox {
    OutboxLevel level[kOutboxLevels];
  } outbox[MCCL_OFFER_RANKS];
  // A piece too large for any outbox is always read in place: big[d] says where the piece of this
  // rank's collective #seq for rank d is, and rank d maps it before it enqueues (big_seen[r]: the last
  // record of rank r's that this rank has read; the owner does not overwrite an unread one).
  struct BigPiece {
    std::atomic<uint64_t> seq;
    int64_t entry;   // of this rank's export table; < 0: cannot be shared
    uint64_t gen;
  } big[MCCL_OFFER_RANKS];
  std::atomic<uint64_t> big_seen[MCCL_OFFER_RANKS];
  P2PBox p2p[kMaxWorld];
};

struct Control {
  uint32_t magic;
  uint32_t world;
  RankSlot slot[1];  // world entries
};

static_assert(std::atomic<uint64_t>::is_always_lock_free, "barrier counters must be lock-free");

// Groups that have exported allocations to their peers, for the allocator's segment-free
// notification (pg_sharing.cpp).
extern std::mutex g_registry_mutex;
extern std::vector<ProcessGroupCCL*> g_registry;
void attachSegmentTracker();

}  // namespace mccl_pg
