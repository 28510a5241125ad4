// c10d backend "ccl" for ROCm tensors: see process_group_ccl.hpp for the design.
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

namespace {

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
constexpr size_t kArenaImportTableOff = 32u << 10;  // mccl_import_table_t: the peers' allocations as this rank has mapped them
constexpr size_t kArenaResolvedOff = 40u << 10;     // MCCL_OFFER_RANKS addresses: the ranks' tensors of the collective under way
constexpr size_t kArenaBytes = kArenaFusedStageOff + 2 * kArenaFusedStageStride;
static_assert(kArenaFusedStateOff + MCCL_FUSED_STATE_BYTES <= kArenaOfferOff && kArenaOfferOff + 2 * kArenaOfferStride <= kArenaFusedFlagsOff, "the offers lie between the epoch state and the flags");
static_assert(sizeof(mccl_offer_t) <= kArenaOfferStride, "an offer fits its slot");
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

bool envFlag(const char* name, bool dflt) {
  const char* v = std::getenv(name);
  if (!v || !*v) return dflt;
  return std::atoi(v) != 0;
}

// cclDatatypes of the reference (src/utils.cpp:46-58)
int dtypeCode(at::ScalarType t) {
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

const char* reduceOpName(c10d::ReduceOp::RedOpType op) {
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
int opCode(const c10d::ReduceOp& op, at::ScalarType t) {
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

void checkRank(int rank, int size) {
  if (!(rank >= 0 && rank < size)) throw std::invalid_argument("unexpected rank");
}

size_t nbytes(const at::Tensor& t) { return (size_t)t.numel() * t.element_size(); }

bool rangesOverlap(const void* a, size_t a_bytes, const void* b, size_t b_bytes) {
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a_bytes && b_bytes && a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

// A rank's small tensor (the output of reduce_scatter_tensor, the input of all_gather_into_tensor)
// against its large one of W slices: does it touch any slice but this rank's own?  In its own slice
// it is the in-place form; anywhere else the peers would read (or write) the large tensor in place
// while this rank writes (reads) the small one, so such a call is staged, where the copy-in comes
// first.
bool touchesForeignSlice(const void* small, size_t small_bytes, const void* large, size_t slice_bytes, int W, int me) {
  if (!rangesOverlap(small, small_bytes, large, slice_bytes * (size_t)W)) return false;
  const uintptr_t s0 = (uintptr_t)small, own = (uintptr_t)large + (size_t)me * slice_bytes;
  return !(s0 >= own && s0 + small_bytes <= own + slice_bytes);
}

size_t roundUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Device-to-device copy on the compute queue (the library's own segment copy): no DMA-engine
// round trip for small messages, full copy bandwidth for large ones.
void copyAsync(void* dst, const void* src, size_t bytes, hipStream_t s) {
  if (!bytes) return;
  mccl_segment_t seg{src, dst, bytes};
  int rc = mccl_copy_segments(&seg, 1, s);
  TORCH_CHECK(rc == MCCL_OK, "ccl backend: copy-in failed: ", mccl_last_error());
}

}  // namespace

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
  P2PBox p2p[kMaxWorld];
};

struct Control {
  uint32_t magic;
  uint32_t world;
  RankSlot slot[1];  // world entries
};

static_assert(std::atomic<uint64_t>::is_always_lock_free, "barrier counters must be lock-free");

// ---------------------------------------------------------------------------------------------
// what a group shares with its Works
// ---------------------------------------------------------------------------------------------
hipEvent_t GroupShared::getEvent() {
  {
    std::lock_guard<std::mutex> lock(mutex);
    if (!free_events.empty()) {
      hipEvent_t e = free_events.back();
      free_events.pop_back();
      return e;
    }
  }
  hipEvent_t e = nullptr;
  HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  return e;
}

void GroupShared::putEvent(hipEvent_t e) {
  std::lock_guard<std::mutex> lock(mutex);
  free_events.push_back(e);
}

std::string GroupShared::failureMessage() {
  if (status && (status[0] != 0 || status[2] != 0) && !failed.load(std::memory_order_acquire)) {
    std::ostringstream os;
    if (status[0] != 0 && status[1] == MCCL_STATUS_UNMAPPED) {
      os << "ccl backend: rank " << (status[0] - 1) << " offered a tensor in an allocation that this rank has not mapped "
            "(standing offers out of step); the group cannot be used any more";
    } else if (status[0] != 0) {
      // epochs count four per collective: #(epoch / 4), wait (epoch % 4): 1 = inputs ready, 2 = between
      // the phases of a two-phase collective, 3 = all ranks done with this rank's buffers
      os << "ccl backend: timed out waiting for rank " << (status[0] - 1)
         << " on the device (cross-rank wait " << (status[1] & 3u) << " of collective #" << (status[1] >> 2)
         << ", modulo 2^30); the group cannot be used any more";
    } else {
      // the one-launch small allreduce counts its own launches, on the device (replays of a recorded
      // graph included, which the host's collective numbers do not see)
      os << "ccl backend: timed out waiting for rank " << (status[2] - 1)
         << " on the device (one-launch allreduce #" << status[3]
         << " of this group, counting those alone, modulo 2^32); the group cannot be used any more";
    }
    fail(os.str());
  }
  if (!failed.load(std::memory_order_acquire)) return std::string();
  std::lock_guard<std::mutex> lock(mutex);
  return failure;
}

void GroupShared::fail(const std::string& why) {
  std::lock_guard<std::mutex> lock(mutex);
  if (failure.empty()) failure = why;
  failed.store(true, std::memory_order_release);
}

GroupShared::~GroupShared() {
  for (hipEvent_t e : free_events) (void)hipEventDestroy(e);
  if (status) (void)hipHostFree((void*)status);
}

// ---------------------------------------------------------------------------------------------
// Work
// ---------------------------------------------------------------------------------------------
ProcessGroupCCL::WorkCCL::WorkCCL(int rank, c10d::OpType op, const char* title,
                                  std::vector<at::Tensor> inputs, std::vector<at::Tensor> outputs,
                                  bool blocking_wait)
    : c10d::Work(rank, op, title), start_(std::chrono::steady_clock::now()), blocking_wait_(blocking_wait),
      inputs_(std::move(inputs)), outputs_(std::move(outputs)) {}

ProcessGroupCCL::WorkCCL::~WorkCCL() {
  if (!end_) return;
  if (shared_) shared_->putEvent(end_);  // a recycled event is only ever re-recorded: safe while pending
  else (void)hipEventDestroy(end_);
}

bool ProcessGroupCCL::WorkCCL::isCompleted() {
  if (pending_polls_ != 0) {
    if (pending_polls_ > 0) --pending_polls_;
    return false;
  }
  if (captured_) return true;  // recorded, not enqueued: nothing of this Work is outstanding
  if (end_) return hipEventQuery(end_) == hipSuccess;
  if (!stream_set_) return true;
  // No event was recorded for this collective (it ran on the caller's stream; with several
  // processes on one GPU an event record costs more than the collective's kernel): the stream
  // having drained is the conservative answer.
  const hipError_t e = hipStreamQuery(stream_);
  if (e == hipErrorNotReady) return false;
  (void)hipGetLastError();
  return true;  // drained, or the stream no longer exists
}

bool ProcessGroupCCL::WorkCCL::isSuccess() const {
  return !shared_ || shared_->failureMessage().empty();
}

std::exception_ptr ProcessGroupCCL::WorkCCL::exception() const {
  if (!shared_) return nullptr;
  const std::string why = shared_->failureMessage();
  if (why.empty()) return nullptr;
  return std::make_exception_ptr(std::runtime_error(why));
}

// The caller's current stream waits for the collective: through its end event; or, when none was
// recorded, not at all on the stream the collective ran on, and through an event recorded now (at
// that stream's current end, which is later than the collective's: conservative) on any other.
void ProcessGroupCCL::WorkCCL::orderCurrentStreamAfter() {
  hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device_).stream();
  if (end_) {
    HIP_CHECK(hipStreamWaitEvent(cur, end_, 0));
  } else if (stream_set_ && cur != stream_) {
    end_ = shared_ ? shared_->getEvent() : nullptr;
    if (!end_) HIP_CHECK(hipEventCreateWithFlags(&end_, hipEventDisableTiming));
    HIP_CHECK(hipEventRecord(end_, stream_));
    HIP_CHECK(hipStreamWaitEvent(cur, end_, 0));
  }
}

void ProcessGroupCCL::WorkCCL::waitInternal(std::chrono::milliseconds timeout) {
  if (blocking_wait_) {
    // synchronizeInternal of the reference (src/utils.h:295-319): poll until done or timed out
    const std::chrono::milliseconds limit = timeout == kNoTimeout ? op_timeout_ : timeout;
    unsigned spins = 0;
    while (!isCompleted()) {
      if (limit.count() > 0) {
        const auto ran = std::chrono::duration_cast<std::chrono::milliseconds>(std::chrono::steady_clock::now() - start_);
        TORCH_CHECK(ran < limit, "[Rank ", rank_, "] Caught collective operation timeout:  ran for ", ran.count(),
                    " milliseconds before timing out.");
      }
      // yield for the first few milliseconds (a sleeping thread wakes up tens of microseconds late,
      // which would show up as skew between the ranks at their next collective), sleep afterwards
      if (++spins > 20000) std::this_thread::sleep_for(std::chrono::microseconds(50));
      else if (spins > 100) sched_yield();
    }
  } else {
    // stream-ordered (the queue barrier of src/gpu/dpcpp_ccl.cpp:440-457)
    c10::DeviceGuard guard(c10::Device(at::kCUDA, (c10::DeviceIndex)device_));
    orderCurrentStreamAfter();
  }
  if (shared_) {
    const std::string why = shared_->failureMessage();
    TORCH_CHECK(why.empty(), why);
  }
}

void ProcessGroupCCL::WorkCCL::synchronize() { waitInternal(kNoTimeout); }

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::pendingWork(int rank, int polls, std::chrono::milliseconds op_timeout) {
  auto work = c10::make_intrusive<WorkCCL>(rank, c10d::OpType::UNKNOWN, "pending", std::vector<at::Tensor>{},
                                           std::vector<at::Tensor>{}, /*blocking_wait=*/true);
  work->pending_polls_ = polls;
  work->op_timeout_ = op_timeout;
  return work;
}

bool ProcessGroupCCL::WorkCCL::wait(std::chrono::milliseconds timeout) {
  waitInternal(timeout);
  return true;
}

std::vector<at::Tensor> ProcessGroupCCL::WorkCCL::result() { return outputs_; }

c10::intrusive_ptr<c10::ivalue::Future> ProcessGroupCCL::WorkCCL::getFuture() {
  if (!future_) {
    std::vector<c10::Device> devs;
    if (end_ || stream_set_) devs.emplace_back(at::kCUDA, (c10::DeviceIndex)device_);
    future_ = c10::make_intrusive<at::ivalue::Future>(c10::ListType::create(c10::TensorType::get()), devs);
    if (auto err = exception()) {  // finishAsyncWorkCCLError of the reference: the future carries the error
      future_->setError(err);
      return future_;
    }
    if (end_ || stream_set_) {
      c10::DeviceGuard guard(c10::Device(at::kCUDA, (c10::DeviceIndex)device_));
      orderCurrentStreamAfter();
    }
    future_->markCompleted(at::IValue(outputs_));  // records the current stream: ordered after the collective
  }
  return future_;
}

// ---------------------------------------------------------------------------------------------
// construction, rendezvous, staging
// ---------------------------------------------------------------------------------------------
namespace {

// Groups that have exported allocations to their peers, for the allocator's segment-free
// notification.  The tracker is attached once per process and never detached (torch offers no way
// to), so it only touches groups that are still registered here.
std::mutex g_registry_mutex;
std::vector<ProcessGroupCCL*> g_registry;
std::once_flag g_tracker_once;

void attachSegmentTracker() {
  std::call_once(g_tracker_once, [] {
    c10::hip::HIPCachingAllocator::attachAllocatorTraceTracker([](const c10::hip::HIPCachingAllocator::TraceEntry& te) {
      if (te.action_ != c10::hip::HIPCachingAllocator::TraceEntry::SEGMENT_FREE &&
          te.action_ != c10::hip::HIPCachingAllocator::TraceEntry::SEGMENT_UNMAP)
        return;
      // called under the allocator's lock: flags only, no HIP and no torch calls
      std::lock_guard<std::mutex> lock(g_registry_mutex);
      for (ProcessGroupCCL* pg : g_registry) pg->segmentFreed((uint64_t)te.addr_);
    });
  });
}

}  // namespace

ProcessGroupCCL::ProcessGroupCCL(const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
                                 std::chrono::milliseconds timeout)
    : c10d::Backend(rank, size), store_(store), timeout_(timeout) {
  TORCH_CHECK(size >= 1 && size <= kMaxWorld, "ccl backend: world size ", size, " outside [1, ", kMaxWorld, "]");
  checkRank(rank, size);
  // same switches as the reference (src/ProcessGroupCCL.hpp:96-102, src/env.cpp:11-33)
  same_stream_ = envFlag("CCL_SAME_STREAM", false);
  blocking_wait_ = envFlag("CCL_BLOCKING_WAIT", false);
  verbose_ = envFlag("ONECCL_BINDINGS_FOR_PYTORCH_ENV_VERBOSE", false);
  profile_ = envFlag("MCCL_PG_PROFILE", false);
  if (const char* v = std::getenv("MCCL_PG_SYNC")) {
    want_device_sync_ = std::string(v) != "host";
    waits_in_data_kernels_ = std::string(v) == "kernel";
  }
  zero_copy_ = envFlag("MCCL_PG_ZERO_COPY", true);
  comm_stream_for_large_ = envFlag("MCCL_PG_COMM_STREAM", false);
  if (const char* v = std::getenv("MCCL_PG_ONE_LAUNCH_MAX_BYTES")) {
    one_launch_max_ = (size_t)std::atoll(v);
    one_launch_max_forced_ = true;  // binds the collectives that are one launch at every size, too
  }
  if (const char* v = std::getenv("MCCL_PG_COMPACT_MAX_BYTES")) compact_max_ = (size_t)std::atoll(v);
  allgather_push_ = envFlag("MCCL_PG_ALLGATHER_PUSH", true);
  standing_offers_ = envFlag("MCCL_PG_STANDING_OFFERS", true);
  if (const char* v = std::getenv("MCCL_PG_STANDING_MAX_BYTES")) standing_max_ = (size_t)std::atoll(v);
  work_only_ = envFlag("TORCH_CCL_WORK_ONLY", false) || envFlag("MCCL_PG_WORK_ONLY", false);
  sync_only_ = envFlag("TORCH_CCL_SYNC_ONLY", false) || envFlag("MCCL_PG_SYNC_ONLY", false);
  disable_allreduce_ = envFlag("TORCH_CCL_DISABLE_ALLREDUCE", false) || envFlag("MCCL_PG_DISABLE_ALLREDUCE", false);
  TORCH_CHECK(!(work_only_ && sync_only_), "ccl backend: TORCH_CCL_WORK_ONLY and TORCH_CCL_SYNC_ONLY exclude each other");
  fused_mode_ = work_only_ ? MCCL_FUSED_WORK_ONLY : sync_only_ ? MCCL_FUSED_SYNC_ONLY : 0u;
  if (work_only_ || sync_only_ || disable_allreduce_)
    TORCH_WARN_ONCE("ccl backend: a bisecting switch is set (", work_only_ ? "work only: no cross-rank waits" : sync_only_ ? "sync only: no data is moved" : "allreduce disabled",
                    "); collectives between rank processes do NOT produce results, this is for timing only");
  if (const char* v = std::getenv("MCCL_PG_WAITING_COMPUTE_UNITS")) waiting_cus_ = (unsigned)std::max(1, std::atoi(v));
  // The staging window can be shrunk (never enlarged) so that tests reach every windowed path
  // with small tensors.
  stage_max_ = kStageMaxDefault;
  if (const char* v = std::getenv("MCCL_STAGE_WINDOW_BYTES")) {
    const long long b = std::atoll(v);
    if (b >= 4096 && (size_t)b < kStageMaxDefault) stage_max_ = (size_t)b & ~(size_t)4095;
  }
  shared_ = std::make_shared<GroupShared>();
}

c10::intrusive_ptr<c10d::Backend> ProcessGroupCCL::create(const c10::intrusive_ptr<c10d::Store>& store,
                                                          int rank, int size,
                                                          std::chrono::milliseconds timeout) {
  return c10::make_intrusive<ProcessGroupCCL>(store, rank, size, timeout);
}

ProcessGroupCCL::~ProcessGroupCCL() {
  {
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    g_registry.erase(std::remove(g_registry.begin(), g_registry.end(), this), g_registry.end());
  }
  if (profile_ && !phase_us_[0].empty()) {
    // medians: the first calls of a group pay for allocations and peer mappings
    std::ostringstream os;
    os << "ccl backend rank " << rank_ << ": " << phase_us_[0].size() << " collectives with a payload, median us per phase:";
    const char* names[4] = {" copy-in enqueue ", device_sync_ ? ", host rendezvous " : ", stream synchronise ",
                            device_sync_ ? ", barrier enqueue " : ", host barrier ", ", kernel enqueue "};
    for (int i = 0; i < 4; ++i) {
      auto& v = phase_us_[i];
      if (v.empty()) continue;
      std::nth_element(v.begin(), v.begin() + (long)(v.size() / 2), v.end());
      os << names[i] << v[v.size() / 2];
    }
    std::cerr << os.str() << std::endl;
  }
  if (!initialised_) return;
  // Peers may still be reading this rank's buffers in their last kernels: wait for our own
  // streams, then give the others a bounded chance to catch up.  A peer that is already gone has
  // finished its kernels, so a timeout here is harmless.
  (void)hipSetDevice(device_);
  if (comm_stream_) (void)hipStreamSynchronize(comm_stream_);
  if (tail_pending_) (void)hipStreamSynchronize(tail_stream_);
  // Leaving never advances the barrier epoch (a rank that leaves early must not satisfy its
  // peers' next barrier); it raises a flag instead.
  ctl_->slot[rank_].departed.store(1, std::memory_order_release);
  if (device_sync_ && size_ > 1) {
    // The departure barrier: its own flag word, so that it can never be mistaken for a collective.
    // Once it has passed (or its 2 s are over) every peer that leaves too has drained its stream.
    if (shared_->failureMessage().empty()) {
      (void)mccl_rank_barrier(final_flags_.data(), size_, rank_, 1, 2000000, nullptr, comm_stream_);
      (void)hipStreamSynchronize(comm_stream_);
    }
  } else {
    // A peer is done with this rank's buffers once it has left too or has arrived at a later collective.
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(2000);
    for (int r = 0; r < size_; ++r) {
      if (r == rank_) continue;
      while (!ctl_->slot[r].departed.load(std::memory_order_acquire) &&
             ctl_->slot[r].arrive.load(std::memory_order_acquire) <= barrier_epoch_ &&
             std::chrono::steady_clock::now() < deadline)
        sched_yield();
    }
  }
  // Messages this rank has sent and nobody has copied out yet live in its staging buffers: give
  // the receivers a bounded time, then flag the failure so that a late receiver raises instead of
  // reading freed memory.
  {
    const auto p2p_deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(10000);
    for (int d = 0; d < size_; ++d) {
      P2PBox& box = ctl_->slot[rank_].p2p[d];
      while (box.consumed.load(std::memory_order_acquire) < box.posted.load(std::memory_order_relaxed)) {
        if (ctl_->slot[d].departed.load(std::memory_order_acquire) || ctl_->slot[d].failed.load(std::memory_order_acquire) ||
            std::chrono::steady_clock::now() > p2p_deadline) {
          ctl_->slot[rank_].failed.store(1, std::memory_order_release);
          break;
        }
        sched_yield();
      }
    }
  }
  (void)hipDeviceSynchronize();
  closeImports();
  for (auto& pr : p2p_recv_)
    for (int i = 0; i < kP2PRing; ++i)
      if (pr.ipc[i] && pr.base[i]) (void)hipIpcCloseMemHandle(pr.base[i]);
  for (auto& ps : p2p_send_)
    for (int i = 0; i < kP2PRing; ++i)
      if (ps.base[i]) (void)hipFree(ps.base[i]);
  for (auto& pm : peers_)
    for (int s = 0; s < 2; ++s)
      if (pm.ipc[s] && pm.base[s]) (void)hipIpcCloseMemHandle(pm.base[s]);
  for (int r = 0; r < (int)peer_arena_.size(); ++r)
    if (r != rank_ && peer_arena_[(size_t)r]) (void)hipIpcCloseMemHandle(peer_arena_[(size_t)r]);
  for (int s = 0; s < 2; ++s)
    if (stage_[s].base) (void)hipFree(stage_[s].base);
  for (void* p : retired_) (void)hipFree(p);
  if (arena_) (void)hipFree(arena_);
  if (fork_event_) (void)hipEventDestroy(fork_event_);
  if (tail_event_) (void)hipEventDestroy(tail_event_);
  if (ctl_) munmap(ctl_, ctl_bytes_);
}

void ProcessGroupCCL::ensureInit(int device) {
  if (initialised_) {
    TORCH_CHECK(device == device_, "ccl backend: a process group is bound to one device (cuda:", device_,
                "), got a tensor on cuda:", device);
    return;
  }
  device_ = device;
  shared_->device = device;
  HIP_CHECK(hipSetDevice(device_));
  comm_stream_ = c10::hip::getStreamFromPoolMasqueradingAsCUDA(false, (c10::DeviceIndex)device_).stream();
  HIP_CHECK(hipEventCreateWithFlags(&fork_event_, hipEventDisableTiming));
  HIP_CHECK(hipEventCreateWithFlags(&tail_event_, hipEventDisableTiming));

  // Groups are created in the same order on every rank, so a per-rank counter in the store
  // yields the same id everywhere.
  const int64_t gid = store_->add("mccl/gid/" + std::to_string(rank_), 1);
  const std::string key = "mccl/shm/" + std::to_string(gid);
  ctl_bytes_ = roundUp(sizeof(Control) + sizeof(RankSlot) * (size_t)size_, 4096);
  int fd = -1;
  if (rank_ == 0) {
    const auto now = std::chrono::steady_clock::now().time_since_epoch().count();
    shm_name_ = "/mccl-" + std::to_string((long)getpid()) + "-" + std::to_string(gid) + "-" +
                std::to_string((long long)now);
    fd = shm_open(shm_name_.c_str(), O_CREAT | O_EXCL | O_RDWR, 0600);
    TORCH_CHECK(fd >= 0, "ccl backend: shm_open(", shm_name_, ") failed: ", std::strerror(errno));
    TORCH_CHECK(ftruncate(fd, (off_t)ctl_bytes_) == 0, "ccl backend: ftruncate failed: ", std::strerror(errno));
  } else {
    auto raw = store_->get(key);  // blocks until rank 0 has published the name
    shm_name_.assign(raw.begin(), raw.end());
    fd = shm_open(shm_name_.c_str(), O_RDWR, 0600);
    TORCH_CHECK(fd >= 0, "ccl backend: shm_open(", shm_name_, ") failed: ", std::strerror(errno));
  }
  void* m = mmap(nullptr, ctl_bytes_, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  TORCH_CHECK(m != MAP_FAILED, "ccl backend: mmap of the control block failed: ", std::strerror(errno));
  ctl_ = static_cast<Control*>(m);
  if (rank_ == 0) {
    ctl_->magic = kMagic;  // fresh shared memory is zero-filled
    ctl_->world = (uint32_t)size_;
    store_->set(key, std::vector<uint8_t>(shm_name_.begin(), shm_name_.end()));
  }
  RankSlot& me = ctl_->slot[rank_];
  me.pid = (int64_t)getpid();
  peers_.assign((size_t)size_, PeerMap{});
  p2p_send_.assign((size_t)size_, P2PSend{});
  p2p_recv_.assign((size_t)size_, P2PRecv{});
  exports_.assign((size_t)kMaxExports, Export{});
  imports_.assign((size_t)size_, std::vector<Import>((size_t)kMaxExports));
  initialised_ = true;
  for (int s = 0; s < 2; ++s) ensureStage(s, std::min(kStageMin, stage_max_));

  // The arena: flag words and the buffers of the one-launch allreduce, zeroed, published before the
  // start-up barrier and mapped by everybody right after it.
  if (size_ > 1) {
    HIP_CHECK(hipMalloc(&arena_, kArenaBytes));
    HIP_CHECK(hipMemset(arena_, 0, kArenaBytes));
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipIpcGetMemHandle(&me.arena_handle, arena_));
    me.arena_ptr = (uint64_t)(uintptr_t)arena_;
    void* host_status = nullptr;
    HIP_CHECK(hipHostMalloc(&host_status, 64, hipHostMallocMapped));
    std::memset(host_status, 0, 64);
    shared_->status = static_cast<volatile uint32_t*>(host_status);
    HIP_CHECK(hipHostGetDevicePointer(&status_dev_, host_status, 0));
  }

  hostBarrier(/*start_up=*/true);
  TORCH_CHECK(ctl_->magic == kMagic && ctl_->world == (uint32_t)size_,
              "ccl backend: control block mismatch (ranks disagree on the world size)");
  if (rank_ == 0) shm_unlink(shm_name_.c_str());  // every rank holds a mapping now

  // Device-side waits need ranks whose kernels can never queue up behind each other: processes of
  // their own.  Every rank sees the same pid table, so the decision is the same everywhere (the
  // environment switch has to agree across ranks like any other setting of the group).
  bool distinct = true;
  for (int a = 0; a < size_; ++a)
    for (int b = a + 1; b < size_; ++b)
      if (ctl_->slot[a].pid == ctl_->slot[b].pid) distinct = false;
  device_sync_ = size_ > 1 && distinct && want_device_sync_;
  distinct_pids_ = size_ > 1 && distinct;
  if (device_sync_ && rank_ == 0) {
    // A kernel that waits for other ranks only makes progress while the hardware queues of all rank
    // processes are mapped at once.  A process owns up to GPU_MAX_HW_QUEUES of them (4 unless set),
    // one per group of streams it uses; with 8 rank processes that use three or more streams each
    // the GPU maps fewer queues than exist and time-slices them, and a collective then takes a
    // scheduling quantum (measured: 11 ms instead of 0.1 ms).  One or two queues per process are safe.
    const char* q = std::getenv("GPU_MAX_HW_QUEUES");
    const long queues = q ? std::atol(q) : 4;
    if (queues * size_ > 16)
      TORCH_WARN_ONCE("ccl backend: ", size_, " rank processes share one GPU and wait for each other on the device; if the "
                      "ranks use more than two streams each, set GPU_MAX_HW_QUEUES=2 (or 1) in their environment, or "
                      "MCCL_PG_SYNC=host: with more hardware queues than the GPU maps at once a collective costs a "
                      "scheduling quantum (about 10 ms)");
  }
  if (size_ > 1) {
    peer_arena_.assign((size_t)size_, nullptr);
    bar_flags_.assign((size_t)size_, nullptr);
    final_flags_.assign((size_t)size_, nullptr);
    for (int sl = 0; sl < 2; ++sl) {
      fused_stage_[sl].assign((size_t)size_, nullptr);
      fused_flags_[sl].assign((size_t)size_, nullptr);
    }
    done_counter_ = static_cast<char*>(arena_) + kArenaDoneCountOff;
    fused_state_ = static_cast<char*>(arena_) + kArenaFusedStateOff;
    import_table_ = reinterpret_cast<mccl_import_table_t*>(static_cast<char*>(arena_) + kArenaImportTableOff);
    resolved_ = static_cast<char*>(arena_) + kArenaResolvedOff;
    for (int sl = 0; sl < 2; ++sl) offer_slots_[sl].assign((size_t)size_, nullptr);
    for (int r = 0; r < size_; ++r) {
      char* base = nullptr;
      if (r == rank_) {
        base = static_cast<char*>(arena_);
      } else if (ctl_->slot[r].pid == (int64_t)getpid()) {
        base = (char*)(uintptr_t)ctl_->slot[r].arena_ptr;
      } else {
        void* p = nullptr;
        HIP_CHECK(hipIpcOpenMemHandle(&p, ctl_->slot[r].arena_handle, hipIpcMemLazyEnablePeerAccess));
        base = static_cast<char*>(p);
      }
      peer_arena_[(size_t)r] = (ctl_->slot[r].pid == (int64_t)getpid()) ? nullptr : base;  // what gets closed
      bar_flags_[(size_t)r] = base + kArenaBarOff;
      final_flags_[(size_t)r] = base + kArenaFinalOff;
      for (int sl = 0; sl < 2; ++sl) {
        offer_slots_[sl][(size_t)r] = base + kArenaOfferOff + (size_t)sl * kArenaOfferStride;
        fused_flags_[sl][(size_t)r] = base + kArenaFusedFlagsOff + (size_t)sl * kArenaFusedFlagsStride;
        fused_stage_[sl][(size_t)r] = base + kArenaFusedStageOff + (size_t)sl * kArenaFusedStageStride + stageOffset(r);
      }
    }
    peer_arena_[(size_t)rank_] = nullptr;
    // nobody starts a collective before everybody has mapped everything
    hostBarrier(/*start_up=*/true);
  }
  // (also with MCCL_PG_SYNC=host: rank processes offer their tensors for the in-place allreduce there,
  // and a freed and re-issued segment must retire its export in that mode, too)
  if (distinct_pids_ && zero_copy_) {
    attachSegmentTracker();
    std::lock_guard<std::mutex> lock(g_registry_mutex);
    g_registry.push_back(this);
  }
}

void* ProcessGroupCCL::ensureStage(int slot, size_t bytes) {
  Stage& st = stage_[slot];
  if (bytes <= st.capacity) return st.ptr;
  TORCH_CHECK(bytes <= stage_max_, "ccl backend: staging request of ", bytes, " bytes exceeds the window");
  size_t cap = kStageMin;
  while (cap < bytes) cap <<= 1;
  void* base = nullptr;
  HIP_CHECK(hipMalloc(&base, cap + kStageStagger * kStageStaggerSlots));
  if (st.base) retired_.push_back(st.base);  // a peer may still hold a mapping: freed with the group
  st.base = base;
  st.ptr = static_cast<char*>(base) + stageOffset(rank_);
  st.capacity = cap;
  if (size_ > 1) HIP_CHECK(hipIpcGetMemHandle(&st.handle, base));
  st.gen += 1;
  return st.ptr;
}

// Copies what the peers need to know of this rank's staging buffer `slot` into the record of the
// current collective.
void ProcessGroupCCL::publishStage(int slot, int pub) {
  RankSlot::Published& rec = ctl_->slot[rank_].pub[pub];
  rec.stage_gen = stage_[slot].gen;
  rec.stage_ptr = (uint64_t)(uintptr_t)stage_[slot].ptr;
  rec.stage_handle = stage_[slot].handle;
}

void ProcessGroupCCL::quiesce() {
  if (tail_pending_) HIP_CHECK(hipStreamSynchronize(tail_stream_));
  tail_pending_ = false;
}

const void* ProcessGroupCCL::peerStage(int peer, int slot, int pub) {
  if (peer == rank_) return stage_[slot].ptr;
  const RankSlot::Published& rec = ctl_->slot[peer].pub[pub];
  const RankSlot& rs = ctl_->slot[peer];
  PeerMap& pm = peers_[(size_t)peer];
  if (pm.gen[slot] != rec.stage_gen) {
    if (pm.ipc[slot] && pm.base[slot]) {
      quiesce();  // earlier kernels of this rank may still read through the old mapping
      (void)hipIpcCloseMemHandle(pm.base[slot]);
    }
    pm.ptr[slot] = nullptr;
    pm.base[slot] = nullptr;
    pm.ipc[slot] = false;
    if (rs.pid == (int64_t)getpid()) {
      pm.ptr[slot] = (void*)(uintptr_t)rec.stage_ptr;  // a thread of this process: same address space
    } else {
      void* p = nullptr;
      HIP_CHECK(hipIpcOpenMemHandle(&p, rec.stage_handle, hipIpcMemLazyEnablePeerAccess));
      pm.base[slot] = p;
      pm.ptr[slot] = static_cast<char*>(p) + stageOffset(peer);
      pm.ipc[slot] = true;
    }
    pm.gen[slot] = rec.stage_gen;
    if (peer < MCCL_OFFER_RANKS) noteImport((uint32_t)peer, MCCL_OFFER_STAGED, (uint32_t)slot, (uint64_t)(uintptr_t)pm.ptr[slot], 0);
  }
  return pm.ptr[slot];
}

// ---------------------------------------------------------------------------------------------
// zero-copy: exporting the caller's allocation, importing the peers'
// ---------------------------------------------------------------------------------------------
void ProcessGroupCCL::segmentFreed(uint64_t base) {
  // g_registry_mutex is held; the allocator's lock too.  The entry stays in the table (its handle
  // is dead) until it is evicted; the generation tells the peers to drop their mapping.
  if (!ctl_) return;
  for (int i = 0; i < kMaxExports; ++i) {
    if (exports_[(size_t)i].valid && exports_[(size_t)i].base == base) {
      exports_[(size_t)i].valid = false;
      ctl_->slot[rank_].exports[i].live.store(0, std::memory_order_release);
      ctl_->slot[rank_].exports[i].gen.fetch_add(1, std::memory_order_release);
    }
  }
}

// Publishes the allocation that holds [ptr, ptr + bytes) and returns its entry in this rank's
// export table (or -1 when it cannot be shared: not an allocation of torch's caching allocator,
// 2 GiB or more, or refused by the runtime).  *offset = where ptr lies inside it.
int ProcessGroupCCL::exportRange(const void* ptr, size_t bytes, uint64_t* offset) {
  if (!bytes) return kEmptyShare;  // nothing to read: trivially shareable
  if (!zero_copy_ || !ptr) return -1;
  // Only allocations whose release this group gets to hear of (the allocator's segment-free
  // notification) are shared: a cached mapping of anything else could go stale unnoticed.
  void* base = nullptr;
  size_t size = 0;
  try {
    base = c10::hip::HIPCachingAllocator::getBaseAllocation(const_cast<void*>(ptr), &size);
  } catch (const c10::Error&) {
    return -1;
  }
  if (!base || size >= kShareMaxAllocation) return -1;
  const uint64_t off = (uint64_t)((const char*)ptr - (const char*)base);
  if (off + bytes > size) return -1;
  RankSlot& me = ctl_->slot[rank_];
  std::lock_guard<std::mutex> lock(g_registry_mutex);
  int idx = -1;
  for (int i = 0; i < kMaxExports; ++i)
    if (exports_[(size_t)i].valid && exports_[(size_t)i].base == (uint64_t)(uintptr_t)base &&
        exports_[(size_t)i].size == size) { idx = i; break; }
  if (idx < 0) {
    hipIpcMemHandle_t h;
    if (hipIpcGetMemHandle(&h, base) != hipSuccess) {
      (void)hipGetLastError();  // e.g. memory of an expandable segment: not shareable
      return -1;
    }
    // An entry that a standing offer has named may only change once every peer has entered a later
    // collective than the offer's: a peer reads this table when it enters a collective, and the
    // kernels of that collective resolve the offer against what it read.
    uint64_t entered = ~0ull;
    for (int r = 0; r < size_; ++r)
      if (r != rank_) entered = std::min(entered, ctl_->slot[r].entered.load(std::memory_order_acquire));
    auto settled = [&](int i) { return last_offer_seq_[i] == 0 || entered >= last_offer_seq_[i] + 1; };
    for (int i = 0; i < kMaxExports && idx < 0; ++i)
      if (!exports_[(size_t)i].valid && settled(i)) idx = i;  // a never-used entry, or one whose allocation is gone
    for (int tries = 0; idx < 0 && tries < kMaxExports; ++tries) {
      // evict round robin, but never an entry of the last two offers: a slow peer may still be
      // opening it
      const int victim = export_clock_;
      export_clock_ = (export_clock_ + 1) % kMaxExports;
      if (victim != recent_export_[0] && victim != recent_export_[1] && settled(victim)) idx = victim;
    }
    if (idx < 0) return -1;  // every entry is still spoken for: this tensor is staged
    me.exports[idx].live.store(0, std::memory_order_release);
    const uint64_t gen = me.exports[idx].gen.fetch_add(1, std::memory_order_acq_rel) + 1;
    me.exports[idx].base = (uint64_t)(uintptr_t)base;
    me.exports[idx].size = size;
    me.exports[idx].handle = h;
    me.exports[idx].live.store(gen, std::memory_order_release);
    last_offer_seq_[idx] = 0;
    exports_[(size_t)idx] = Export{(uint64_t)(uintptr_t)base, size, true};
  }
  *offset = off;
  recent_export_[1] = recent_export_[0];
  recent_export_[0] = idx;
  return idx;
}

// The range rank `peer` offered in record `pub`, in this process's address space.  Call after the
// rendezvous.
const void* ProcessGroupCCL::importRange(int peer, int pub) {
  const RankSlot& rs = ctl_->slot[peer];
  const RankSlot::Published& rec = rs.pub[pub];
  const int idx = (int)rec.share_entry;
  if (idx == kEmptyShare) return nullptr;
  TORCH_CHECK(idx >= 0 && idx < kMaxExports, "ccl backend: rank ", peer, " published no shareable range");
  Import& im = imports_[(size_t)peer][(size_t)idx];
  const uint64_t gen = rec.share_gen;
  if (im.gen != gen || !im.base) {
    if (im.base) {
      quiesce();  // earlier kernels of this rank may still read through the old mapping
      (void)hipIpcCloseMemHandle(im.base);
      im.base = nullptr;
    }
    void* p = nullptr;
    HIP_CHECK(hipIpcOpenMemHandle(&p, rs.exports[idx].handle, hipIpcMemLazyEnablePeerAccess));
    im.base = p;
    im.gen = gen;
    if (peer < MCCL_OFFER_RANKS && size_ <= MCCL_OFFER_RANKS) {  // the standing offers go by the same mappings
      noteImport((uint32_t)peer, (uint32_t)idx, 0, (uint64_t)(uintptr_t)p, gen);
      seen_live_[peer][idx] = gen;
      acknowledge(peer, idx, gen, seq_ - 1);  // (run() has counted this collective already)
    }
  }
  return static_cast<const char*>(im.base) + rec.share_off;
}

// ---------------------------------------------------------------------------------------------
// standing offers: collectives between rank processes that only enqueue
// ---------------------------------------------------------------------------------------------
// The reference exchanges the handles of its buffers once (src/gpu/dpcpp_ccl.cpp:105-121); after
// that an allreduce is a pure enqueue.  Here the buffers are the callers' tensors, so what is
// exchanged once is the ALLOCATION a tensor lives in -- a rank announces it in its export table,
// every peer maps it when it next enters a collective and says so (acked) -- and what changes from
// call to call, which allocation and where in it, travels on the device: the barrier kernel of the
// collective publishes this rank's offer and resolves the peers' against this rank's table of
// mappings (mccl_rank_barrier_offers).  No host thread waits for another: a rank whose allocation
// the peers have not all mapped yet (or that cannot be shared at all) copies its tensor into its
// staging buffer, which every peer has mapped since the group last grew it, and offers that.

// A mapping of this rank changed: the device table learns of it in stream order, before the next
// barrier that resolves offers (the values travel in the launch).
void ProcessGroupCCL::noteImport(uint32_t rank, uint32_t entry, uint32_t slot, uint64_t base, uint64_t gen) {
  for (auto& u : table_updates_)
    if (u.rank == rank && u.entry == entry && (entry != MCCL_OFFER_STAGED || u.slot == slot)) {
      u.base = base;
      u.generation = gen;
      return;
    }
  mccl_import_update_t u{};
  u.rank = rank;
  u.entry = entry;
  u.slot = slot;
  u.base = base;
  u.generation = gen;
  table_updates_.push_back(u);
}

void ProcessGroupCCL::flushImportTable(hipStream_t s) {
  for (size_t at = 0; at < table_updates_.size(); at += MCCL_IMPORT_UPDATES) {
    const int n = (int)std::min<size_t>(MCCL_IMPORT_UPDATES, table_updates_.size() - at);
    MCCL_CHECK(mccl_import_table_update(import_table_, table_updates_.data() + at, n, s));
  }
  table_updates_.clear();
}

void ProcessGroupCCL::acknowledge(int owner, int entry, uint64_t gen, uint64_t from_seq) {
  RankSlot::Ack& a = ctl_->slot[rank_].acked[owner][entry];
  a.gen.store(0, std::memory_order_release);
  a.from_seq.store(from_seq, std::memory_order_release);
  a.gen.store(gen, std::memory_order_release);
}

// Maps what the peers have announced since this rank last looked, drops what they have retired,
// and acknowledges: the kernels of collective `seq` and later see these mappings.  Nobody is waited
// for; an entry that changes while it is read is left for the next look.
void ProcessGroupCCL::scanPeerExports(uint64_t seq) {
  for (int r = 0; r < size_; ++r) {
    if (r == rank_) continue;
    RankSlot& rs = ctl_->slot[r];
    for (int e = 0; e < kMaxExports; ++e) {
      const uint64_t live = rs.exports[e].live.load(std::memory_order_acquire);
      if (live == seen_live_[r][e]) continue;
      Import& im = imports_[(size_t)r][(size_t)e];
      if (im.base && im.gen != live) {
        quiesce();  // earlier kernels of this rank may still read through the old mapping
        (void)hipIpcCloseMemHandle(im.base);
        im = Import{};
        noteImport((uint32_t)r, (uint32_t)e, 0, 0, 0);
      }
      if (live == 0) {
        seen_live_[r][e] = 0;
        acknowledge(r, e, 0, seq);
        continue;
      }
      const hipIpcMemHandle_t handle = rs.exports[e].handle;
      if (rs.exports[e].live.load(std::memory_order_acquire) != live) continue;  // being rewritten: next time
      if (!im.base) {
        void* p = nullptr;
        if (hipIpcOpenMemHandle(&p, handle, hipIpcMemLazyEnablePeerAccess) != hipSuccess) {
          (void)hipGetLastError();
          seen_live_[r][e] = live;  // cannot be mapped here: never acknowledged, its owner keeps staging
          continue;
        }
        im.base = p;
        im.gen = live;
        noteImport((uint32_t)r, (uint32_t)e, 0, (uint64_t)(uintptr_t)p, live);
      }
      seen_live_[r][e] = live;
      acknowledge(r, e, live, seq);
    }
  }
}

// Have all peers mapped this rank's export entry at this generation, for collectives from `seq` on?
bool ProcessGroupCCL::allAcknowledged(int entry, uint64_t gen, uint64_t seq) const {
  for (int r = 0; r < size_; ++r) {
    if (r == rank_) continue;
    const RankSlot::Ack& a = ctl_->slot[r].acked[rank_][entry];
    if (a.gen.load(std::memory_order_acquire) != gen) return false;
    const uint64_t from = a.from_seq.load(std::memory_order_acquire);
    if (a.gen.load(std::memory_order_acquire) != gen || from > seq) return false;
  }
  return true;
}

// Staging buffers of both slots that hold `bytes` on every rank and that every peer has mapped:
// what a rank falls back to without asking anybody.  Grown when a message exceeds it, which every
// rank finds at the same collective (the sizes of an allreduce agree), in two rendezvous of the host
// threads -- the only ones this path ever has.
void ProcessGroupCCL::growStandingCapacity(size_t bytes) {
  size_t cap = kStageMin;
  while (cap < bytes) cap <<= 1;
  cap = std::min(cap, stage_max_);
  for (int sl = 0; sl < 2; ++sl) {
    ensureStage(sl, cap);
    const int pub = (int)(rendezvous_count_++ & 1);
    ctl_->slot[rank_].pub[pub].share_entry = -1;
    publishStage(sl, pub);
    hostBarrier();
    for (int r = 0; r < size_; ++r) (void)peerStage(r, sl, pub);
  }
  standing_capacity_ = cap;
}

bool ProcessGroupCCL::standingFits(const Plan& plan) const {
  return standing_offers_ && plan.standing.ok && device_sync_ && distinct_pids_ && zero_copy_ && !waits_in_data_kernels_ &&
         !work_only_ && !sync_only_ && size_ <= MCCL_OFFER_RANKS && plan.standing.bytes > 0 &&
         plan.standing.bytes <= std::min(stage_max_, standing_max_);
}

void ProcessGroupCCL::runStanding(Plan& plan, hipStream_t s, int slot, uint64_t seq) {
  const Plan::Standing& st = plan.standing;
  const size_t bytes = st.bytes;
  const uint64_t epoch = 4 * seq;
  uint64_t off = 0;
  // (small buffers live in the allocator's 2 MiB segments, many of them: announcing those would turn
  // the table of allocations over all the time, and copying them costs next to nothing)
  const int entry = (st.force_staged || bytes < kZeroCopyMinBytes) ? -1 : exportRange(st.buffer, bytes, &off);
  // A message larger than the staging every rank keeps mapped: the host threads meet (all at this
  // collective: the sizes agree) -- and since they do, they also look at what everybody has just
  // announced before anybody decides, so that the first collective of a new size already runs in place.
  const bool grow = bytes > standing_capacity_;
  if (grow) growStandingCapacity(bytes);
  scanPeerExports(seq);
  if (grow) hostBarrier();
  const uint64_t gen = entry >= 0 ? ctl_->slot[rank_].exports[entry].gen.load(std::memory_order_acquire) : 0;
  const bool in_place = entry >= 0 && allAcknowledged(entry, gen, seq);
  mccl_offer_t mine{};
  void* buffer = st.buffer;
  if (in_place) {
    mine.entry = (uint32_t)entry;
    mine.generation = gen;
    mine.offset = off;
    last_offer_seq_[entry] = seq + 1;  // in the units of `entered`: collective `seq` is under way at seq + 1
  } else {
    buffer = stage_[slot].ptr;
    if (st.copy_in) copyAsync(buffer, st.buffer, bytes, s);
    mine.entry = MCCL_OFFER_STAGED;
    mine.slot = (uint32_t)slot;
  }
  last_path_ = in_place ? "standing offers, peers read in place" : "standing offers, this rank staged";
  if (verbose_) {
    std::ostringstream os;
    os << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "#" << (seq + 1) << "] " << last_path_;
    std::cout << os.str() << std::endl;
  }
  ++enqueue_only_count_;
  flushImportTable(s);
  const uint64_t limit_us = (uint64_t)waitLimit(false).count() * 1000ull;
  mccl_xsync_t sync{};
  sync.words = bar_flags_.data();
  sync.n = size_;
  sync.rank = rank_;
  sync.done_epoch = epoch + 3;  // nobody's stream goes on before every rank is done with every rank's buffer
  sync.done_counter = done_counter_;
  sync.timeout_us = limit_us;
  sync.status = status_dev_;
  if ((double)bytes * st.compact_cost <= (double)compact_max_) {
    // little to move: ONE launch on this rank's share of half of the compute units, which carries the
    // offers itself (its opening wait is the barrier) -- with several processes on the GPU every
    // launch waits for its turn at the dispatcher, which costs more than the data at these sizes
    sync.ready_epoch = epoch + 1;
    sync.max_compute_units = std::max(1u, waiting_cus_ / (unsigned)size_);
    st.one_launch(!in_place, sync, mine, buffer, offer_slots_[slot].data(), import_table_, s);
  } else {
    MCCL_CHECK(mccl_rank_barrier_offers(bar_flags_.data(), size_, rank_, epoch + 1, limit_us, status_dev_, &mine, buffer,
                                        offer_slots_[slot].data(), import_table_, resolved_, s));
    st.behind_barrier(resolved_, !in_place, sync, s);
  }
  if (!in_place && st.copy_out) copyAsync(st.buffer, buffer, bytes, s);
}

void ProcessGroupCCL::closeImports() {
  for (auto& per_peer : imports_)
    for (auto& im : per_peer)
      if (im.base) {
        (void)hipIpcCloseMemHandle(im.base);
        im.base = nullptr;
      }
}

std::chrono::milliseconds ProcessGroupCCL::waitLimit(bool start_up) const {
  // Floor of 30 s under short user timeouts; MCCL_BARRIER_TIMEOUT_MS overrides it, e.g. to
  // exercise the failure path quickly.  The first barrier of a group waits for ranks that may
  // still be starting (a first import on a cold machine takes a minute): two minutes at least.
  std::chrono::milliseconds limit = std::max(timeout_, std::chrono::milliseconds(start_up ? 120000 : 30000));
  if (const char* v = start_up ? nullptr : std::getenv("MCCL_BARRIER_TIMEOUT_MS")) {
    const long ms = std::atol(v);
    if (ms > 0) limit = std::chrono::milliseconds(ms);
  }
  return limit;
}

// How long a kernel's own wait for the other ranks may last.  Normally the group's limit.  With
// MCCL_PG_SYNC=kernel whole grids wait, and a late rank whose other kernels find no room beside them
// only gets in once those waits have given up: twenty seconds there, not the minutes of the
// group's timeout (MCCL_PG_DEVICE_WAIT_MS or MCCL_BARRIER_TIMEOUT_MS say otherwise).
std::chrono::milliseconds ProcessGroupCCL::deviceWaitLimit() const {
  if (const char* v = std::getenv("MCCL_PG_DEVICE_WAIT_MS")) {
    const long ms = std::atol(v);
    if (ms > 0) return std::chrono::milliseconds(ms);
  }
  const std::chrono::milliseconds limit = waitLimit(false);
  if (waits_in_data_kernels_ && !std::getenv("MCCL_BARRIER_TIMEOUT_MS")) return std::min(limit, std::chrono::milliseconds(20000));
  return limit;
}

void ProcessGroupCCL::hostBarrier(bool start_up) {
  const uint64_t epoch = ++barrier_epoch_;
  ctl_->slot[rank_].arrive.store(epoch, std::memory_order_release);
  const auto deadline = std::chrono::steady_clock::now() + waitLimit(start_up);
  for (int r = 0; r < size_; ++r) {
    unsigned spins = 0;
    while (ctl_->slot[r].arrive.load(std::memory_order_acquire) < epoch) {
      if (ctl_->slot[r].failed.load(std::memory_order_acquire)) {
        shared_->fail(c10::str("ccl backend: rank ", r, " reported a failure; aborting the collective"));
        TORCH_CHECK(false, "ccl backend: rank ", r, " reported a failure; aborting the collective", lastEnqueued());
      }
      if (ctl_->slot[r].departed.load(std::memory_order_acquire)) {
        ctl_->slot[rank_].failed.store(1, std::memory_order_release);
        shared_->fail(c10::str("ccl backend: rank ", r, " left the group before collective #", seq_));
        TORCH_CHECK(false, "ccl backend: rank ", r, " left the group before collective #", seq_);
      }
      if (++spins < 2000) continue;
      // A peer may be late because it is still sending to this rank and has run out of send
      // buffers: take in what has arrived for the receives this rank has posted.
      if (!start_up)
        for (int src = 0; src < size_; ++src)
          if (!p2p_recv_[(size_t)src].pending.empty()) progressRecvLocked(src, nullptr, /*blocking=*/false);
      sched_yield();
      if ((spins & 0x3ff) == 0 && std::chrono::steady_clock::now() > deadline) {
        ctl_->slot[rank_].failed.store(1, std::memory_order_release);
        shared_->fail(c10::str("ccl backend: timed out waiting for rank ", r, " at collective #", seq_));
        TORCH_CHECK(false, "ccl backend: timed out waiting for rank ", r, " at collective #", seq_);
      }
    }
  }
}

// A rank with posted receives must not park a waiting kernel on its stream while a peer is still
// blocked in a send to it (the peer would never reach the collective, and the copy out of the
// peer's buffers would queue up behind the waiting kernel).  So it first takes messages in until
// every peer's host thread has entered this collective.  Ranks without posted receives only
// announce themselves.
void ProcessGroupCCL::awaitPeersEntered(uint64_t seq) {
  ctl_->slot[rank_].entered.store(seq + 1, std::memory_order_release);
  bool pending = false;
  for (const auto& pr : p2p_recv_) pending = pending || !pr.pending.empty();
  if (!pending) return;
  const auto deadline = std::chrono::steady_clock::now() + waitLimit(false);
  for (int r = 0; r < size_; ++r) {
    unsigned spins = 0;
    while (ctl_->slot[r].entered.load(std::memory_order_acquire) < seq + 1) {
      if (ctl_->slot[r].failed.load(std::memory_order_acquire) || ctl_->slot[r].departed.load(std::memory_order_acquire))
        return;  // the collective itself reports it
      for (int src = 0; src < size_; ++src)
        if (!p2p_recv_[(size_t)src].pending.empty()) progressRecvLocked(src, nullptr, /*blocking=*/false);
      if (++spins < 64) continue;
      sched_yield();
      if ((spins & 0x3ff) == 0 && std::chrono::steady_clock::now() > deadline) return;
    }
  }
}

void ProcessGroupCCL::throwIfFailed() {
  const std::string why = shared_->failureMessage();
  if (why.empty()) return;
  if (ctl_) ctl_->slot[rank_].failed.store(1, std::memory_order_release);
  TORCH_CHECK(false, why, lastEnqueued());
}

// What this rank enqueued last, for failure reports: a peer that others waited for in vain says
// here how far it had come.
std::string ProcessGroupCCL::lastEnqueued() const {
  if (!last_title_) return std::string();
  std::ostringstream os;
  os << " [rank " << rank_ << " had last enqueued collective #" << last_seq_ << " (" << last_title_ << ", " << last_path_ << ")";
  if (tail_pending_) os << (hipStreamQuery(tail_stream_) == hipSuccess ? ", its stream is idle" : ", its stream is still busy");
  os << "]";
  return os.str();
}

// The device-side cross-rank barrier on `s` (the sync kernels of src/gpu/allreduce.h:731-769).
void ProcessGroupCCL::deviceBarrier(uint64_t epoch, hipStream_t s) {
  const uint64_t limit_us = (uint64_t)waitLimit(false).count() * 1000ull;
  MCCL_CHECK(mccl_rank_barrier(bar_flags_.data(), size_, rank_, epoch, limit_us, status_dev_, s));
}

// ---------------------------------------------------------------------------------------------
// the engine: make the input visible to the peers, cross-rank barrier, data-path kernels
// ---------------------------------------------------------------------------------------------
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::run(Plan& plan) {
  std::lock_guard<std::mutex> lock(mutex_);
  int device = -1;
  for (const auto& t : plan.inputs) if (t.defined()) { device = t.get_device(); break; }
  if (device < 0) for (const auto& t : plan.outputs) if (t.defined()) { device = t.get_device(); break; }
  if (device < 0) device = initialised_ ? device_ : 0;  // barrier without tensors
  c10::DeviceGuard guard(c10::Device(at::kCUDA, (c10::DeviceIndex)device));
  hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA((c10::DeviceIndex)device).stream();
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HIP_CHECK(hipStreamIsCapturing(cur, &capture));
  if (capture != hipStreamCaptureStatusNone) {
    // The caller is recording a HIP graph.  What can be recorded is the one launch of the small
    // allreduce in its replayable form: its epoch and buffer choice live on the device, it needs no
    // rendezvous of the host threads, no memset and no allocation, so every replay is a complete
    // collective.  Everything else publishes tables or handles from the host at call time, which a
    // replay would not repeat: refused here rather than recorded wrongly.
    TORCH_CHECK(capture == hipStreamCaptureStatusActive, "ccl backend: the stream's capture has been invalidated");
    TORCH_CHECK(initialised_ && device == device_,
                "ccl backend: run one collective of this group before recording a HIP graph (the group's buffers are "
                "allocated and exchanged at its first collective, which cannot happen under stream capture)");
    throwIfFailed();
    TORCH_CHECK(device_sync_ && fusedFits(plan), "ccl backend: ", plan.title, " cannot be recorded into a HIP graph: under "
                "stream capture this backend takes all_reduce of at most ",
                (size_t)std::max(1u, (waits_in_data_kernels_ ? kComputeUnits : waiting_cus_) / (unsigned)size_) * kFusedBytesPerComputeUnit,
                " bytes per tensor (and not more than ", kFusedMaxBytes, ") between at most ", MCCL_FUSED_MAX_RANKS,
                " rank processes; larger tensors and the other collectives exchange tables or memory handles on the host "
                "at call time");
    // Not numbered: seq_ counts what the host has enqueued (the staging slots of the other
    // collectives alternate with it), and a recorded launch runs whenever its graph is replayed.
    if (verbose_) std::cout << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "] recorded (stream capture)" << std::endl;
    launchFused(plan, cur);
    return finishRun(plan, cur, /*same_stream=*/true, /*device_work=*/false, /*capturing=*/true);
  }
  ensureInit(device);
  TORCH_CHECK((int)plan.table.size() <= kTableMax, "ccl backend: too many tensors in one collective");
  throwIfFailed();

  // Which stream: the reference runs collectives on a communication stream that waits for the
  // caller's (src/gpu/dpcpp_ccl.cpp:186-197) unless CCL_SAME_STREAM=1.  Here all ranks share one
  // GPU, where the fork and join (two event records, two stream waits: packets of their own that
  // each wait for the process's turn at the dispatcher) cost several times the collective, and a
  // second queue per process with a waiting kernel in it makes the scheduler time-slice (measured:
  // 14 ms per collective with 8 processes).  So device-synchronised groups stay on the caller's
  // stream unless MCCL_PG_COMM_STREAM=1; host-synchronised ones use the communication stream for
  // large messages as before.
  const size_t payload = std::max(plan.stage_bytes, plan.share ? plan.share_bytes : (size_t)0);
  const bool same_stream = same_stream_ || payload <= kInlineStreamMax || (device_sync_ && !comm_stream_for_large_);
  hipStream_t s = same_stream ? cur : comm_stream_;
  if (!same_stream) {  // sync_streams of the reference (src/gpu/dpcpp_ccl.cpp:186-197)
    HIP_CHECK(hipEventRecord(fork_event_, cur));
    HIP_CHECK(hipStreamWaitEvent(comm_stream_, fork_event_, 0));
  }

  const uint64_t seq = seq_;
  const int slot = (int)(seq_ & 1);
  ++seq_;
  if (verbose_) {
    std::ostringstream os;
    os << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "#" << seq_ << "]";
    for (const auto& t : plan.inputs) os << " in" << t.sizes();
    for (const auto& t : plan.outputs) os << " out" << t.sizes();
    std::cout << os.str() << std::endl;
  }
  if (device_sync_) {
    runDeviceSynced(plan, s, slot, seq);
  } else {
    runHostSynced(plan, s, slot);
  }
  return finishRun(plan, s, same_stream, /*device_work=*/true);
}

// Ranks that share a process (or MCCL_PG_SYNC=host): copy-in, hipStreamSynchronize, host barrier,
// kernels.  No kernel ever waits for another rank.
void ProcessGroupCCL::runHostSynced(Plan& plan, hipStream_t s, int slot) {
  RankSlot& me = ctl_->slot[rank_];
  const int pub = slot;  // every collective meets at the host barrier: the records alternate with the slots
  using clk = std::chrono::steady_clock;
  auto us_since = [](clk::time_point t) { return std::chrono::duration<double, std::micro>(clk::now() - t).count(); };
  const bool timed = profile_ && plan.stage_bytes > 0 && phase_us_[0].size() < (1u << 20);
  auto t0 = clk::now();
  // In place (rank processes only): an allreduce whose tensors all ranks can share needs no staging
  // at all -- every rank reduces its shard of all tensors and writes it into all of them -- and the
  // two host barriers the staged two-shot form needs anyway order it: tensors complete / everybody
  // done.  The kernel is the one-launch kernel of the device-synchronised mode with its waits off.
  const bool candidate = distinct_pids_ && zero_copy_ && plan.share && plan.exec_sync && plan.exec_sync_in_place_only &&
                         size_ <= MCCL_FUSED_MAX_RANKS;
  if (candidate) {
    bool in_place = true;
    try {
      RankSlot::Published& rec = me.pub[pub];
      uint64_t off = 0;
      const int entry = exportRange(plan.share_ptr, plan.share_bytes, &off);
      rec.share_entry = entry;
      rec.share_off = off;
      rec.share_gen = (entry >= 0 && entry < kMaxExports) ? me.exports[entry].gen.load(std::memory_order_acquire) : 0;
      if (tail_pending_ && tail_stream_ != s) HIP_CHECK(hipStreamSynchronize(tail_stream_));
      HIP_CHECK(hipStreamSynchronize(s));
    } catch (...) {
      me.failed.store(1, std::memory_order_release);
      throw;
    }
    hostBarrier();  // every rank's tensor is complete and its offer published
    for (int r = 0; r < size_; ++r)
      if (ctl_->slot[r].pub[pub].share_entry < 0) in_place = false;
    if (in_place) {
      try {
        PeerView pv;
        pv.zero_copy = true;
        pv.user.resize((size_t)size_);
        for (int r = 0; r < size_; ++r) pv.user[(size_t)r] = (r == rank_) ? plan.share_ptr : importRange(r, pub);
        mccl_xsync_t sync{};
        sync.n = size_;
        sync.rank = rank_;  // ready_epoch 0: no waits inside the kernel
        TORCH_CHECK(plan.exec_sync(pv, sync, s), "ccl backend: the in-place plan declined");
        HIP_CHECK(hipStreamSynchronize(s));
      } catch (...) {
        me.failed.store(1, std::memory_order_release);
        throw;
      }
      hostBarrier();  // every rank has written its shard everywhere
      if (timed) phase_us_[3].push_back((float)us_since(t0));
      return;
    }
    // somebody cannot share: the staged form below (every rank sees the same offers)
  }
  try {
    void* stage = ensureStage(slot, plan.stage_bytes);
    publishStage(slot, pub);
    for (size_t i = 0; i < plan.table.size(); ++i) me.pub[pub].table[i] = plan.table[i];
    if (plan.copy_in) plan.copy_in(stage, s);
    if (timed) { phase_us_[0].push_back((float)us_since(t0)); t0 = clk::now(); }
    // This rank's staging buffer must be complete before any peer reads it, and (two
    // collectives later) every peer must be done reading before it is overwritten: one host
    // barrier per collective plus the two alternating buffers give both, provided the
    // synchronisation below covers this rank's earlier kernels.  On one stream it does; a
    // previous collective that ran on another stream is waited for through its tail event.
    if (tail_pending_ && tail_stream_ != s) HIP_CHECK(hipStreamSynchronize(tail_stream_));
    HIP_CHECK(hipStreamSynchronize(s));
  } catch (...) {
    // this rank will not arrive: tell the peers now instead of letting them run into the timeout
    me.failed.store(1, std::memory_order_release);
    throw;
  }
  if (timed) { phase_us_[1].push_back((float)us_since(t0)); t0 = clk::now(); }
  hostBarrier();
  if (timed) { phase_us_[2].push_back((float)us_since(t0)); t0 = clk::now(); }

  if (plan.exec) {
    PeerView pv;
    pv.stage.resize((size_t)size_);
    pv.tables.resize((size_t)size_);
    try {
      for (int r = 0; r < size_; ++r) {
        pv.stage[(size_t)r] = peerStage(r, slot, pub);
        pv.tables[(size_t)r] = ctl_->slot[r].pub[pub].table;
      }
      plan.exec(pv, s);
      if (plan.exec2 && (!plan.two_phase || plan.two_phase(pv))) HIP_CHECK(hipStreamSynchronize(s));
    } catch (...) {
      me.failed.store(1, std::memory_order_release);  // the peers must not wait for this rank at the next barrier
      throw;
    }
    if (plan.exec2 && (!plan.two_phase || plan.two_phase(pv))) {
      hostBarrier();
      try {
        plan.exec2(pv, s);
      } catch (...) {
        me.failed.store(1, std::memory_order_release);
        throw;
      }
    }
  }
  if (timed) phase_us_[3].push_back((float)us_since(t0));
}

// Ranks that are processes of their own: everything a collective needs from its peers on the
// device arrives through flag kernels on the collective's stream; the host only enqueues.  What
// the host still exchanges -- tables of the v-collectives, new staging handles, the ranges offered
// for zero-copy -- goes through the control block in a rendezvous of the host threads (no GPU
// synchronisation); the one-launch allreduce needs none of it.
//
// Why one barrier per collective is enough to reuse the two alternating staging slots: the device
// work of collective k contains a wait for every peer's START of its collective k (barrier flag
// or tile flags), and a rank's collectives execute in order on the device.  So when this rank's
// collective k + 1 has completed, every peer has started k + 1 and therefore finished k: slot
// (k & 1) is free when this rank's collective k + 2 writes it.
void ProcessGroupCCL::runDeviceSynced(Plan& plan, hipStream_t s, int slot, uint64_t seq) {
  RankSlot& me = ctl_->slot[rank_];
  using clk = std::chrono::steady_clock;
  auto us_since = [](clk::time_point t) { return std::chrono::duration<double, std::micro>(clk::now() - t).count(); };
  const bool timed = profile_ && plan.stage_bytes > 0 && phase_us_[0].size() < (1u << 20);
  auto t0 = clk::now();
  const uint64_t epoch = 4 * seq;  // up to three barriers per collective: epoch + 1, + 2, + 3
  try {
    awaitPeersEntered(seq);
    // a rank's collectives are totally ordered on the device, whichever streams they use
    // (the event is only recorded when a collective changes streams: a record is a packet of its
    // own, and with several processes on one GPU every packet waits for the process's turn)
    if (tail_pending_ && tail_stream_ != s) {
      HIP_CHECK(hipEventRecord(tail_event_, tail_stream_));
      HIP_CHECK(hipStreamWaitEvent(s, tail_event_, 0));
    }
    last_title_ = plan.title;
    last_seq_ = seq + 1;
    last_path_ = "one launch, fused";
    auto say_path = [&] {
      if (!verbose_) return;
      std::ostringstream os;
      os << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "#" << (seq + 1) << "] " << last_path_;
      std::cout << os.str() << std::endl;
    };
    if (fusedFits(plan)) {
      say_path();
      launchFused(plan, s);
      if (timed) phase_us_[3].push_back((float)us_since(t0));
      return;
    }
    if (standingFits(plan)) {
      runStanding(plan, s, slot, seq);
      if (timed) phase_us_[3].push_back((float)us_since(t0));
      return;
    }
    const bool candidate = zero_copy_ && plan.share;
    // the record this collective publishes in: they alternate per collective that rendezvous
    const int pub = (int)(rendezvous_count_++ & 1);
    RankSlot::Published& rec = me.pub[pub];
    for (size_t i = 0; i < plan.table.size(); ++i) rec.table[i] = plan.table[i];
    void* stage = nullptr;
    if (candidate) {
      uint64_t off = 0;
      const int entry = exportRange(plan.share_ptr, plan.share_bytes, &off);
      rec.share_entry = entry;
      rec.share_off = off;
      rec.share_gen = (entry >= 0 && entry < kMaxExports) ? me.exports[entry].gen.load(std::memory_order_acquire) : 0;
      stage = ensureStage(slot, plan.zero_copy_stage_bytes);
    } else {
      rec.share_entry = -1;
      stage = ensureStage(slot, plan.stage_bytes);
    }
    publishStage(slot, pub);
    if (timed) { phase_us_[0].push_back((float)us_since(t0)); t0 = clk::now(); }
    hostBarrier();  // of the host threads only: tables, handles and offers are published
    bool zero_copy = candidate;
    if (candidate) {
      for (int r = 0; r < size_; ++r)
        if (ctl_->slot[r].pub[pub].share_entry < 0) zero_copy = false;
      if (!zero_copy) {  // somebody cannot share: everybody stages (every rank sees the same offers)
        stage = ensureStage(slot, plan.stage_bytes);
        publishStage(slot, pub);  // nobody reads the staging part of a record before the second rendezvous
        hostBarrier();
      }
    }
    PeerView pv;
    pv.stage.resize((size_t)size_);
    pv.tables.resize((size_t)size_);
    pv.zero_copy = zero_copy;
    for (int r = 0; r < size_; ++r) {
      pv.stage[(size_t)r] = peerStage(r, slot, pub);
      pv.tables[(size_t)r] = ctl_->slot[r].pub[pub].table;
    }
    if (zero_copy) {
      pv.user.resize((size_t)size_);
      for (int r = 0; r < size_; ++r) pv.user[(size_t)r] = (r == rank_) ? plan.share_ptr : importRange(r, pub);
    }
    if (timed) { phase_us_[1].push_back((float)us_since(t0)); t0 = clk::now(); }
    if (sync_only_) {
      // bisecting: the cross-rank waits of the default form and nothing else
      last_path_ = "sync only";
      say_path();
      deviceBarrier(epoch + 1, s);
      if (zero_copy) deviceBarrier(epoch + 3, s);
      return;
    }
    if (work_only_) {
      // bisecting: the data movement alone, nobody waits for anybody (results are not valid)
      last_path_ = "work only";
      say_path();
      if (!zero_copy && plan.copy_in) plan.copy_in(stage, s);
      mccl_xsync_t none{};
      none.n = size_;
      none.rank = rank_;
      if (plan.exec_sync && size_ <= MCCL_FUSED_MAX_RANKS && (zero_copy || !plan.exec_sync_in_place_only) && plan.exec_sync(pv, none, s)) return;
      if (plan.exec) plan.exec(pv, s);
      if (plan.exec2 && (!plan.two_phase || plan.two_phase(pv))) plan.exec2(pv, s);
      return;
    }
    // One launch: the kernel itself announces this rank, waits for the others, does the work and
    // (in place: where a tensor must not be touched before the peers have read it) waits again.
    // With several processes on the GPU every launch waits for its turn at the dispatcher, so this
    // is worth more than any bandwidth.  Staged collectives get the same kernel behind their
    // copy-in (two launches instead of three): the launch says "my staging buffer is complete",
    // and no closing wait is needed, as for every staged collective (see the slot rule above).
    const size_t moved = zero_copy ? plan.share_bytes : plan.stage_bytes;
    const bool can_wait_inside = plan.exec_sync && size_ <= MCCL_FUSED_MAX_RANKS && (zero_copy || !plan.exec_sync_in_place_only);
    // (compact: all ranks' waiting workgroups together on at most half of the compute units)
    const bool compact = !waits_in_data_kernels_ && can_wait_inside && (double)moved * plan.compact_cost <= (double)compact_max_;
    const bool one_launch = compact || (waits_in_data_kernels_ && can_wait_inside &&
                                        ((zero_copy && plan.one_launch_any_size && !one_launch_max_forced_) || moved <= one_launch_max_));
    last_path_ = one_launch ? (zero_copy ? "one launch, peers read in place" : "copy-in and one launch")
                            : zero_copy ? "barrier kernel, peers read in place"
                                        : candidate ? "staged: a rank cannot share its tensor" : "staged";
    say_path();
    if (one_launch) {
      if (!zero_copy && plan.copy_in) plan.copy_in(stage, s);
      mccl_xsync_t sync{};
      sync.words = bar_flags_.data();
      sync.n = size_;
      sync.rank = rank_;
      sync.ready_epoch = epoch + 1;
      sync.done_epoch = zero_copy ? epoch + 3 : 0;
      sync.max_compute_units = compact ? std::max(1u, waiting_cus_ / (unsigned)size_) : 0u;
      sync.done_counter = done_counter_;
      sync.timeout_us = (uint64_t)deviceWaitLimit().count() * 1000ull;
      sync.status = status_dev_;
      if (plan.exec_sync(pv, sync, s)) {
        if (timed) { phase_us_[2].push_back(0.f); phase_us_[3].push_back((float)us_since(t0)); }
        return;
      }
      TORCH_CHECK(zero_copy || !plan.copy_in, "ccl backend: a staged one-launch plan declined after its copy-in");
    }
    if (!zero_copy && plan.copy_in) plan.copy_in(stage, s);
    deviceBarrier(epoch + 1, s);  // every rank's input is complete (staged, or ready in place)
    if (timed) { phase_us_[2].push_back((float)us_since(t0)); t0 = clk::now(); }
    if (zero_copy && plan.exec_sync && size_ <= MCCL_FUSED_MAX_RANKS &&
        (plan.exec_sync_in_place_only || plan.share_bytes <= one_launch_max_)) {
      // Peers' tensors in place behind a barrier kernel: the data kernel starts without a wait
      // (ready_epoch 0) and only its last workgroup waits, for the closing epoch -- nobody may touch
      // its tensor before every peer has read (allreduce: written) it.  Two launches, and never
      // more than one waiting wavefront per rank on the GPU.
      mccl_xsync_t sync{};
      sync.words = bar_flags_.data();
      sync.n = size_;
      sync.rank = rank_;
      sync.done_epoch = epoch + 3;
      sync.done_counter = done_counter_;
      sync.timeout_us = (uint64_t)deviceWaitLimit().count() * 1000ull;
      sync.status = status_dev_;
      if (plan.exec_sync(pv, sync, s)) {
        if (timed) phase_us_[3].push_back((float)us_since(t0));
        return;
      }
    }
    if (plan.exec) plan.exec(pv, s);
    if (plan.exec2 && (!plan.two_phase || plan.two_phase(pv))) {
      deviceBarrier(epoch + 2, s);
      plan.exec2(pv, s);
    }
    // in place: nobody may touch its tensor again before every peer has read it
    if (zero_copy) deviceBarrier(epoch + 3, s);
    if (timed) phase_us_[3].push_back((float)us_since(t0));
  } catch (...) {
    // this rank may not have enqueued what its peers wait for: tell them now
    me.failed.store(1, std::memory_order_release);
    shared_->fail("ccl backend: a collective of this rank failed on the host; the group cannot be used any more");
    throw;
  }
}

// On this rank's share of the compute units that all ranks' waiting launches may hold together (a
// share takes 64 KiB per compute unit).  With MCCL_PG_SYNC=kernel the share is one workgroup per
// compute unit and rank, half of what the GPU holds: a wavefront of this kernel waits for the same
// tile of every peer, so all of a late rank's workgroups must still find room beside the waiting
// ones, and a launch per 16 KiB (8 ranks x 1 MiB: 512 workgroups, exactly what fits when nothing
// else runs) leaves none to spare.
bool ProcessGroupCCL::fusedFits(const Plan& plan) const {
  const unsigned units = std::max(1u, (waits_in_data_kernels_ ? kComputeUnits : waiting_cus_) / (unsigned)size_);
  return plan.fused_ok && size_ <= MCCL_FUSED_MAX_RANKS &&
         plan.fused_count * mccl_dtype_size(plan.fused_dtype) <= (size_t)units * kFusedBytesPerComputeUnit;
}

// The epoch of the launch and its choice between the two sets of staging buffers and flags are read
// from this rank's arena by the launch itself and advanced by it, so the same launch serves eager
// calls and replays of a recorded graph, in any mixture, and all ranks' counters agree as long as
// the ranks issue the same collectives (which they must anyway).
void ProcessGroupCCL::launchFused(const Plan& plan, hipStream_t s) {
  const unsigned units = std::max(1u, (waits_in_data_kernels_ ? kComputeUnits : waiting_cus_) / (unsigned)size_);
  last_title_ = plan.title;
  last_path_ = "one launch, fused";
  ++enqueue_only_count_;
  const uint64_t limit_us = (uint64_t)deviceWaitLimit().count() * 1000ull;
  MCCL_CHECK(mccl_allreduce_fused_replayable(plan.fused_ptr, plan.fused_ptr, plan.fused_count, plan.fused_dtype, plan.fused_op,
                                             fused_stage_[0].data(), fused_flags_[0].data(), kArenaFusedStageStride,
                                             kArenaFusedFlagsStride, fused_state_, size_, rank_, limit_us,
                                             static_cast<char*>(status_dev_) + 8, units, fused_mode_, s));
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::finishRun(Plan& plan, hipStream_t s, bool same_stream, bool device_work, bool capturing) {
  if (device_work) {
    tail_stream_ = s;
    tail_pending_ = true;
  }
  auto work = c10::make_intrusive<WorkCCL>(rank_, plan.op, plan.title, plan.inputs, plan.outputs, blocking_wait_ && !capturing);
  work->captured_ = capturing;
  work->device_ = device_;
  work->shared_ = shared_;
  work->op_timeout_ = timeout_;
  work->stream_ = s;
  work->stream_set_ = true;
  if (!same_stream) {
    // the collective ran on the communication stream: its end is an event the caller's streams
    // can wait for
    work->end_ = shared_->getEvent();
    HIP_CHECK(hipEventRecord(work->end_, s));
    // record_tensor of the reference (src/gpu/dpcpp_ccl.cpp:199-207)
    auto cs = c10::hip::getStreamFromExternalMasqueradingAsCUDA(comm_stream_, (c10::DeviceIndex)device_);
    for (const auto* list : {&plan.inputs, &plan.outputs})
      for (const auto& t : *list)
        if (t.defined() && t.has_storage() && t.numel() > 0)
          c10::hip::HIPCachingAllocatorMasqueradingAsCUDA::recordStreamMasqueradingAsCUDA(t.storage().data_ptr(), cs);
  }
  if (same_stream && blocking_wait_ && !capturing) {
    // CCL_BLOCKING_WAIT: wait() polls until THIS collective is done or its time is up, so its end is
    // marked -- the state of the whole stream would count kernels the caller enqueues behind the
    // collective against its timeout.  The record is a packet of its own, paid in this mode only.
    work->end_ = shared_->getEvent();
    HIP_CHECK(hipEventRecord(work->end_, s));
  }
  if (plan.host_complete) {
    // a barrier returns once every rank has arrived: the host waits for the flag kernel
    work->blocking_wait_ = true;
    work->waitInternal(kNoTimeout);
    work->blocking_wait_ = blocking_wait_;
  }
  if (coalescing_) last_work_ = work;
  return work;
}

// The list as one range of memory: its non-empty tensors are consecutive views of one storage
// (computeLengthsAndCheckFlat of the reference, src/utils.cpp:157-193).  A list of empty tensors
// is flat and empty.
ProcessGroupCCL::FlatSpan ProcessGroupCCL::flatSpan(const std::vector<at::Tensor>& tensors) {
  FlatSpan span;
  span.flat = true;
  const at::Tensor* first = nullptr;
  for (const auto& t : tensors) {
    const size_t b = nbytes(t);
    if (!b) continue;
    if (!first) {
      first = &t;
      span.ptr = t.data_ptr();
    } else if (!first->storage().is_alias_of(t.storage()) || (const char*)t.data_ptr() != (const char*)span.ptr + span.bytes) {
      return FlatSpan{};
    }
    span.bytes += b;
  }
  return span;
}

void ProcessGroupCCL::checkDeviceTensors(const std::vector<at::Tensor>& tensors) const {
  // checkSingleTensorHelper / checkSameType of the reference (src/utils.cpp:217-255) with the
  // device test turned around: this backend takes GPU tensors only.
  TORCH_CHECK(!tensors.empty(), "ccl backend: empty tensor list");
  const auto& first = tensors[0];
  for (const auto& t : tensors)
    TORCH_CHECK(t.scalar_type() == first.scalar_type(), "Tensors are not equal in data type");
  for (const auto& t : tensors) {
    TORCH_CHECK(t.is_cuda(), "Tensors are not in same device type. Expect: cuda But got: ", t.device().type());
    TORCH_CHECK(t.get_device() == first.get_device(), "ccl backend: tensors of one collective must share a device");
    TORCH_CHECK(!t.is_sparse(), "ccl backend: sparse tensors are not supported");
    TORCH_CHECK(t.is_contiguous(t.suggest_memory_format()), "input dense tensor has to be contiguous");
  }
}

void ProcessGroupCCL::startCoalescing() { coalescing_ = true; }

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::endCoalescing() {
  // Collectives issued between start and end have already been enqueued in order on the
  // communication stream; the last Work covers them all.
  coalescing_ = false;
  if (last_work_) {
    auto w = last_work_;
    last_work_.reset();
    return w;
  }
  return c10::make_intrusive<WorkCCL>(rank_, c10d::OpType::COALESCED, "endCoalescing",
                                      std::vector<at::Tensor>{}, std::vector<at::Tensor>{}, blocking_wait_);
}

// ---------------------------------------------------------------------------------------------
// collectives
// ---------------------------------------------------------------------------------------------
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::broadcast(std::vector<at::Tensor>& tensors,
                                                          const c10d::BroadcastOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::broadcast", std::vector<c10::IValue>({tensors}));
  checkRank((int)opts.rootRank, size_);
  TORCH_CHECK(tensors.size() == 1, "CCL process group does not support tensors count ", tensors.size());
  checkDeviceTensors(tensors);
  at::Tensor t = tensors[0];
  const int root = (int)opts.rootRank;
  const size_t total = nbytes(t);
  c10::intrusive_ptr<c10d::Work> work;
  size_t off = 0;
  do {
    const size_t len = std::min(total - off, stage_max_);
    char* base = total ? (char*)t.data_ptr() + off : nullptr;
    Plan p;
    p.op = c10d::OpType::BROADCAST;
    p.title = "broadcast";
    p.inputs = {t};
    p.outputs = {t};
    p.stage_bytes = (rank_ == root) ? len : 0;
    // large messages: the peers read the root's tensor in place (every rank offers its own tensor:
    // the offer has to look the same on all ranks)
    p.share = len >= kZeroCopyMinBytes;
    p.share_ptr = base;
    p.share_bytes = len;
    if (rank_ == root && len)
      p.copy_in = [=](void* stage, hipStream_t s) {
        copyAsync(stage, base, len, s);
      };
    if (rank_ != root && len)
      p.exec = [=](const PeerView& pv, hipStream_t s) {
        mccl_segment_t seg{pv.zero_copy ? pv.user[(size_t)root] : pv.stage[(size_t)root], base, len};
        MCCL_CHECK(mccl_copy_segments(&seg, 1, s));
      };
    if (len) {
      const int me = rank_;
      p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
        mccl_segment_t seg{pv.zero_copy ? pv.user[(size_t)root] : pv.stage[(size_t)root], base, len};
        MCCL_CHECK(mccl_copy_segments_sync(&seg, me == root ? 0 : 1, MCCL_COPY_SHARED_SOURCES, &sync, s));  // the root only takes part in the waits
        return true;
      };
    }
    work = run(p);
    off += len;
  } while (off < total);
  return work;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::allreduce(std::vector<at::Tensor>& tensors,
                                                          const c10d::AllreduceOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::allreduce", std::vector<c10::IValue>({tensors}));
  TORCH_CHECK(tensors.size() == 1, "CCL process group does not support tensors count ", tensors.size());
  checkDeviceTensors(tensors);
  at::Tensor t = tensors[0];
  const int dtype = dtypeCode(t.scalar_type());
  const int op = opCode(opts.reduceOp, t.scalar_type());
  const size_t es = t.element_size();
  const size_t total = (size_t)t.numel();
  // one staging window holds the input; the two-shot form reduces each shard in place there
  const size_t chunk = stage_max_ / es;
  c10::intrusive_ptr<c10d::Work> work;
  size_t off = 0;
  do {
    const size_t len = std::min(total - off, chunk);
    char* base = total ? (char*)t.data_ptr() + off * es : nullptr;
    Plan p;
    p.op = c10d::OpType::ALLREDUCE;
    p.title = "allreduce";
    p.inputs = {t};
    p.outputs = {t};
    if (size_ > 1 && len && !disable_allreduce_) {  // world == 1 or switched off: nothing to add (src/gpu/dpcpp_ccl.cpp:752-756)
      const int W = size_;
      const int me = rank_;
      // elements per shard: a whole number of 64-element groups, so that every shard starts on a
      // 16-byte boundary of the staging buffers whatever the element size; the last may be shorter
      const size_t shard = roundUp((len + (size_t)W - 1) / (size_t)W, 64);
      const bool two_shot = W >= kTwoShotMinRanks && len * es >= kTwoShotMinBytes;
      auto shard_len = [=](int r) {
        const size_t lo = std::min(len, (size_t)r * shard);
        return std::min(len, lo + shard) - lo;
      };
      // Small messages between rank processes: one launch does copy-in, rank synchronisation and
      // the N-peer sum (the reference's small allreduce, src/gpu/allreduce_small.h:166-361).
      p.fused_ok = len * es <= kFusedMaxBytes;
      // whatever is too large for that launch: where the tensors are is exchanged on the device, no rendezvous
      p.standing.ok = true;
      p.standing.buffer = base;
      p.standing.bytes = len * es;
      p.standing.copy_in = p.standing.copy_out = true;
      p.standing.compact_cost = 1.0;
      p.standing.behind_barrier = [=](const void* resolved, bool, const mccl_xsync_t& sync, hipStream_t s) {
        MCCL_CHECK(mccl_allreduce_sync_resolved(resolved, len, dtype, op, &sync, s));
      };
      p.standing.one_launch = [=](bool, const mccl_xsync_t& sync, const mccl_offer_t& mine, const void* buffer, void* const* offers,
                                  const mccl_import_table_t* imports, hipStream_t s) {
        MCCL_CHECK(mccl_allreduce_sync_offers(len, dtype, op, &sync, &mine, buffer, offers, imports, s));
      };
      p.fused_ptr = base;
      p.fused_count = len;
      p.fused_dtype = dtype;
      p.fused_op = op;
      // Large messages between rank processes: the peers read this tensor in place.  Rank r
      // reduces shard r of all tensors into its staging buffer (nobody writes a tensor while
      // anybody reads one), then all ranks gather the W finished shards into their tensors:
      // about 3 S bytes per rank and no copy-in, against (4 + 1/W) S for the staged two-shot.
      p.share = !p.fused_ok && len * es >= kZeroCopyMinBytes;
      p.share_ptr = base;
      p.share_bytes = len * es;
      p.zero_copy_stage_bytes = shard * es;
      p.stage_bytes = len * es;
      p.copy_in = [=](void* stage, hipStream_t s) { copyAsync(stage, base, len * es, s); };
      p.two_phase = [=](const PeerView& pv) { return pv.zero_copy || two_shot; };
      p.exec = [=](const PeerView& pv, hipStream_t s) {
        if (pv.zero_copy) {
          const size_t n_me = shard_len(me);
          if (!n_me) return;
          std::vector<const void*> in((size_t)W);
          for (int k = 0; k < W; ++k) in[(size_t)k] = (const char*)pv.user[(size_t)k] + (size_t)me * shard * es;
          MCCL_CHECK(mccl_reduce_n(in.data(), W, (void*)pv.stage[(size_t)me], n_me, dtype, op, MCCL_VARIANT_AUTO, s));
        } else if (!two_shot) {
          // This rank's contribution is read from the tensor itself (its staging copy holds the
          // same bytes), which makes the reduction in place: the output lands on DRAM pages the
          // kernel has just read (5 % faster than a separate output on large messages).
          std::vector<const void*> in = pv.stage;
          in[(size_t)me] = base;
          MCCL_CHECK(mccl_reduce_n(in.data(), W, base, len, dtype, op, MCCL_VARIANT_AUTO, s));
        } else {
          // Rank r reduces shard r of all staged inputs in place in its own staging buffer: nobody
          // else reads that range in this phase (rank k reads shard k of every buffer), the output
          // lands on DRAM pages the kernel has just read, and after the second barrier shard r of
          // staging buffer r is the finished shard.
          const size_t n_me = shard_len(me);
          if (!n_me) return;
          std::vector<const void*> in((size_t)W);
          for (int k = 0; k < W; ++k) in[(size_t)k] = (const char*)pv.stage[(size_t)k] + (size_t)me * shard * es;
          void* red = (char*)pv.stage[(size_t)me] + (size_t)me * shard * es;  // pv.stage[me] is this rank's own staging buffer
          MCCL_CHECK(mccl_reduce_n(in.data(), W, red, n_me, dtype, op, MCCL_VARIANT_AUTO, s));
        }
      };
      // One launch, at most eight ranks: rank r reduces shard r of all tensors and writes the result
      // into shard r of every rank's tensor (the peers' mappings are writable): S bytes read and S
      // written per rank, nothing staged.  Faster than the launches of the form above at every
      // size measured (16 MiB to 512 MiB per rank), so it is not subject to the one-launch limit.
      p.one_launch_any_size = true;
      p.exec_sync_in_place_only = true;
      p.compact_cost = 1.0;
      p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
        std::vector<void*> tensors((size_t)W);
        for (int k = 0; k < W; ++k) tensors[(size_t)k] = const_cast<void*>(pv.user[(size_t)k]);
        MCCL_CHECK(mccl_allreduce_sync(tensors.data(), len, dtype, op, &sync, s));
        return true;
      };
      p.exec2 = [=](const PeerView& pv, hipStream_t s) {
        // the finished shard of rank r: the start of its staging buffer (zero-copy) or shard r of it
        std::vector<mccl_segment_t> segs;
        for (int r = 0; r < W; ++r) {
          const size_t n_r = shard_len(r);
          const size_t at = pv.zero_copy ? 0 : (size_t)r * shard * es;
          if (n_r) segs.push_back({(const char*)pv.stage[(size_t)r] + at, base + (size_t)r * shard * es, n_r * es});
        }
        MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
      };
    }
    work = run(p);
    off += len;
  } while (off < total);
  return work;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::allreduce_coalesced(
    std::vector<at::Tensor>& tensors, const c10d::AllreduceCoalescedOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::allreduce_coalesced", std::vector<c10::IValue>({tensors}));
  checkDeviceTensors(tensors);
  const int dtype = dtypeCode(tensors[0].scalar_type());
  const int op = opCode(opts.reduceOp, tensors[0].scalar_type());
  // one staging image: the tensors back to back, each on a 16-byte boundary
  std::vector<size_t> offs(tensors.size());
  size_t total = 0;
  for (size_t i = 0; i < tensors.size(); ++i) {
    offs[i] = total;
    total += roundUp(nbytes(tensors[i]), 16);
  }
  if (total > stage_max_) {
    // more than one staging window: one (windowed) allreduce per tensor; same results, same order
    // on every rank (the shapes of a coalesced call agree across ranks)
    c10::intrusive_ptr<c10d::Work> last;
    c10d::AllreduceOptions one;
    one.reduceOp = opts.reduceOp;
    for (auto& t : tensors) {
      std::vector<at::Tensor> v{t};
      last = allreduce(v, one);
    }
    return last;
  }
  Plan p;
  p.op = c10d::OpType::ALLREDUCE_COALESCED;
  p.title = "allreduce_coalesced";
  p.inputs = tensors;
  p.outputs = tensors;
  if (size_ > 1 && total) {
    p.stage_bytes = total;
    std::vector<at::Tensor> ts = tensors;
    const int W = size_;
    p.copy_in = [=](void* stage, hipStream_t s) {
      std::vector<mccl_segment_t> segs;
      for (size_t i = 0; i < ts.size(); ++i)
        if (ts[i].numel()) segs.push_back({ts[i].data_ptr(), (char*)stage + offs[i], nbytes(ts[i])});
      MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
    };
    p.exec = [=](const PeerView& pv, hipStream_t s) {
      std::vector<const void*> in;
      std::vector<void*> out;
      std::vector<size_t> counts;
      for (size_t i = 0; i < ts.size(); ++i) {
        if (!ts[i].numel()) continue;
        for (int k = 0; k < W; ++k) in.push_back((const char*)pv.stage[(size_t)k] + offs[i]);
        out.push_back(ts[i].data_ptr());
        counts.push_back((size_t)ts[i].numel());
      }
      MCCL_CHECK(mccl_reduce_multi(in.data(), W, out.data(), counts.data(), (int)out.size(), dtype, op, s));
    };
  }
  return run(p);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::_allgather_base(at::Tensor& output, at::Tensor& input,
                                                                const c10d::AllgatherOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::_allgather_base", std::vector<c10::IValue>({input}));
  checkDeviceTensors({output, input});
  TORCH_CHECK(input.numel() * size_ == output.numel(),
              "output tensor size must be equal to world_size times input tensor size");
  const size_t per_rank = nbytes(input);
  c10::intrusive_ptr<c10d::Work> work;
  size_t off = 0;
  do {
    const size_t len = std::min(per_rank - off, stage_max_);
    char* in = per_rank ? (char*)input.data_ptr() + off : nullptr;
    char* out = per_rank ? (char*)output.data_ptr() + off : nullptr;
    Plan p;
    p.op = c10d::OpType::_ALLGATHER_BASE;
    p.title = "_allgather_base";
    p.inputs = {input};
    p.outputs = {output};
    if (len) {
      p.stage_bytes = len;
      const int W = size_;
      const int me = rank_;
      p.copy_in = [=](void* stage, hipStream_t s) {
        copyAsync(stage, in, len, s);
      };
      auto pulls = [=](const PeerView& pv) {
        std::vector<mccl_segment_t> segs((size_t)W);
        for (int r = 0; r < W; ++r)
          segs[(size_t)r] = {pv.zero_copy ? pv.user[(size_t)r] : pv.stage[(size_t)r], out + (size_t)r * per_rank, len};
        return segs;
      };
      // Between rank processes the contributions are pushed: what the ranks offer each other is the
      // OUTPUT, and rank r writes its input into slice r of every rank's output in one pass (read
      // once, written W times; the peers' mappings are writable) -- pulls have every rank read all
      // W inputs (64 MiB per rank, 8 rank processes: 1.04 ms pushed, 1.43 ms pulled).  An output
      // too large to be shared leaves the pulls: the inputs are offered instead.  Which of the two
      // depends on sizes only, which agree across the ranks.
      const bool push = allgather_push_ && (uint64_t)per_rank * (uint64_t)W < kShareMaxAllocation;
      if (push && len == per_rank && W <= MCCL_OFFER_RANKS) {
        // One window, at most eight ranks: no rendezvous.  What the peers address is this rank's whole
        // OUTPUT, into which rank r writes slice r; a rank that stages receives in its staging buffer
        // and copies it out afterwards (also when its input lies inside another rank's slice of its
        // output).  In place -- the input is this rank's slice of its output -- nothing is written there.
        const bool input_is_own_slice = (const char*)input.data_ptr() == (const char*)output.data_ptr() + (size_t)me * per_rank;
        p.standing.ok = true;
        p.standing.buffer = output.data_ptr();
        p.standing.bytes = per_rank * (size_t)W;
        p.standing.copy_out = true;
        p.standing.force_staged = touchesForeignSlice(input.data_ptr(), per_rank, output.data_ptr(), per_rank, W, me);
        p.standing.compact_cost = 1.0;
        p.standing.behind_barrier = [=](const void* resolved, bool staged, const mccl_xsync_t& sync, hipStream_t s) {
          MCCL_CHECK(mccl_fanout_sync_resolved(in, resolved, (size_t)me * per_rank, per_rank, !staged && input_is_own_slice, &sync, s));
        };
        p.standing.one_launch = [=](bool staged, const mccl_xsync_t& sync, const mccl_offer_t& mine, const void* buffer, void* const* offers,
                                    const mccl_import_table_t* imports, hipStream_t s) {
          MCCL_CHECK(mccl_fanout_sync_offers(in, (size_t)me * per_rank, per_rank, !staged && input_is_own_slice, &sync, &mine, buffer,
                                             offers, imports, s));
        };
      }
      if (push) {
        p.share = len * (size_t)W >= kZeroCopyMinBytes;
        // (an input inside another rank's slice of the output: nothing is offered, and then every rank stages)
        p.share_ptr = touchesForeignSlice(input.data_ptr(), per_rank, output.data_ptr(), per_rank, W, me) ? nullptr : output.data_ptr();
        p.share_bytes = per_rank * (size_t)W;
        auto destinations = [=](const PeerView& pv, int k0, int k1) {
          std::vector<void*> dst;
          for (int k = k0; k < k1; ++k)
            dst.push_back((char*)const_cast<void*>(pv.user[(size_t)k]) + off + (size_t)me * per_rank);
          return dst;
        };
        p.exec = [=](const PeerView& pv, hipStream_t s) {
          if (!pv.zero_copy) {
            const auto segs = pulls(pv);
            MCCL_CHECK(mccl_copy_segments(segs.data(), W, s));
            return;
          }
          // between barrier kernels: plain one-to-many copies, eight destinations per launch
          mccl_xsync_t none{};
          none.n = 1;
          for (int k0 = 0; k0 < W; k0 += MCCL_FUSED_MAX_RANKS) {
            const auto dst = destinations(pv, k0, std::min(W, k0 + MCCL_FUSED_MAX_RANKS));
            MCCL_CHECK(mccl_fanout_sync(in, dst.data(), (int)dst.size(), len, &none, s));
          }
        };
        p.compact_cost = 1.0;
        p.one_launch_any_size = true;
        p.exec_sync_in_place_only = true;
        p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
          const auto dst = destinations(pv, 0, W);
          MCCL_CHECK(mccl_fanout_sync(in, dst.data(), W, len, &sync, s));
          return true;
        };
      } else {
        p.share = len >= kZeroCopyMinBytes;  // the inputs are read in place by the peers
        p.share_ptr = touchesForeignSlice(input.data_ptr(), per_rank, output.data_ptr(), per_rank, W, me) ? nullptr : in;
        p.share_bytes = len;
        p.exec = [=](const PeerView& pv, hipStream_t s) {
          const auto segs = pulls(pv);
          MCCL_CHECK(mccl_copy_segments(segs.data(), W, s));
        };
        p.compact_cost = 2.0 * (double)size_;
        p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
          const auto segs = pulls(pv);
          MCCL_CHECK(mccl_copy_segments_sync(segs.data(), W, MCCL_COPY_SHARED_SOURCES, &sync, s));
          return true;
        };
      }
    }
    work = run(p);
    off += len;
  } while (off < per_rank);
  return work;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::allgather(std::vector<std::vector<at::Tensor>>& outputs,
                                                          std::vector<at::Tensor>& inputs,
                                                          const c10d::AllgatherOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::allgather", std::vector<c10::IValue>({inputs}));
  TORCH_CHECK(inputs.size() == 1 && outputs.size() == 1,
              "CCL process group does not support tensors count ", inputs.size());
  TORCH_CHECK((int)outputs[0].size() == size_, "allgather: number of output tensors should equal to the world size");
  std::vector<at::Tensor> all = outputs[0];
  all.push_back(inputs[0]);
  checkDeviceTensors(all);
  at::Tensor input = inputs[0];
  std::vector<at::Tensor> outs = outputs[0];
  const size_t mine = nbytes(input);
  size_t largest = mine;
  for (const auto& o : outs) largest = std::max(largest, nbytes(o));  // what each rank sends: known everywhere
  if (largest > stage_max_) {
    // more than one staging window: one (windowed) broadcast per rank, straight into outs[r]
    c10::intrusive_ptr<c10d::Work> last;
    for (int r = 0; r < size_; ++r) {
      c10d::BroadcastOptions bo;
      bo.rootRank = r;
      bo.rootTensor = 0;
      if (r == rank_) {
        TORCH_CHECK(mine == nbytes(outs[(size_t)r]), "allgather: output tensor ", r, " does not match the size rank ", r, " sends");
        std::vector<at::Tensor> v{input};
        last = broadcast(v, bo);
        hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(input.get_device()).stream();
        copyAsync(outs[(size_t)r].data_ptr(), input.data_ptr(), mine, cur);
      } else {
        std::vector<at::Tensor> v{outs[(size_t)r]};
        last = broadcast(v, bo);
      }
    }
    return last;
  }
  Plan p;
  p.op = c10d::OpType::ALLGATHER;
  p.title = "allgather";
  p.inputs = {input};
  p.outputs = outs;
  p.stage_bytes = mine;
  p.table = {(int64_t)mine};
  const int W = size_;
  if (mine)
    p.copy_in = [=](void* stage, hipStream_t s) {
      copyAsync(stage, input.data_ptr(), mine, s);
    };
  // Large inputs are read in place by the peers.  `largest` is what the longest contribution of
  // the group measures, which every rank knows from its output list: the offer is the same everywhere.
  p.share = largest >= kZeroCopyMinBytes;
  p.share_ptr = mine ? input.data_ptr() : nullptr;
  // (an input that one of this rank's outputs overlaps, other than as the very tensor it is gathered
  // into: not offered, the peers would read it while this rank's copies write over it)
  for (size_t r = 0; r < outs.size() && p.share_ptr; ++r)
    if (rangesOverlap(input.data_ptr(), mine, outs[r].data_ptr(), nbytes(outs[r])) && !((int)r == rank_ && outs[r].data_ptr() == input.data_ptr()))
      p.share_ptr = nullptr;
  p.share_bytes = mine;
  auto pulls = [=](const PeerView& pv) {
    std::vector<mccl_segment_t> segs;
    for (int r = 0; r < W; ++r) {
      const size_t b = (size_t)pv.tables[(size_t)r][0];  // allgatherv: every rank announces its byte count
      TORCH_CHECK(b == nbytes(outs[(size_t)r]), "allgather: output tensor ", r, " does not match the size rank ", r, " sends");
      if (b) segs.push_back({pv.zero_copy ? pv.user[(size_t)r] : pv.stage[(size_t)r], outs[(size_t)r].data_ptr(), b});
    }
    return segs;
  };
  p.exec = [=](const PeerView& pv, hipStream_t s) {
    const auto segs = pulls(pv);
    MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
  };
  p.compact_cost = 2.0 * (double)size_;
  p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
    const auto segs = pulls(pv);
    MCCL_CHECK(mccl_copy_segments_sync(segs.data(), (int)segs.size(), MCCL_COPY_SHARED_SOURCES, &sync, s));
    return true;
  };
  return run(p);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::allgather_coalesced(std::vector<std::vector<at::Tensor>>&,
                                                                    std::vector<at::Tensor>&,
                                                                    const c10d::AllgatherOptions&) {
  TORCH_CHECK(false, "ProcessGroupCCL does not support allgather_coalesced");
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::allgather_into_tensor_coalesced(
    std::vector<at::Tensor>& outputs, std::vector<at::Tensor>& inputs, const c10d::AllgatherOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::allgather_into_tensor_coalesced", std::vector<c10::IValue>({inputs}));
  TORCH_CHECK(outputs.size() == inputs.size(), "allgather_into_tensor_coalesced: list sizes differ");
  checkDeviceTensors(inputs);
  std::vector<size_t> offs(inputs.size());
  size_t total = 0;
  for (size_t i = 0; i < inputs.size(); ++i) {
    checkDeviceTensors({outputs[i], inputs[i]});
    TORCH_CHECK(inputs[i].numel() * size_ == outputs[i].numel(),
                "output tensor size must be equal to world_size times input tensor size");
    offs[i] = total;
    total += roundUp(nbytes(inputs[i]), 16);
  }
  if (total > stage_max_) {  // more than one staging window: one (windowed) all-gather per tensor
    c10::intrusive_ptr<c10d::Work> last;
    for (size_t i = 0; i < inputs.size(); ++i) last = _allgather_base(outputs[i], inputs[i], c10d::AllgatherOptions());
    return last;
  }
  Plan p;
  p.op = c10d::OpType::ALLGATHER_COALESCED;
  p.title = "allgather_into_tensor_coalesced";
  p.inputs = inputs;
  p.outputs = outputs;
  p.stage_bytes = total;
  std::vector<at::Tensor> ins = inputs, outs = outputs;
  const int W = size_;
  p.copy_in = [=](void* stage, hipStream_t s) {
    std::vector<mccl_segment_t> segs;
    for (size_t i = 0; i < ins.size(); ++i)
      if (ins[i].numel()) segs.push_back({ins[i].data_ptr(), (char*)stage + offs[i], nbytes(ins[i])});
    MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
  };
  p.exec = [=](const PeerView& pv, hipStream_t s) {
    std::vector<mccl_segment_t> segs;
    for (size_t i = 0; i < ins.size(); ++i) {
      const size_t b = nbytes(ins[i]);
      if (!b) continue;
      for (int r = 0; r < W; ++r)
        segs.push_back({(const char*)pv.stage[(size_t)r] + offs[i], (char*)outs[i].data_ptr() + (size_t)r * b, b});
    }
    MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
  };
  return run(p);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::_reduce_scatter_base(at::Tensor& output, at::Tensor& input,
                                                                     const c10d::ReduceScatterOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::_reduce_scatter_base", std::vector<c10::IValue>({input}));
  checkDeviceTensors({output, input});
  TORCH_CHECK(input.numel() == output.numel() * size_,
              "input tensor must be the same size as output size times world size");
  const int dtype = dtypeCode(output.scalar_type());
  const int op = opCode(opts.reduceOp, output.scalar_type());
  const size_t es = output.element_size();
  const size_t M = (size_t)output.numel();
  const int W = size_;
  // one window holds the same sub-range [m0, m0+len) of all W shards, back to back
  const size_t chunk = std::max<size_t>(1, stage_max_ / es / (size_t)W);
  c10::intrusive_ptr<c10d::Work> work;
  size_t m0 = 0;
  do {
    const size_t len = std::min(M - m0, chunk);
    Plan p;
    p.op = c10d::OpType::_REDUCE_SCATTER_BASE;
    p.title = "_reduce_scatter_base";
    p.inputs = {input};
    p.outputs = {output};
    if (len) {
      p.stage_bytes = len * es * (size_t)W;
      char* in = (char*)input.data_ptr();
      char* out = (char*)output.data_ptr() + m0 * es;
      const int me = rank_;
      p.copy_in = [=](void* stage, hipStream_t s) {
        if (len == M) {
          copyAsync(stage, in, M * es * (size_t)W, s);
        } else {
          std::vector<mccl_segment_t> segs((size_t)W);
          for (int k = 0; k < W; ++k)
            segs[(size_t)k] = {in + ((size_t)k * M + m0) * es, (char*)stage + (size_t)k * len * es, len * es};
          MCCL_CHECK(mccl_copy_segments(segs.data(), W, s));
        }
      };
      // One window, at most eight ranks: no rendezvous.  What the peers address is this rank's whole
      // input (rank r reads slice r of everybody's); a rank that stages copies its input first,
      // which is also how an output inside another rank's slice of the input is handled.
      if (len == M) {
        p.standing.ok = true;
        p.standing.buffer = in;
        p.standing.bytes = M * es * (size_t)W;
        p.standing.copy_in = true;
        p.standing.force_staged = touchesForeignSlice(output.data_ptr(), M * es, in, M * es, W, me);
        p.standing.compact_cost = 0.5;
        p.standing.behind_barrier = [=](const void* resolved, bool, const mccl_xsync_t& sync, hipStream_t s) {
          MCCL_CHECK(mccl_reduce_sync_resolved(resolved, (size_t)me * M * es, out, M, dtype, op, &sync, s));
        };
        p.standing.one_launch = [=](bool, const mccl_xsync_t& sync, const mccl_offer_t& mine, const void* buffer, void* const* offers,
                                    const mccl_import_table_t* imports, hipStream_t s) {
          MCCL_CHECK(mccl_reduce_sync_offers((size_t)me * M * es, out, M, dtype, op, &sync, &mine, buffer, offers, imports, s));
        };
      }
      // large inputs are read in place by the peers: rank r reduces slice r of every rank's tensor
      p.share = len * es * (size_t)W >= kZeroCopyMinBytes;
      // (an output inside another rank's slice of the input: nothing is offered, and then every rank stages)
      p.share_ptr = touchesForeignSlice(output.data_ptr(), M * es, in, M * es, W, me) ? nullptr : in;
      p.share_bytes = M * es * (size_t)W;
      p.exec = [=](const PeerView& pv, hipStream_t s) {
        void* o = out;
        if (pv.zero_copy) {
          std::vector<const void*> src((size_t)W);
          for (int k = 0; k < W; ++k) src[(size_t)k] = (const char*)pv.user[(size_t)k] + ((size_t)me * M + m0) * es;
          MCCL_CHECK(mccl_reduce_n(src.data(), W, o, len, dtype, op, MCCL_VARIANT_AUTO, s));
        } else {
          MCCL_CHECK(mccl_reduce_scatter_n(pv.stage.data(), W, &o, len, me, 1, dtype, op, s));
        }
      };
      p.compact_cost = 0.5;
      p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
        std::vector<const void*> src((size_t)W);
        for (int k = 0; k < W; ++k)  // in place: slice `me` of rank k's tensor; staged: slice `me` of the window rank k staged
          src[(size_t)k] = pv.zero_copy ? (const char*)pv.user[(size_t)k] + ((size_t)me * M + m0) * es
                                        : (const char*)pv.stage[(size_t)k] + (size_t)me * len * es;
        MCCL_CHECK(mccl_reduce_sync(src.data(), out, len, dtype, op, &sync, s));
        return true;
      };
    }
    work = run(p);
    m0 += len;
  } while (m0 < M);
  return work;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::reduce_scatter(std::vector<at::Tensor>& outputs,
                                                               std::vector<std::vector<at::Tensor>>& inputs,
                                                               const c10d::ReduceScatterOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::reduce_scatter", std::vector<c10::IValue>({outputs}));
  TORCH_CHECK(outputs.size() == 1 && inputs.size() == 1,
              "CCL process group does not support tensors count ", outputs.size());
  TORCH_CHECK((int)inputs[0].size() == size_, "reduce_scatter: number of input tensors should equal to the world size");
  std::vector<at::Tensor> all = inputs[0];
  all.push_back(outputs[0]);
  checkDeviceTensors(all);
  at::Tensor out = outputs[0];
  std::vector<at::Tensor> ins = inputs[0];
  const int dtype = dtypeCode(out.scalar_type());
  const int op = opCode(opts.reduceOp, out.scalar_type());
  const int W = size_;
  const int me = rank_;
  // Slot d of every rank's list is reduced into rank d's output; slots may differ in size
  // (the reference degrades to W rooted reduces then, src/gpu/dpcpp_ccl.cpp:952-964).  The
  // staging image is the list packed back to back; the table announces offset and size per slot.
  Plan p;
  p.op = c10d::OpType::REDUCE_SCATTER;
  p.title = "reduce_scatter";
  p.inputs = ins;
  p.outputs = {out};
  p.table.resize((size_t)(2 * W));
  const FlatSpan span = flatSpan(ins);
  size_t total = 0, payload = 0, padded = 0;
  std::vector<size_t> offs((size_t)W);
  for (int d = 0; d < W; ++d) {
    offs[(size_t)d] = total;
    p.table[(size_t)d] = (int64_t)total;
    p.table[(size_t)(W + d)] = (int64_t)nbytes(ins[(size_t)d]);
    payload += nbytes(ins[(size_t)d]);
    padded += roundUp(nbytes(ins[(size_t)d]), 16);
    // a flat list is its own image; any other is packed with each slot on a 16-byte boundary
    total += span.flat ? nbytes(ins[(size_t)d]) : roundUp(nbytes(ins[(size_t)d]), 16);
  }
  if (padded > stage_max_) {  // (the padded size: the same on every rank, flat list or not)
    // more than one staging window: W (windowed) rooted reduces, as the reference does for slots of
    // unequal size.  The root reduces in place in its output, which first takes its own slot.
    c10::intrusive_ptr<c10d::Work> last;
    for (int d = 0; d < W; ++d) {
      c10d::ReduceOptions ro;
      ro.reduceOp = opts.reduceOp;
      ro.rootRank = d;
      ro.rootTensor = 0;
      if (d == me) {
        TORCH_CHECK(nbytes(out) == nbytes(ins[(size_t)d]), "reduce_scatter: output tensor does not match slot ", d);
        hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(out.get_device()).stream();
        copyAsync(out.data_ptr(), ins[(size_t)d].data_ptr(), nbytes(out), cur);
        std::vector<at::Tensor> v{out};
        last = reduce(v, ro);
      } else {
        std::vector<at::Tensor> v{ins[(size_t)d]};  // only staged: a non-root tensor keeps its values
        last = reduce(v, ro);
      }
    }
    return last;
  }
  p.stage_bytes = total;
  p.copy_in = [=](void* stage, hipStream_t s) {
    std::vector<mccl_segment_t> segs;
    for (int d = 0; d < W; ++d)
      if (ins[(size_t)d].numel())
        segs.push_back({ins[(size_t)d].data_ptr(), (char*)stage + offs[(size_t)d], nbytes(ins[(size_t)d])});
    MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
  };
  // A large list that is one range of memory (src/utils.cpp:157-193) is read in place by the
  // peers.  The offer depends on the unpadded size of the list, which is the same on every rank
  // of a valid call; a rank whose list is not flat offers nothing, and then every rank stages.
  p.share = payload >= kZeroCopyMinBytes;
  p.share_ptr = span.flat ? span.ptr : nullptr;
  p.share_bytes = span.flat ? span.bytes : payload;
  auto sources = [=](const PeerView& pv) {
    std::vector<const void*> in((size_t)W);
    for (int k = 0; k < W; ++k) {
      TORCH_CHECK((size_t)pv.tables[(size_t)k][W + me] == nbytes(out),
                  "reduce_scatter: rank ", k, "'s input for rank ", me, " does not match the output size");
      in[(size_t)k] = (const char*)(pv.zero_copy ? pv.user[(size_t)k] : pv.stage[(size_t)k]) + pv.tables[(size_t)k][me];
    }
    return in;
  };
  p.exec = [=](const PeerView& pv, hipStream_t s) {
    const auto in = sources(pv);
    if (out.numel())
      MCCL_CHECK(mccl_reduce_n(in.data(), W, out.data_ptr(), (size_t)out.numel(), dtype, op, MCCL_VARIANT_AUTO, s));
  };
  p.compact_cost = 0.5;
  p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
    const auto in = sources(pv);
    MCCL_CHECK(mccl_reduce_sync(in.data(), out.data_ptr(), (size_t)out.numel(), dtype, op, &sync, s));
    return true;
  };
  return run(p);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::reduce_scatter_tensor_coalesced(
    std::vector<at::Tensor>& outputs, std::vector<at::Tensor>& inputs, const c10d::ReduceScatterOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::reduce_scatter_tensor_coalesced", std::vector<c10::IValue>({inputs}));
  TORCH_CHECK(outputs.size() == inputs.size(), "reduce_scatter_tensor_coalesced: list sizes differ");
  checkDeviceTensors(inputs);
  checkDeviceTensors(outputs);
  TORCH_CHECK(inputs[0].scalar_type() == outputs[0].scalar_type(), "Tensors are not equal in data type");
  const int dtype = dtypeCode(outputs[0].scalar_type());
  const int op = opCode(opts.reduceOp, outputs[0].scalar_type());
  std::vector<size_t> offs(inputs.size());
  size_t total = 0;
  for (size_t i = 0; i < inputs.size(); ++i) {
    TORCH_CHECK(inputs[i].numel() == outputs[i].numel() * size_,
                "input tensor must be the same size as output size times world size");
    offs[i] = total;
    total += roundUp(nbytes(inputs[i]), 16);
  }
  if (total > stage_max_) {  // more than one staging window: one (windowed) reduce-scatter per tensor
    c10::intrusive_ptr<c10d::Work> last;
    c10d::ReduceScatterOptions one;
    one.reduceOp = opts.reduceOp;
    for (size_t i = 0; i < inputs.size(); ++i) last = _reduce_scatter_base(outputs[i], inputs[i], one);
    return last;
  }
  Plan p;
  p.op = c10d::OpType::COALESCED;
  p.title = "reduce_scatter_tensor_coalesced";
  p.inputs = inputs;
  p.outputs = outputs;
  p.stage_bytes = total;
  std::vector<at::Tensor> ins = inputs, outs = outputs;
  const int W = size_;
  const int me = rank_;
  p.copy_in = [=](void* stage, hipStream_t s) {
    std::vector<mccl_segment_t> segs;
    for (size_t i = 0; i < ins.size(); ++i)
      if (ins[i].numel()) segs.push_back({ins[i].data_ptr(), (char*)stage + offs[i], nbytes(ins[i])});
    MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
  };
  p.exec = [=](const PeerView& pv, hipStream_t s) {
    std::vector<const void*> in;
    std::vector<void*> out;
    std::vector<size_t> counts;
    for (size_t i = 0; i < ins.size(); ++i) {
      if (!outs[i].numel()) continue;
      const size_t shard = nbytes(outs[i]);
      for (int k = 0; k < W; ++k) in.push_back((const char*)pv.stage[(size_t)k] + offs[i] + (size_t)me * shard);
      out.push_back(outs[i].data_ptr());
      counts.push_back((size_t)outs[i].numel());
    }
    MCCL_CHECK(mccl_reduce_multi(in.data(), W, out.data(), counts.data(), (int)out.size(), dtype, op, s));
  };
  return run(p);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::alltoall_base(at::Tensor& output, at::Tensor& input,
                                                              std::vector<int64_t>& outputSplitSizes,
                                                              std::vector<int64_t>& inputSplitSizes,
                                                              const c10d::AllToAllOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::alltoall_base", std::vector<c10::IValue>({input}));
  checkDeviceTensors({output, input});
  const int W = size_;
  const int me = rank_;
  const size_t es = input.element_size();
  std::vector<size_t> send((size_t)W), recv((size_t)W);
  if (outputSplitSizes.empty() && inputSplitSizes.empty()) {
    // src/gpu/dpcpp_ccl.cpp:1384-1390
    TORCH_CHECK(output.numel() == input.numel() && output.scalar_type() == input.scalar_type(),
                "alltoall_base: tensors are not equal in size or data type");
    TORCH_CHECK(output.size(0) % W == 0, "alltoall_base: tensor's dim 0 does not divide equally across group size");
    const size_t c = (size_t)output.numel() / (size_t)W * es;
    for (int i = 0; i < W; ++i) send[(size_t)i] = recv[(size_t)i] = c;
  } else {
    // count arithmetic of src/gpu/dpcpp_ccl.cpp:1431-1445
    c10d::checkSplitSizes(inputSplitSizes, input, W);
    c10d::checkSplitSizes(outputSplitSizes, output, W);
    const bool in_equal = inputSplitSizes.empty(), out_equal = outputSplitSizes.empty();
    size_t in_len = (size_t)input.numel(), out_len = (size_t)output.numel();
    if (in_len) in_len /= (in_equal ? (size_t)W : (size_t)input.size(0));
    if (out_len) out_len /= (out_equal ? (size_t)W : (size_t)output.size(0));
    for (int i = 0; i < W; ++i) {
      send[(size_t)i] = (in_equal ? in_len : (size_t)inputSplitSizes[(size_t)i] * in_len) * es;
      recv[(size_t)i] = (out_equal ? out_len : (size_t)outputSplitSizes[(size_t)i] * out_len) * es;
    }
  }
  std::vector<size_t> send_displ((size_t)W);
  std::vector<void*> dst((size_t)W);
  size_t displ = 0, roff = 0;
  for (int d = 0; d < W; ++d) {  // displacements = exclusive prefix sums of the counts
    send_displ[(size_t)d] = displ;
    dst[(size_t)d] = (char*)output.data_ptr() + roff;
    displ += send[(size_t)d];
    roff += recv[(size_t)d];
  }
  ExchangeImage image;
  image.flat = nbytes(input) ? input.data_ptr() : nullptr;
  image.offs = std::move(send_displ);
  image.sizes = std::move(send);
  image.total = nbytes(input);
  return exchange(c10d::OpType::ALLTOALL_BASE, "alltoall_base", {input}, {output}, image, dst, recv);
}

// The all-to-all engine behind alltoall_base and alltoall.  Every rank has an image -- W pieces,
// piece d for rank d, at image.offs[d] -- that is either a range of the caller's memory
// (image.flat: the peers read it in place when every rank can share) or packed into the staging
// buffer from image.pieces by the copy-in (the pack of src/gpu/dpcpp_ccl.cpp:1505-1515).  A rank pulls
// piece `me` of every image straight to dst[r] (which is the unpack, :1528-1538).
//
// Images larger than one staging window travel in windows: window w holds bytes
// [w * window, (w + 1) * window) of every rank's image, and a rank pulls the part of each of its
// pieces that lies inside.  How many windows there are depends on the largest image of the
// group, which every rank learns from the tables of the first window.
//
// The images differ in size and kind from rank to rank, so the zero-copy offer cannot depend on
// either: every exchange offers (a packed image offers nothing, and then every rank stages).
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::exchange(c10d::OpType op, const char* title,
                                                          const std::vector<at::Tensor>& inputs,
                                                          const std::vector<at::Tensor>& outputs,
                                                          const ExchangeImage& image, const std::vector<void*>& dst,
                                                          const std::vector<size_t>& recv) {
  const int W = size_;
  const int me = rank_;
  const bool is_base = op == c10d::OpType::ALLTOALL_BASE;
  const size_t total = image.total;
  auto nwin = std::make_shared<size_t>(1);
  const size_t window = stage_max_;
  c10::intrusive_ptr<c10d::Work> work;
  for (size_t w = 0; w < *nwin; ++w) {
    const size_t w0 = w * window, w1 = w0 + window;
    const size_t wlen = w0 < total ? std::min(total - w0, window) : 0;
    Plan p;
    p.op = op;
    p.title = title;
    p.inputs = inputs;
    p.outputs = outputs;
    p.stage_bytes = wlen;
    p.table.resize((size_t)(2 * W + 1));
    for (int d = 0; d < W; ++d) {
      p.table[(size_t)d] = (int64_t)image.offs[(size_t)d];
      p.table[(size_t)(W + d)] = (int64_t)image.sizes[(size_t)d];
    }
    p.table[(size_t)(2 * W)] = (int64_t)total;
    p.share = true;
    p.share_ptr = image.flat;  // null with total > 0: a packed image, which cannot be shared
    // (nor can an image that a destination of this rank overlaps: the peers would read it while this
    // rank's copies write over it; staged, the copy-in comes first)
    for (size_t d = 0; d < dst.size() && p.share_ptr; ++d)
      if (rangesOverlap(image.flat, total, dst[d], recv[d])) p.share_ptr = nullptr;
    p.share_bytes = total;
    if (wlen) {
      if (image.flat) {
        const char* flat = (const char*)image.flat;
        p.copy_in = [=](void* stage, hipStream_t s) { copyAsync(stage, flat + w0, wlen, s); };
      } else {
        const std::vector<at::Tensor> pieces = image.pieces;
        const std::vector<size_t> offs = image.offs;
        p.copy_in = [=](void* stage, hipStream_t s) {
          std::vector<mccl_segment_t> segs;
          for (int d = 0; d < W; ++d) {  // the part of piece d that lies inside the window
            const size_t lo = std::max(offs[(size_t)d], w0), hi = std::min(offs[(size_t)d] + nbytes(pieces[(size_t)d]), w1);
            if (lo < hi)
              segs.push_back({(const char*)pieces[(size_t)d].data_ptr() + (lo - offs[(size_t)d]), (char*)stage + (lo - w0), hi - lo});
          }
          if (!segs.empty()) MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
        };
      }
    }
    // the segments this rank pulls in this window (and, from the tables, how many windows there are)
    auto pulls = [=](const PeerView& pv) {
      size_t largest = 0;
      std::vector<mccl_segment_t> segs;
      for (int r = 0; r < W; ++r) {
        const int64_t* tr = pv.tables[(size_t)r];
        if (is_base) {
          TORCH_CHECK((size_t)tr[W + me] == recv[(size_t)r],
                      "alltoall_base: rank ", r, " sends ", tr[W + me], " bytes to rank ", me,
                      " which expects ", recv[(size_t)r]);
        } else {
          TORCH_CHECK((size_t)tr[W + me] == recv[(size_t)r], "alltoall: output tensor ", r,
                      " does not match what rank ", r, " sends");
        }
        largest = std::max(largest, (size_t)tr[2 * W]);
        // the piece addressed to this rank inside rank r's image, cut to the window
        const size_t seg0 = (size_t)tr[me], seg1 = seg0 + recv[(size_t)r];
        const size_t lo = std::max(seg0, w0), hi = std::min(seg1, w1);
        if (lo < hi)
          segs.push_back({pv.zero_copy ? (const char*)pv.user[(size_t)r] + lo : (const char*)pv.stage[(size_t)r] + (lo - w0),
                          (char*)dst[(size_t)r] + (lo - seg0), hi - lo});
      }
      *nwin = std::max<size_t>(1, (largest + window - 1) / window);
      return segs;
    };
    p.exec = [=](const PeerView& pv, hipStream_t s) {
      const auto segs = pulls(pv);
      if (!segs.empty()) MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
    };
    p.exec_sync = [=](const PeerView& pv, mccl_xsync_t& sync, hipStream_t s) {
      const auto segs = pulls(pv);
      MCCL_CHECK(mccl_copy_segments_sync(segs.data(), (int)segs.size(), 0u, &sync, s));  // empty: still takes part in the waits
      return true;
    };
    work = run(p);
  }
  return work;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::alltoall(std::vector<at::Tensor>& outputs,
                                                         std::vector<at::Tensor>& inputs,
                                                         const c10d::AllToAllOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::alltoall", std::vector<c10::IValue>({inputs}));
  TORCH_CHECK((int)inputs.size() == size_ && (int)outputs.size() == size_,
              "alltoall: number of input and output tensors should equal to the world size");
  std::vector<at::Tensor> all = inputs;
  all.insert(all.end(), outputs.begin(), outputs.end());
  checkDeviceTensors(all);
  const int W = size_;
  // A list whose tensors are consecutive views of one storage is an image already (the flat check
  // of src/utils.cpp:157-215, used at src/gpu/dpcpp_ccl.cpp:1499-1504): no pack, and the peers can
  // read it in place.  Any other list is packed by the copy-in, each piece on a 16-byte boundary.
  ExchangeImage image;
  image.sizes.resize((size_t)W);
  image.offs.resize((size_t)W);
  const FlatSpan span = flatSpan(inputs);
  size_t total = 0;
  for (int d = 0; d < W; ++d) {
    image.sizes[(size_t)d] = nbytes(inputs[(size_t)d]);
    image.offs[(size_t)d] = total;
    total += span.flat ? image.sizes[(size_t)d] : roundUp(image.sizes[(size_t)d], 16);
  }
  image.total = total;
  if (span.flat) image.flat = span.ptr;
  else image.pieces = inputs;
  std::vector<void*> dst((size_t)W);
  std::vector<size_t> recv((size_t)W);
  for (int r = 0; r < W; ++r) {
    dst[(size_t)r] = outputs[(size_t)r].data_ptr();
    recv[(size_t)r] = nbytes(outputs[(size_t)r]);
  }
  return exchange(c10d::OpType::ALLTOALL, "alltoall", inputs, outputs, image, dst, recv);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::barrier(const c10d::BarrierOptions& /*opts*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::barrier", std::vector<c10::IValue>{});
  Plan p;
  p.op = c10d::OpType::BARRIER;
  p.title = "barrier";
  p.host_complete = true;
  auto work = run(p);
  // a barrier returns once every rank has arrived: nothing is pending on the stream
  return work;
}

// Rooted reduction (XPUCCLStubs::reduce_, src/gpu/dpcpp_ccl.cpp:820-857): every rank stages its
// tensor, the root runs the N-buffer reduction into its own; the other ranks' tensors keep their
// values.
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::reduce(std::vector<at::Tensor>& tensors,
                                                       const c10d::ReduceOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::reduce", std::vector<c10::IValue>({tensors}));
  checkRank((int)opts.rootRank, size_);
  TORCH_CHECK(tensors.size() == 1, "CCL process group does not support tensors count ", tensors.size());
  checkDeviceTensors(tensors);
  at::Tensor t = tensors[0];
  const int dtype = dtypeCode(t.scalar_type());
  const int op = opCode(opts.reduceOp, t.scalar_type());
  const int root = (int)opts.rootRank;
  const size_t es = t.element_size();
  const size_t total = (size_t)t.numel();
  const size_t chunk = stage_max_ / es;
  c10::intrusive_ptr<c10d::Work> work;
  size_t off = 0;
  do {
    const size_t len = std::min(total - off, chunk);
    char* base = total ? (char*)t.data_ptr() + off * es : nullptr;
    Plan p;
    p.op = c10d::OpType::REDUCE;
    p.title = "reduce";
    p.inputs = {t};
    p.outputs = {t};
    if (size_ > 1 && len) {
      const int W = size_;
      p.stage_bytes = len * es;
      p.copy_in = [=](void* stage, hipStream_t s) { copyAsync(stage, base, len * es, s); };
      if (rank_ == root)
        p.exec = [=](const PeerView& pv, hipStream_t s) {
          std::vector<const void*> in = pv.stage;
          in[(size_t)root] = base;  // in place on the root's tensor, as in allreduce
          MCCL_CHECK(mccl_reduce_n(in.data(), W, base, len, dtype, op, MCCL_VARIANT_AUTO, s));
        };
    }
    work = run(p);
    off += len;
  } while (off < total);
  return work;
}

// gather (XPUCCLStubs::gather_, src/gpu/dpcpp_ccl.cpp:1237-1299): every rank stages its tensor and
// announces its size; the root copies all of them into its output list in one launch.
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::gather(std::vector<std::vector<at::Tensor>>& outputs,
                                                       std::vector<at::Tensor>& inputs,
                                                       const c10d::GatherOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::gather", std::vector<c10::IValue>({inputs}));
  checkRank((int)opts.rootRank, size_);
  TORCH_CHECK(inputs.size() == 1, "CCL process group does not support tensors count ", inputs.size());
  const int root = (int)opts.rootRank;
  std::vector<at::Tensor> outs;
  if (rank_ != root) {
    TORCH_CHECK(outputs.size() == 0, "gather: number of output tensors should be 0 for non-root");
    checkDeviceTensors(inputs);
  } else {
    TORCH_CHECK(outputs.size() == 1, "gather: multi-GPU collective is not supported");
    TORCH_CHECK((int)outputs[0].size() == size_, "gather: number of output tensors should equal to the world size");
    outs = outputs[0];
    std::vector<at::Tensor> all = outs;
    all.push_back(inputs[0]);
    checkDeviceTensors(all);
  }
  at::Tensor input = inputs[0];
  const size_t mine = nbytes(input);
  if (mine > stage_max_) {
    // more than one staging window: point to point (every rank sends the same number of bytes,
    // src/gpu/dpcpp_ccl.cpp:1270-1289)
    if (rank_ != root) return send(inputs, root, 0);
    std::vector<c10::intrusive_ptr<c10d::Work>> pending;
    for (int r = 0; r < size_; ++r) {
      TORCH_CHECK(nbytes(outs[(size_t)r]) == mine, "gather: output tensor ", r, " does not match the size rank ", r, " sends");
      if (r == root) continue;
      std::vector<at::Tensor> v{outs[(size_t)r]};
      pending.push_back(recv(v, r, 0));
    }
    hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(input.get_device()).stream();
    copyAsync(outs[(size_t)root].data_ptr(), input.data_ptr(), mine, cur);
    for (auto& w : pending) w->wait();
    return c10::make_intrusive<WorkCCL>(rank_, c10d::OpType::GATHER, "gather", std::vector<at::Tensor>{input}, outs, blocking_wait_);
  }
  Plan p;
  p.op = c10d::OpType::GATHER;
  p.title = "gather";
  p.inputs = {input};
  p.outputs = outs;
  p.stage_bytes = mine;
  p.table = {(int64_t)mine};
  const int W = size_;
  if (mine) p.copy_in = [=](void* stage, hipStream_t s) { copyAsync(stage, input.data_ptr(), mine, s); };
  if (rank_ == root)
    p.exec = [=](const PeerView& pv, hipStream_t s) {
      std::vector<mccl_segment_t> segs;
      for (int r = 0; r < W; ++r) {
        const size_t b = (size_t)pv.tables[(size_t)r][0];
        TORCH_CHECK(b == nbytes(outs[(size_t)r]), "gather: output tensor ", r, " does not match the size rank ", r, " sends");
        if (b) segs.push_back({pv.stage[(size_t)r], outs[(size_t)r].data_ptr(), b});
      }
      MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
    };
  return run(p);
}

// scatter (XPUCCLStubs::scatter_, src/gpu/dpcpp_ccl.cpp:1301-1369): the root stages its input list
// back to back and announces where each piece lies; every rank pulls its own piece.
c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::scatter(std::vector<at::Tensor>& outputs,
                                                        std::vector<std::vector<at::Tensor>>& inputs,
                                                        const c10d::ScatterOptions& opts) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::scatter", std::vector<c10::IValue>({outputs}));
  checkRank((int)opts.rootRank, size_);
  const int root = (int)opts.rootRank;
  const int W = size_;
  std::vector<at::Tensor> ins;
  if (rank_ == root) {
    if (inputs.size() != 1) {
      std::ostringstream ss;
      ss << "ProcessGroupCCL::scatter: requires a single-element input list containing a list with " << W << " tensors.";
      C10_THROW_ERROR(ValueError, ss.str());
    }
    if ((int)inputs[0].size() != W) {
      std::ostringstream ss;
      ss << "ProcessGroupCCL::scatter: Incorrect input list size " << inputs[0].size()
         << ". Input list size should be " << W << ", same as size of the process group.";
      C10_THROW_ERROR(ValueError, ss.str());
    }
    ins = inputs[0];
  } else {
    TORCH_CHECK(inputs.size() == 0, "scatter: number of input tensors should be 0 for non-root");
  }
  TORCH_CHECK(outputs.size() == 1, "CCL process group does not support tensors count ", outputs.size());
  std::vector<at::Tensor> all = ins;
  all.push_back(outputs[0]);
  checkDeviceTensors(all);
  at::Tensor out = outputs[0];
  // Every rank receives the same number of bytes (src/gpu/dpcpp_ccl.cpp:1341-1359), so all ranks
  // know the size of the root's staging image from their own output.  More than one staging
  // window: point to point.
  if ((size_t)(W - 1) * roundUp(nbytes(out), 16) > stage_max_) {
    if (rank_ != root) return recv(outputs, root, 0);
    for (int r = 0; r < W; ++r) {
      TORCH_CHECK(nbytes(ins[(size_t)r]) == nbytes(out), "scatter: input tensor ", r, " does not match the size rank ", r, " receives");
      if (r == root) continue;
      std::vector<at::Tensor> v{ins[(size_t)r]};
      send(v, r, 0);
    }
    hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(out.get_device()).stream();
    copyAsync(out.data_ptr(), ins[(size_t)root].data_ptr(), nbytes(out), cur);
    return c10::make_intrusive<WorkCCL>(rank_, c10d::OpType::SCATTER, "scatter", ins, std::vector<at::Tensor>{out}, blocking_wait_);
  }
  Plan p;
  p.op = c10d::OpType::SCATTER;
  p.title = "scatter";
  p.inputs = ins;
  p.outputs = {out};
  const int me = rank_;
  if (rank_ == root) {
    // staging image: the W pieces back to back, each on a 16-byte boundary; table = W offsets, W sizes
    std::vector<size_t> offs((size_t)W);
    size_t total = 0;
    p.table.assign((size_t)(2 * W), 0);
    for (int r = 0; r < W; ++r) {
      offs[(size_t)r] = total;
      p.table[(size_t)r] = (int64_t)total;
      p.table[(size_t)(W + r)] = (int64_t)nbytes(ins[(size_t)r]);
      if (r != root) total += roundUp(nbytes(ins[(size_t)r]), 16);  // the root's own piece is not staged
    }
    TORCH_CHECK(total <= stage_max_, "ccl backend: scatter larger than the staging window");
    TORCH_CHECK(nbytes(ins[(size_t)root]) == nbytes(out), "scatter: output tensor does not match the size the root sends");
    p.stage_bytes = total;
    p.copy_in = [=](void* stage, hipStream_t s) {
      std::vector<mccl_segment_t> segs;
      for (int r = 0; r < W; ++r)
        if (r != root && ins[(size_t)r].numel())
          segs.push_back({ins[(size_t)r].data_ptr(), (char*)stage + offs[(size_t)r], nbytes(ins[(size_t)r])});
      if (!segs.empty()) MCCL_CHECK(mccl_copy_segments(segs.data(), (int)segs.size(), s));
    };
    p.exec = [=](const PeerView& pv, hipStream_t s) {
      copyAsync(out.data_ptr(), ins[(size_t)root].data_ptr(), nbytes(out), s);
    };
  } else {
    p.exec = [=](const PeerView& pv, hipStream_t s) {
      const size_t b = (size_t)pv.tables[(size_t)root][W + me];
      TORCH_CHECK(b == nbytes(out), "scatter: output tensor does not match the size the root sends");
      copyAsync(out.data_ptr(), (const char*)pv.stage[(size_t)root] + pv.tables[(size_t)root][me], b, s);
    };
  }
  return run(p);
}
// ---------------------------------------------------------------------------------------------
// point to point
// ---------------------------------------------------------------------------------------------
void ProcessGroupCCL::spinUntil(const std::function<bool()>& ready, int peer, const char* what,
                                const std::function<bool()>& abandoned, const std::function<void()>& idle,
                                std::chrono::milliseconds limit_override) {
  // a wait(timeout) of the caller's wins over the group's limit
  const std::chrono::milliseconds limit = limit_override.count() > 0 ? limit_override : waitLimit(false);
  const auto deadline = std::chrono::steady_clock::now() + limit;
  unsigned spins = 0;
  while (!ready()) {
    if (ctl_->slot[peer].failed.load(std::memory_order_acquire))
      TORCH_CHECK(false, "ccl backend: rank ", peer, " reported a failure while this rank was waiting for ", what);
    if (ctl_->slot[peer].departed.load(std::memory_order_acquire) && abandoned() && !ready()) {
      ctl_->slot[rank_].failed.store(1, std::memory_order_release);
      TORCH_CHECK(false, "ccl backend: rank ", peer, " left the group while this rank was waiting for ", what);
    }
    if (idle) idle();
    if (++spins < 2000) continue;
    sched_yield();
    if ((spins & 0x3ff) == 0 && std::chrono::steady_clock::now() > deadline) {
      ctl_->slot[rank_].failed.store(1, std::memory_order_release);
      TORCH_CHECK(false, "ccl backend: timed out waiting for ", what, " (rank ", peer, ")");
    }
  }
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::send(std::vector<at::Tensor>& tensors, int dstRank, int /*tag*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::send", std::vector<c10::IValue>({tensors}));
  checkRank(dstRank, size_);
  TORCH_CHECK(tensors.size() == 1, "CCL process group does not support tensors count ", tensors.size());
  checkDeviceTensors(tensors);
  at::Tensor t = tensors[0];
  std::lock_guard<std::mutex> lock(mutex_);
  c10::DeviceGuard dev_guard(t.device());
  ensureInit(t.get_device());
  hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA((c10::DeviceIndex)device_).stream();
  P2PBox& box = ctl_->slot[rank_].p2p[dstRank];
  P2PSend& mine = p2p_send_[(size_t)dstRank];
  const size_t total = nbytes(t);
  size_t off = 0;
  do {  // an empty tensor still travels as one (empty) message, so that sends and receives pair up
    const size_t len = std::min(total - off, stage_max_);
    const uint64_t k = box.posted.load(std::memory_order_relaxed) + 1;
    spinUntil([&] { return k - box.consumed.load(std::memory_order_acquire) <= (uint64_t)kRing; }, dstRank,
              "a free send buffer", [] { return true; },
              [&] {  // while waiting, take in what others have sent to this rank's posted receives
                for (int src = 0; src < size_; ++src)
                  if (!p2p_recv_[(size_t)src].pending.empty()) progressRecvLocked(src, nullptr, /*blocking=*/false);
              });
    const int slot = (int)((k - 1) % kRing);
    P2PEntry& e = box.ring[slot];
    if (len > mine.capacity[slot]) {
      size_t cap = kP2PMinBytes;
      while (cap < len) cap <<= 1;
      void* base = nullptr;
      HIP_CHECK(hipMalloc(&base, cap));
      if (mine.base[slot]) retired_.push_back(mine.base[slot]);  // the receiver may still hold a mapping
      mine.base[slot] = base;
      mine.capacity[slot] = cap;
      if (size_ > 1) HIP_CHECK(hipIpcGetMemHandle(&e.handle, base));
      e.ptr = (uint64_t)(uintptr_t)base;
      e.capacity = cap;
      e.gen += 1;
    }
    if (len) {
      copyAsync(mine.base[slot], (const char*)t.data_ptr() + off, len, cur);
      HIP_CHECK(hipStreamSynchronize(cur));  // the message is published only once it is complete
    }
    e.bytes = len;
    box.posted.store(k, std::memory_order_release);
    off += len;
  } while (off < total);
  // the data has left the tensor: nothing is pending
  return c10::make_intrusive<WorkCCL>(rank_, c10d::OpType::SEND, "send", std::vector<at::Tensor>{t},
                                      std::vector<at::Tensor>{}, blocking_wait_);
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::recv(std::vector<at::Tensor>& tensors, int srcRank, int /*tag*/) {
  RECORD_FUNCTION("oneccl_bindings_for_pytorch::recv", std::vector<c10::IValue>({tensors}));
  checkRank(srcRank, size_);
  TORCH_CHECK(tensors.size() == 1, "CCL process group does not support tensors count ", tensors.size());
  checkDeviceTensors(tensors);
  auto state = std::make_shared<RecvState>();
  state->tensor = tensors[0];
  state->src = srcRank;
  {
    std::lock_guard<std::mutex> lock(mutex_);
    c10::DeviceGuard dev_guard(state->tensor.device());
    ensureInit(state->tensor.get_device());
    P2PRecv& pr = p2p_recv_[(size_t)srcRank];
    const size_t total = nbytes(state->tensor);
    const uint64_t nmsg = total ? (total + stage_max_ - 1) / stage_max_ : 1;
    state->next_seq = pr.assigned + 1;
    pr.assigned += nmsg;
    pr.pending.push_back(state);
  }
  auto self = c10::intrusive_ptr<ProcessGroupCCL>::unsafe_reclaim_from_nonowning(this);
  return c10::make_intrusive<RecvWorkCCL>(std::move(self), std::move(state), rank_);
}

void ProcessGroupCCL::progressRecv(int src, const RecvState* target, bool blocking, std::chrono::milliseconds limit) {
  std::lock_guard<std::mutex> lock(mutex_);
  progressRecvLocked(src, target, blocking, limit);
}

void ProcessGroupCCL::progressRecvLocked(int src, const RecvState* target, bool blocking, std::chrono::milliseconds limit) {
  if (target && target->done) return;
  c10::DeviceGuard guard(c10::Device(at::kCUDA, (c10::DeviceIndex)device_));
  hipStream_t cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA((c10::DeviceIndex)device_).stream();
  P2PBox& box = ctl_->slot[src].p2p[rank_];
  P2PRecv& pr = p2p_recv_[(size_t)src];
  while (!pr.pending.empty()) {
    std::shared_ptr<RecvState> st = pr.pending.front();
    const size_t total = nbytes(st->tensor);
    // message by message; what has arrived is kept when a non-blocking call has to stop half way
    for (bool finished = false; !finished;) {
      const uint64_t k = st->next_seq;
      if (box.posted.load(std::memory_order_acquire) < k) {
        if (!blocking) return;
        spinUntil([&] { return box.posted.load(std::memory_order_acquire) >= k; }, src, "a message",
                  [&] { return box.posted.load(std::memory_order_acquire) < k; },
                  [&] {  // meanwhile, whatever other ranks have sent to receives posted here
                    for (int other = 0; other < size_; ++other)
                      if (other != src && !p2p_recv_[(size_t)other].pending.empty())
                        progressRecvLocked(other, nullptr, /*blocking=*/false);
                  }, limit);
      }
      const size_t len = std::min(total - st->off, stage_max_);
      const int slot = (int)((k - 1) % kRing);
      const P2PEntry& e = box.ring[slot];
      if (e.bytes != len) {
        // The two sides disagree about the message stream: drop the message and the receive, and
        // flag the group as failed (what follows on this pair can no longer be matched reliably).
        // The error belongs to this receive: its own wait() raises it, whichever call got here.
        const uint64_t have = e.bytes;
        box.consumed.store(k, std::memory_order_release);
        const std::string why = c10::str("ccl backend: recv expects ", len, " bytes from rank ", src,
                                         " but the message holds ", have);
        st->error = std::make_exception_ptr(std::runtime_error(why));
        st->done = true;
        pr.pending.pop_front();
        ctl_->slot[rank_].failed.store(1, std::memory_order_release);
        shared_->fail(why);
        if (st.get() == target) std::rethrow_exception(st->error);
        break;  // go on with the next posted receive of this source
      }
      if (len) {
        const void* from = nullptr;
        if (ctl_->slot[src].pid == (int64_t)getpid()) {
          from = (const void*)(uintptr_t)e.ptr;
        } else {
          if (pr.gen[slot] != e.gen) {
            if (pr.ipc[slot] && pr.base[slot]) (void)hipIpcCloseMemHandle(pr.base[slot]);
            pr.base[slot] = nullptr;
            pr.ipc[slot] = false;
            void* m = nullptr;
            HIP_CHECK(hipIpcOpenMemHandle(&m, e.handle, hipIpcMemLazyEnablePeerAccess));
            pr.base[slot] = m;
            pr.ipc[slot] = true;
            pr.gen[slot] = e.gen;
          }
          from = pr.base[slot];
        }
        TORCH_CHECK(!ctl_->slot[src].failed.load(std::memory_order_acquire),
                    "ccl backend: rank ", src, " gave up on a message before it was received");
        copyAsync((char*)st->tensor.data_ptr() + st->off, from, len, cur);
        HIP_CHECK(hipStreamSynchronize(cur));  // the sender may reuse the buffer once `consumed` moves
      }
      box.consumed.store(k, std::memory_order_release);
      st->next_seq = k + 1;
      st->off += len;
      finished = st->off >= total;
    }
    if (st->error) continue;  // dropped above
    st->done = true;
    pr.pending.pop_front();
    if (st.get() == target) return;
  }
}

ProcessGroupCCL::RecvWorkCCL::RecvWorkCCL(c10::intrusive_ptr<ProcessGroupCCL> pg, std::shared_ptr<RecvState> state,
                                          int rank)
    : c10d::Work(rank, c10d::OpType::RECV, "recv"), pg_(std::move(pg)), state_(std::move(state)) {}

bool ProcessGroupCCL::RecvWorkCCL::isCompleted() {
  if (!state_->done) {
    try {
      pg_->progressRecv(state_->src, state_.get(), /*blocking=*/false);
    } catch (...) {
      if (!state_->error) throw;  // this receive's own failure is reported by wait() / exception()
    }
  }
  return state_->done;
}

bool ProcessGroupCCL::RecvWorkCCL::isSuccess() const { return !state_->error; }

std::exception_ptr ProcessGroupCCL::RecvWorkCCL::exception() const { return state_->error; }

void ProcessGroupCCL::RecvWorkCCL::synchronize() { wait(kNoTimeout); }

bool ProcessGroupCCL::RecvWorkCCL::wait(std::chrono::milliseconds timeout) {
  if (!state_->done) pg_->progressRecv(state_->src, state_.get(), /*blocking=*/true, timeout);
  if (state_->error) std::rethrow_exception(state_->error);
  return true;
}

std::vector<at::Tensor> ProcessGroupCCL::RecvWorkCCL::result() { return {state_->tensor}; }

c10::intrusive_ptr<c10::ivalue::Future> ProcessGroupCCL::RecvWorkCCL::getFuture() {
  if (!future_) {
    synchronize();  // the host has waited for the copy: the tensor is ready for any stream
    future_ = c10::make_intrusive<at::ivalue::Future>(c10::ListType::create(c10::TensorType::get()));
    future_->markCompleted(at::IValue(std::vector<at::Tensor>{state_->tensor}));
  }
  return future_;
}

c10::intrusive_ptr<c10d::Work> ProcessGroupCCL::recvAnysource(std::vector<at::Tensor>&, int) {
  TORCH_CHECK(false, "ProcessGroupCCL does not support recvAnysource");
}

}  // namespace mccl_pg
