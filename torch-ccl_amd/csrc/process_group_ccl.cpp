// c10d backend "ccl" for ROCm tensors: the group, its Works, and how a collective runs (see process_group_ccl.hpp for the design).
#include "pg_internal.hpp"

namespace mccl_pg {

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
    if (status[0] != 0 && status[1] == MCCL_STATUS_MISMATCH) {
      os << "ccl backend: alltoall: the piece rank " << (status[0] - 1) << " sends to this rank does not have the length this rank "
            "expects (the split sizes of the ranks do not match: outputSplitSizes[r] here must equal rank r's inputSplitSizes "
            "for this rank); the group cannot be used any more";
    } else if (status[0] != 0 && status[1] == MCCL_STATUS_UNMAPPED) {
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
// construction, rendezvous
// ---------------------------------------------------------------------------------------------
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
  for (auto& in : outbox_in_)
    if (in.base) (void)hipIpcCloseMemHandle(in.base);
  for (auto& out : outbox_out_)
    if (out.base) (void)hipFree(out.base);
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
    for (int sl = 0; sl < 2; ++sl) {
      offer_slots_[sl].assign((size_t)size_, nullptr);
      offer_rows_[sl].assign((size_t)size_, nullptr);
    }
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
        offer_rows_[sl][(size_t)r] = base + kArenaOfferRowOff + (size_t)sl * kArenaOfferRowStride;
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
    if (plan.standing_exchange.ok) {
      runStandingExchange(plan, s, slot, seq);
      if (timed) phase_us_[3].push_back((float)us_since(t0));
      return;
    }
    if (staticStagedFits(plan)) {
      runStaticStaged(plan, s, slot, seq);
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

}  // namespace mccl_pg
