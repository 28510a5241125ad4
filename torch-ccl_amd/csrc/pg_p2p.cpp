// c10d backend "ccl" for ROCm tensors: point to point.
#include "pg_internal.hpp"

namespace mccl_pg {

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
