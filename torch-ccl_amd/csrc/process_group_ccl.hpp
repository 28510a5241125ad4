// c10d backend "ccl" for ROCm tensors on one MI355X: the host-side mirror of the reference's
// ProcessGroupCCL (src/ProcessGroupCCL.hpp:111-310) over the C ABI of include/mccl.h.
//
// Single-GPU mode: every rank of the group (a process, or a thread of one process) uses
// device 0.  Each rank owns two staging buffers in HBM.  A collective
//   1. copies (or packs) the caller's input into the rank's staging buffer   [device copy]
//   2. waits, on the host, until every rank has finished step 1              [barrier]
//   3. runs the local-reduce / pull kernel over the N ranks' staging buffers,
//      writing straight into the caller's output tensor                      [the hot path]
// which is the structure of the reference's IPC allreduce (copy-in, cross-rank barrier, sum of
// the N peer buffers: src/gpu/allreduce_small.h:166-361).  Peers' staging buffers are reached
// through hipIpcOpenMemHandle (other processes) or directly (threads of the same process); the
// handles, a host barrier and small per-collective tables live in a POSIX shared-memory control
// block whose name is published through the c10d Store (the role of
// src/ccl_comm_collector.cpp:10-45 and src/gpu/allreduce.h:1208-1248).
// A staging buffer is at most 1 GiB (shared allocations stay well below 2 GiB); longer messages
// travel in windows.  Point-to-point messages use a mailbox per ordered pair of ranks in the same
// control block (see send / recv below).
#pragma once

#include <hip/hip_runtime_api.h>
#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Utils.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>

#include <chrono>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace mccl_pg {

struct Control;  // shared-memory control block (process_group_ccl.cpp)

class ProcessGroupCCL : public c10d::Backend {
 public:
  // Stream-ordered Work (the contract of XPUWorkCCL, src/gpu/dpcpp_ccl.cpp:382-472): the op is
  // complete when `end_` has fired on the communication stream; wait() makes the caller's current
  // stream wait for it, or blocks the host when CCL_BLOCKING_WAIT=1.
  class WorkCCL : public c10d::Work {
   public:
    WorkCCL(int rank, c10d::OpType op, const char* title, std::vector<at::Tensor> inputs,
            std::vector<at::Tensor> outputs, bool blocking_wait);
    ~WorkCCL() override;
    bool isCompleted() override;
    bool isSuccess() const override;
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    void synchronize() override;
    std::vector<at::Tensor> result() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

   private:
    friend class ProcessGroupCCL;
    hipEvent_t end_ = nullptr;
    int device_ = 0;
    bool blocking_wait_ = false;
    std::vector<at::Tensor> inputs_;   // held until the Work dies (ownership rule of the reference)
    std::vector<at::Tensor> outputs_;
    c10::intrusive_ptr<c10::ivalue::Future> future_;
  };

  // What a posted receive still has to do; the group keeps these per source in posting order.
  struct RecvState {
    at::Tensor tensor;
    int src = 0;
    uint64_t next_seq = 0;  // sequence number (from 1) of the next message of this receive
    size_t off = 0;         // bytes of the tensor already filled (a long tensor travels as several messages)
    bool done = false;
  };

  // Work of a receive (XPUP2PAsyncWork of the reference, src/gpu/dpcpp_ccl.cpp:1590-1627).  The
  // message is matched and copied out when somebody waits for it (or polls isCompleted once the
  // sender has published it): no progress thread runs behind the caller's back.
  class RecvWorkCCL : public c10d::Work {
   public:
    RecvWorkCCL(c10::intrusive_ptr<ProcessGroupCCL> pg, std::shared_ptr<RecvState> state, int rank);
    bool isCompleted() override;
    bool isSuccess() const override { return true; }
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    void synchronize() override;
    std::vector<at::Tensor> result() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

   private:
    c10::intrusive_ptr<ProcessGroupCCL> pg_;  // a pending receive keeps its group alive
    std::shared_ptr<RecvState> state_;
    c10::intrusive_ptr<c10::ivalue::Future> future_;
  };

  static constexpr int64_t OP_TIMEOUT_MILLIS = 10 * 1000;  // src/ProcessGroupCCL.cpp:876

  ProcessGroupCCL(const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
                  std::chrono::milliseconds timeout);
  ~ProcessGroupCCL() override;

  static c10::intrusive_ptr<c10d::Backend> create(const c10::intrusive_ptr<c10d::Store>& store,
                                                  int rank, int size,
                                                  std::chrono::milliseconds timeout);

  const std::string getBackendName() const override { return "ccl"; }
  bool supportsCoalescing() const override { return true; }
  void startCoalescing() override;
  c10::intrusive_ptr<c10d::Work> endCoalescing() override;
  void setTimeout(std::chrono::milliseconds t) override { timeout_ = t; }
  void setSequenceNumberForGroup() override {}
  uint64_t getSequenceNumberForGroup() override { return seq_; }

  c10::intrusive_ptr<c10d::Work> broadcast(std::vector<at::Tensor>& tensors,
                                           const c10d::BroadcastOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> allreduce(std::vector<at::Tensor>& tensors,
                                           const c10d::AllreduceOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> allreduce_coalesced(
      std::vector<at::Tensor>& tensors, const c10d::AllreduceCoalescedOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> allgather(std::vector<std::vector<at::Tensor>>& outputs,
                                           std::vector<at::Tensor>& inputs,
                                           const c10d::AllgatherOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> _allgather_base(at::Tensor& output, at::Tensor& input,
                                                 const c10d::AllgatherOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> allgather_coalesced(
      std::vector<std::vector<at::Tensor>>& outputs, std::vector<at::Tensor>& inputs,
      const c10d::AllgatherOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> allgather_into_tensor_coalesced(
      std::vector<at::Tensor>& outputs, std::vector<at::Tensor>& inputs,
      const c10d::AllgatherOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> reduce_scatter(std::vector<at::Tensor>& outputs,
                                                std::vector<std::vector<at::Tensor>>& inputs,
                                                const c10d::ReduceScatterOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> _reduce_scatter_base(at::Tensor& output, at::Tensor& input,
                                                      const c10d::ReduceScatterOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> reduce_scatter_tensor_coalesced(
      std::vector<at::Tensor>& outputs, std::vector<at::Tensor>& inputs,
      const c10d::ReduceScatterOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> alltoall_base(at::Tensor& output, at::Tensor& input,
                                               std::vector<int64_t>& outputSplitSizes,
                                               std::vector<int64_t>& inputSplitSizes,
                                               const c10d::AllToAllOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> alltoall(std::vector<at::Tensor>& outputs,
                                          std::vector<at::Tensor>& inputs,
                                          const c10d::AllToAllOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> barrier(const c10d::BarrierOptions& opts) override;

  // Rooted forms over the same kernels: the root reduces / pulls, the others only stage.
  c10::intrusive_ptr<c10d::Work> reduce(std::vector<at::Tensor>& tensors, const c10d::ReduceOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> gather(std::vector<std::vector<at::Tensor>>& outputs, std::vector<at::Tensor>& inputs,
                                        const c10d::GatherOptions& opts) override;
  c10::intrusive_ptr<c10d::Work> scatter(std::vector<at::Tensor>& outputs, std::vector<std::vector<at::Tensor>>& inputs,
                                         const c10d::ScatterOptions& opts) override;
  // Point to point: a send copies the tensor into one of a few staging buffers kept per
  // destination and publishes it; it returns as soon as the data has left the tensor and blocks
  // only while all of those buffers hold unconsumed messages.  A receive is matched in posting
  // order per source when it is waited for.  The tag is ignored, as in the reference.
  c10::intrusive_ptr<c10d::Work> send(std::vector<at::Tensor>& tensors, int dstRank, int tag) override;
  c10::intrusive_ptr<c10d::Work> recv(std::vector<at::Tensor>& tensors, int srcRank, int tag) override;
  // Not supported by the reference either (src/ProcessGroupCCL.cpp:1217-1222).
  c10::intrusive_ptr<c10d::Work> recvAnysource(std::vector<at::Tensor>&, int) override;

 private:
  // What one collective needs from the engine.
  struct Plan {
    c10d::OpType op = c10d::OpType::UNKNOWN;
    const char* title = "";
    std::vector<at::Tensor> inputs;
    std::vector<at::Tensor> outputs;
    size_t stage_bytes = 0;                 // bytes this rank puts into its staging buffer
    std::vector<int64_t> table;             // per-collective scalars published to the peers
    // enqueue the copy-in on `s`; `stage` is this rank's staging buffer
    std::function<void(void* stage, hipStream_t s)> copy_in;
    // enqueue the data-path kernels on `s`; peer[r] is rank r's staging buffer,
    // tables[r] the scalars rank r published
    std::function<void(const std::vector<const void*>& peer,
                       const std::vector<const int64_t*>& tables, hipStream_t s)> exec;
    // optional second phase: runs after every rank has finished `exec` (one more stream
    // synchronisation and host barrier); used by the two-shot allreduce
    std::function<void(const std::vector<const void*>& peer,
                       const std::vector<const int64_t*>& tables, hipStream_t s)> exec2;
  };

  c10::intrusive_ptr<c10d::Work> run(Plan& plan);
  void ensureInit(int device);
  void* ensureStage(int slot, size_t bytes);
  // start_up: the first barrier of a group, which also absorbs the ranks' different start-up
  // times: at least two minutes, and not shortened by MCCL_BARRIER_TIMEOUT_MS
  void hostBarrier(bool start_up = false);
  const void* peerStage(int peer, int slot);
  void checkDeviceTensors(const std::vector<at::Tensor>& tensors) const;
  // Spins (then yields) until ready() holds; raises when `peer` reports a failure, when it has
  // left and abandoned() says that what is awaited can no longer come, or at the time limit.
  // `idle`, when given, runs between polls (a send that waits for a free buffer uses it to
  // complete this rank's own posted receives, so that ranks sending round a ring cannot block
  // each other for good).
  void spinUntil(const std::function<bool()>& ready, int peer, const char* what,
                 const std::function<bool()>& abandoned, const std::function<void()>& idle = nullptr);
  // Completes the receives posted for `src` in order, up to and including `target` (all of them
  // when target is null).  With blocking == false it stops at the first message the sender has
  // not published yet.  progressRecv takes the group's mutex, the Locked form expects it held.
  void progressRecv(int src, const RecvState* target, bool blocking);
  void progressRecvLocked(int src, const RecvState* target, bool blocking);

  c10::intrusive_ptr<c10d::Store> store_;
  std::chrono::milliseconds timeout_;
  bool blocking_wait_ = false;  // CCL_BLOCKING_WAIT
  bool same_stream_ = false;    // CCL_SAME_STREAM
  bool verbose_ = false;        // ONECCL_BINDINGS_FOR_PYTORCH_ENV_VERBOSE
  bool profile_ = false;        // MCCL_PG_PROFILE: host-side phase timers, printed when the group dies
  size_t stage_max_ = 0;        // bytes of one staging window (1 GiB; MCCL_STAGE_WINDOW_BYTES shrinks it for tests)
  // per collective with a payload: copy-in enqueue, stream synchronise, host barrier, kernel enqueue
  std::vector<float> phase_us_[4];
  bool coalescing_ = false;
  c10::intrusive_ptr<WorkCCL> last_work_;  // only kept between startCoalescing and endCoalescing
  std::mutex mutex_;  // one collective of a group at a time (the reference serialises on a global mutex)

  bool initialised_ = false;
  int device_ = 0;
  hipStream_t comm_stream_ = nullptr;
  hipEvent_t fork_event_ = nullptr;
  // End of the previous collective's device work and the stream it ran on.  A collective that runs
  // on another stream waits for it on the host before its barrier, so that "every earlier kernel of
  // this rank has finished reading the peers' staging buffers" holds whichever streams were used.
  hipEvent_t tail_event_ = nullptr;
  hipStream_t tail_stream_ = nullptr;
  bool tail_pending_ = false;
  uint64_t seq_ = 0;
  uint64_t barrier_epoch_ = 0;

  Control* ctl_ = nullptr;
  size_t ctl_bytes_ = 0;
  std::string shm_name_;

  struct Stage {
    void* base = nullptr;  // the allocation
    void* ptr = nullptr;   // where this rank's data starts (staggered by rank inside the allocation)
    size_t capacity = 0;
  };
  Stage stage_[2];
  std::vector<void*> retired_;  // outgrown staging buffers, freed with the group

  struct PeerMap {
    void* base[2] = {nullptr, nullptr};  // mapping of the peer's allocation (what gets closed)
    void* ptr[2] = {nullptr, nullptr};   // the peer's data inside it
    uint64_t gen[2] = {0, 0};
    bool ipc[2] = {false, false};
  };
  std::vector<PeerMap> peers_;

  // point to point
  static constexpr int kP2PRing = 4;
  struct P2PSend {  // per destination: this rank's staging buffers
    void* base[kP2PRing] = {nullptr, nullptr, nullptr, nullptr};
    size_t capacity[kP2PRing] = {0, 0, 0, 0};
  };
  struct P2PRecv {  // per source
    uint64_t assigned = 0;  // messages handed to posted receives so far
    std::deque<std::shared_ptr<RecvState>> pending;
    void* base[kP2PRing] = {nullptr, nullptr, nullptr, nullptr};  // mappings of the sender's buffers
    uint64_t gen[kP2PRing] = {0, 0, 0, 0};
    bool ipc[kP2PRing] = {false, false, false, false};
  };
  std::vector<P2PSend> p2p_send_;
  std::vector<P2PRecv> p2p_recv_;
};

}  // namespace mccl_pg
