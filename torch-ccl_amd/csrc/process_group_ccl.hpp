// c10d backend "ccl" for ROCm tensors on one MI355X: the host-side mirror of the reference's
// ProcessGroupCCL (src/ProcessGroupCCL.hpp:111-310) over the C ABI of include/mccl.h.
//
// Single-GPU mode: every rank of the group (a process, or a thread of one process) uses
// device 0.  A collective is the structure of the reference's IPC allreduce (copy-in, cross-rank
// barrier, sum of the N peer buffers: src/gpu/allreduce_small.h:166-361):
//   1. the peers get to see this rank's input: a copy (or pack) into the rank's staging buffer
//      in HBM, or -- for large single-tensor collectives whose tensors the peers can map -- the
//      caller's tensor itself (the reference hands the user buffer to the IPC exchange the same
//      way, src/gpu/allreduce.h:1214-1224);
//   2. a cross-rank barrier;
//   3. the local-reduce / pull kernel over the N ranks' buffers, writing straight into the
//      caller's output tensor                                                [the hot path]
// When the ranks are processes of their own, step 2 is a flag kernel on the collective's stream
// (mccl_rank_barrier): no host thread waits for the GPU and no stream is synchronised, so a
// collective only enqueues work.  Allreduces of up to 1 MiB are one kernel that does all three
// steps (mccl_allreduce_fused).  Ranks that are threads of one process share streams and hardware
// queues, where a waiting kernel could block the kernel it waits for: they keep the host barrier
// (hipStreamSynchronize + a spin on the control block), which MCCL_PG_SYNC=host also selects.
// Peers' buffers are reached through hipIpcOpenMemHandle (other processes) or directly (threads of
// the same process); the handles, the host rendezvous and small per-collective tables live in a
// POSIX shared-memory control block whose name is published through the c10d Store (the role of
// src/ccl_comm_collector.cpp:10-45 and src/gpu/allreduce.h:1208-1248).
// A staging buffer is at most 1 GiB (shared allocations stay well below 2 GiB); longer messages
// travel in windows.  Point-to-point messages use a mailbox per ordered pair of ranks in the same
// control block (see send / recv below).
#pragma once

#include <hip/hip_runtime_api.h>

#include "mccl.h"
#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Utils.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>

#include <atomic>
#include <chrono>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <tuple>
#include <vector>

namespace mccl_pg {

struct Control;  // shared-memory control block (pg_internal.hpp)

// What the Works of a group share with it and may outlive it with: recycled events and the
// group's health.  `status` is pinned host memory the device-side waits write when they give up:
// words 0-1 (1 + the late rank, the epoch) for the barrier and the one-launch collectives, words
// 2-3 the same for the one-launch small allreduce, whose epochs are counted on the device and in a
// numbering of their own; `failed` is raised by the host side.
struct GroupShared {
  std::mutex mutex;
  std::vector<hipEvent_t> free_events;
  volatile uint32_t* status = nullptr;
  std::atomic<bool> failed{false};
  std::string failure;  // guarded by mutex
  int device = 0;

  hipEvent_t getEvent();
  void putEvent(hipEvent_t e);
  // Non-empty once a device-side wait has timed out or the host side has given up.
  std::string failureMessage();
  void fail(const std::string& why);
  ~GroupShared();
};

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
    // false once the group has failed (a peer did not arrive in time, a rank reported a failure);
    // exception() then carries the reason (src/ProcessGroupCCL.cpp:866-869)
    bool isSuccess() const override;
    std::exception_ptr exception() const override;
    // Non-blocking mode: the caller's stream waits for the collective.  CCL_BLOCKING_WAIT=1: the
    // host waits, at most `timeout` (the group's timeout when kNoTimeout is passed), and raises
    // "Caught collective operation timeout" like the reference (src/utils.h:295-319).  Both raise
    // when the group has failed.
    bool wait(std::chrono::milliseconds timeout = kNoTimeout) override;
    void synchronize() override;
    std::vector<at::Tensor> result() override;
    c10::intrusive_ptr<c10::ivalue::Future> getFuture() override;

   private:
    friend class ProcessGroupCCL;
    void waitInternal(std::chrono::milliseconds timeout);
    void orderCurrentStreamAfter();
    hipEvent_t end_ = nullptr;      // recorded after the collective, when it ran on the communication stream
    hipStream_t stream_ = nullptr;  // the stream the collective ran on
    bool stream_set_ = false;
    std::shared_ptr<GroupShared> shared_;
    std::chrono::milliseconds op_timeout_{0};
    std::chrono::steady_clock::time_point start_;
    int device_ = 0;
    bool blocking_wait_ = false;
    int pending_polls_ = 0;  // > 0: isCompleted() says "not yet" this many more times, < 0: for good (pendingWork)
    // Recorded into a HIP graph under stream capture: nothing has been enqueued, the stream must not
    // be queried, and when the work runs is up to whoever replays the graph.
    bool captured_ = false;
    std::vector<at::Tensor> inputs_;   // held until the Work dies (ownership rule of the reference)
    std::vector<at::Tensor> outputs_;
    c10::intrusive_ptr<c10::ivalue::Future> future_;
  };

  // A Work that is not backed by device work: it completes after `polls` calls of isCompleted()
  // (never, when polls < 0).  For exercising wait(timeout) without a GPU.
  static c10::intrusive_ptr<c10d::Work> pendingWork(int rank, int polls, std::chrono::milliseconds op_timeout);

  // What a posted receive still has to do; the group keeps these per source in posting order.
  struct RecvState {
    at::Tensor tensor;
    int src = 0;
    uint64_t next_seq = 0;  // sequence number (from 1) of the next message of this receive
    size_t off = 0;         // bytes of the tensor already filled (a long tensor travels as several messages)
    bool done = false;
    std::exception_ptr error;  // why the receive failed; raised by its own wait(), whoever progressed it
  };

  // Work of a receive (XPUP2PAsyncWork of the reference, src/gpu/dpcpp_ccl.cpp:1590-1627).  The
  // message is matched and copied out when somebody waits for it (or polls isCompleted once the
  // sender has published it): no progress thread runs behind the caller's back.
  class RecvWorkCCL : public c10d::Work {
   public:
    RecvWorkCCL(c10::intrusive_ptr<ProcessGroupCCL> pg, std::shared_ptr<RecvState> state, int rank);
    bool isCompleted() override;
    bool isSuccess() const override;
    std::exception_ptr exception() const override;
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
  // What the data-path kernels of one collective get to see of the peers.
  struct PeerView {
    std::vector<const void*> stage;         // rank r's staging buffer (this process's mapping)
    std::vector<const int64_t*> tables;     // the scalars rank r published
    bool zero_copy = false;                 // the peers' tensors are read in place: nothing was staged
    std::vector<const void*> user;          // zero_copy: rank r's published tensor range
  };
  using ExecFn = std::function<void(const PeerView& pv, hipStream_t s)>;
  // The whole device side of a zero-copy collective as ONE launch with the rank waits inside the
  // kernel (mccl_*_sync).  Returns false when the collective does not fit that form; the engine then
  // runs barrier kernels around exec / exec2.
  using SyncExecFn = std::function<bool(const PeerView& pv, mccl_xsync_t& sync, hipStream_t s)>;

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
    // enqueue the data-path kernels on `s`
    ExecFn exec;
    // optional second phase: runs after every rank has finished `exec` (one more barrier);
    // used by the two-shot allreduce.  two_phase, when set, says whether this run needs it.
    ExecFn exec2;
    std::function<bool(const PeerView& pv)> two_phase;
    SyncExecFn exec_sync;
    // Zero-copy offer (device-synchronised groups only): the byte range of the caller's tensor
    // that the peers may read in place of a staged copy.  `share` must come out the same on every
    // rank (it may depend on sizes all ranks agree on, never on this rank's own).  The offer is
    // taken when every rank of the group can share its range (an allocation of torch's caching
    // allocator below 2 GiB); copy_in is then skipped, exec / exec2 run with pv.zero_copy set, and
    // a closing barrier keeps every rank from touching its tensor before all peers have read it.
    bool share = false;
    const void* share_ptr = nullptr;
    size_t share_bytes = 0;
    size_t zero_copy_stage_bytes = 0;       // staging this rank still needs in zero-copy mode
    bool exec_sync_in_place_only = false;   // exec_sync writes into the peers' tensors: not for staged runs
    bool one_launch_any_size = false;       // exec_sync wins at every size: the default one-launch limit does not apply
    // What a byte of share_bytes / stage_bytes costs exec_sync's launch, in bytes of a plain copy's
    // traffic (read + write): 2 for a pull, 2 W for an allgather (W times the input is read and
    // written), less for reductions, whose wavefronts keep eight loads in flight each.  Decides up to
    // which size a launch limited to few compute units beats a barrier kernel and a full grid.
    double compact_cost = 2.0;
    // Eligible for the one-launch small allreduce (device-synchronised groups of at most 8 ranks):
    // no staging slot, no table, no rendezvous.  The staged plan above stays as the fallback.
    bool fused_ok = false;
    void* fused_ptr = nullptr;
    size_t fused_count = 0;
    int fused_dtype = 0;
    int fused_op = 0;
    // Eligible for the path that exchanges where the ranks' buffers are on the device and never meets
    // on the host (runStanding): what this rank's peers address, and the kernels over the resolved
    // addresses.  `ok` and `bytes` must come out the same on every rank (sizes all ranks agree on).
    struct Standing {
      bool ok = false;
      void* buffer = nullptr;      // the tensor the peers read (allreduce, reduce_scatter: the input) or write (all_gather: the output)
      size_t bytes = 0;
      // the storage (one block of the allocator) the buffer is part of: what is announced to the peers, so
      // that a view somewhere inside a larger tensor is read in place like any other
      const void* block = nullptr;
      size_t block_bytes = 0;
      bool copy_in = false;        // a rank that stages copies its tensor into the staging buffer first ...
      bool copy_out = false;       // ... and / or the staging buffer back into it afterwards
      bool force_staged = false;   // this rank's tensors overlap in a way only a staged run handles (its own matter: the peers do not care)
      double compact_cost = 1.0;   // as Plan::compact_cost: up to which size ONE launch on few compute units wins
      // the data kernel behind the barrier kernel that resolved the offers into `resolved`
      std::function<void(const void* resolved, bool staged, const mccl_xsync_t& sync, hipStream_t s)> behind_barrier;
      // one launch that exchanges the offers itself
      std::function<void(bool staged, const mccl_xsync_t& sync, const mccl_offer_t& mine, const void* buffer,
                         void* const* offers, const mccl_import_table_t* imports, hipStream_t s)> one_launch;
    } standing;
    // An all-to-all on the same footing (runStandingExchange): a rank offers every reader its own piece.
    // `ok` depends on the group alone; the sizes differ from rank to rank and decide nothing that more
    // than the two ranks of a pair have to agree on.
    struct StandingExchange {
      bool ok = false;
      std::vector<const void*> piece;  // where this rank's piece for rank d is
      std::vector<size_t> send;        // its length
      // the storage (one block of the allocator) the piece is part of: what can be announced to the peers
      // (small ones are not worth it)
      std::vector<const void*> block;
      std::vector<size_t> block_bytes;
      std::vector<void*> dst;          // where rank r's piece for this rank goes
      std::vector<size_t> recv;        // its length
      bool force_staged = false;       // input and output overlap: every piece is copied out of the way first
      // all_gather into a list, broadcast: every reader gets the SAME piece, and every rank knows how long
      // every rank's piece is (`unanimous_bytes`: the longest).  A rank that cannot offer it in place copies
      // it into its staging buffer once, as in runStanding, instead of into an outbox per reader.
      bool same_piece = false;
      size_t unanimous_bytes = 0;
      // reduce_scatter from a list: what arrives is not copied to dst but reduced, by this kernel over the
      // resolved addresses (rank r's piece for this rank, this rank's own included)
      std::function<void(const void* resolved, const mccl_xsync_t& sync, hipStream_t s)> reduce;
    } standing_exchange;
    // Everything this collective needs of its peers is in their staging buffers, at places every rank
    // computes for itself (the shapes of a coalesced call agree across ranks): exec reads pv.stage and
    // nothing else of pv.  Between rank processes such a collective needs no rendezvous once the
    // staging buffers are large enough and mapped (runStaticStaged).
    bool static_staged = false;
    bool host_complete = false;             // the call returns only when the device work is done (barrier)
  };

  // A tensor list that is one range of memory (its non-empty tensors back to back in one storage)
  struct FlatSpan {
    const void* ptr = nullptr;
    size_t bytes = 0;
    bool flat = false;
  };
  static FlatSpan flatSpan(const std::vector<at::Tensor>& tensors);
  // What a rank contributes to an all-to-all: W pieces at offs[d] of an image of `total` bytes that
  // is either caller memory (flat) or packed from `pieces` into the staging buffer
  struct ExchangeImage {
    const void* flat = nullptr;
    std::vector<at::Tensor> pieces;
    std::vector<size_t> offs, sizes;
    size_t total = 0;
  };
  c10::intrusive_ptr<c10d::Work> exchange(c10d::OpType op, const char* title, const std::vector<at::Tensor>& inputs,
                                          const std::vector<at::Tensor>& outputs, const ExchangeImage& image,
                                          const std::vector<void*>& dst, const std::vector<size_t>& recv);
  c10::intrusive_ptr<c10d::Work> run(Plan& plan);
  c10::intrusive_ptr<c10d::Work> finishRun(Plan& plan, hipStream_t s, bool same_stream, bool device_work, bool capturing = false);
  // The one-launch small allreduce of `plan` on `s` (also under stream capture: the launch carries
  // nothing that changes from replay to replay).
  void launchFused(const Plan& plan, hipStream_t s);
  bool fusedFits(const Plan& plan) const;
  void runHostSynced(Plan& plan, hipStream_t s, int slot);
  void runDeviceSynced(Plan& plan, hipStream_t s, int slot, uint64_t seq);
  void deviceBarrier(uint64_t epoch, hipStream_t s);
  // standing offers (pg_sharing.cpp)
  bool standingFits(const Plan& plan) const;
  void runStanding(Plan& plan, hipStream_t s, int slot, uint64_t seq);
  void growStandingCapacity(size_t bytes);
  bool standingExchangeFits() const;
  bool staticStagedFits(const Plan& plan) const;
  void runStaticStaged(Plan& plan, hipStream_t s, int slot, uint64_t seq);
  bool standingExchangeNow(const std::vector<at::Tensor>& inputs, const std::vector<at::Tensor>& outputs);
  void runStandingExchange(Plan& plan, hipStream_t s, int slot, uint64_t seq);
  struct PieceWhere {  // what a reader can be offered in place: entry of this rank's export table, its generation, where in it
    int entry = -1;
    uint64_t gen = 0, off = 0;
  };
  bool announcePieces(const Plan& plan, uint64_t seq, size_t outbox_max, PieceWhere* where);
  void awaitPeerPieces(const Plan& plan, uint64_t seq, size_t outbox_max, bool grew);
  void growOutbox(int peer, int level);
  void mapOutbox(int peer, int level);
  bool acknowledgedBy(int peer, int entry, uint64_t gen, uint64_t seq) const;
  void scanPeerExports(uint64_t seq);
  bool allAcknowledged(int entry, uint64_t gen, uint64_t seq) const;
  void acknowledge(int owner, int entry, uint64_t gen, uint64_t from_seq);
  void noteImport(uint32_t rank, uint32_t entry, uint32_t slot, uint64_t base, uint64_t gen);
  void flushImportTable(hipStream_t s);
  std::chrono::milliseconds deviceWaitLimit() const;
  void throwIfFailed();
  std::string lastEnqueued() const;
  void awaitPeersEntered(uint64_t seq);
  // zero-copy: publish / map caller-owned allocations
  int exportRange(const void* ptr, size_t bytes, uint64_t* offset);
  const void* importRange(int peer, int pub);
  void closeImports();
  void quiesce();  // host waits for this rank's outstanding collective work (before a mapping is closed)
  void ensureInit(int device);
  void* ensureStage(int slot, size_t bytes);
  // start_up: the first barrier of a group, which also absorbs the ranks' different start-up
  // times: at least two minutes, and not shortened by MCCL_BARRIER_TIMEOUT_MS
  void hostBarrier(bool start_up = false);
  std::chrono::milliseconds waitLimit(bool start_up) const;
  const void* peerStage(int peer, int slot, int pub);
  void publishStage(int slot, int pub);
  void checkDeviceTensors(const std::vector<at::Tensor>& tensors) const;
  // Spins (then yields) until ready() holds; raises when `peer` reports a failure, when it has
  // left and abandoned() says that what is awaited can no longer come, or at the time limit.
  // `idle`, when given, runs between polls (a send that waits for a free buffer uses it to
  // complete this rank's own posted receives, so that ranks sending round a ring cannot block
  // each other for good).
  void spinUntil(const std::function<bool()>& ready, int peer, const char* what,
                 const std::function<bool()>& abandoned, const std::function<void()>& idle = nullptr,
                 std::chrono::milliseconds limit_override = std::chrono::milliseconds(0));
  // Completes the receives posted for `src` in order, up to and including `target` (all of them
  // when target is null).  With blocking == false it stops at the first message the sender has
  // not published yet.  progressRecv takes the group's mutex, the Locked form expects it held.
  // `limit` > 0 replaces the group's time limit for the blocking wait (a wait(timeout) of the caller's).
  void progressRecv(int src, const RecvState* target, bool blocking,
                    std::chrono::milliseconds limit = std::chrono::milliseconds(0));
  void progressRecvLocked(int src, const RecvState* target, bool blocking,
                          std::chrono::milliseconds limit = std::chrono::milliseconds(0));

  c10::intrusive_ptr<c10d::Store> store_;
  std::chrono::milliseconds timeout_;
  bool blocking_wait_ = false;  // CCL_BLOCKING_WAIT
  bool same_stream_ = false;    // CCL_SAME_STREAM
  bool verbose_ = false;        // ONECCL_BINDINGS_FOR_PYTORCH_ENV_VERBOSE
  bool profile_ = false;        // MCCL_PG_PROFILE: host-side phase timers, printed when the group dies
  bool want_device_sync_ = true;  // MCCL_PG_SYNC != "host"
  // MCCL_PG_SYNC=kernel: a collective is ONE launch whose workgroups wait for the other ranks
  // themselves.  Fastest, but such a kernel keeps up to 512 wavefronts per rank resident while it
  // waits; with 7 of 8 rank processes waiting on one GPU that is 3 to 4 wavefronts of 120 registers
  // on every SIMD, and a kernel the late rank still has to run before it can join (a GEMM with
  // 128 or more registers per lane: measured with torch.mm) finds no room to start: the waits
  // end at their time limit.  One rank per GPU has no such problem.  The default therefore waits
  // in a one-wavefront barrier kernel in front of the data kernel, whose last workgroup alone
  // waits for the closing epoch: two launches per collective, one waiting wavefront per rank.
  bool waits_in_data_kernels_ = false;
  bool zero_copy_ = true;         // MCCL_PG_ZERO_COPY != 0
  // Largest tensor (bytes per rank) whose zero-copy collective is ONE launch with the rank waits
  // inside the kernel; larger ones run the bandwidth-tuned kernels between barrier kernels.  With 8
  // rank processes the two forms meet at 128-256 MiB per rank for reduce_scatter_tensor and
  // all_to_all_single (one launch is 2x faster at 4-16 MiB, 15-20 % slower at 1 GiB: a persistent
  // grid moves fewer bytes per second than fresh workgroups); the allreduce is one launch at every
  // size.  MCCL_PG_ONE_LAUNCH_MAX_BYTES overrides (and then binds the allreduce, too).
  size_t one_launch_max_ = 128u << 20;
  bool one_launch_max_forced_ = false;
  // Without MCCL_PG_SYNC=kernel a collective is still one launch with the waits inside when its
  // launch moves at most this much (in bytes of a plain copy's traffic, see Plan::compact_cost): the
  // launch is then limited to its share of half of the GPU's compute units (workgroups of sixteen
  // wavefronts), which is enough for a small message and leaves a late rank's other kernels room to
  // run.  Measured with 8 rank processes, back to back, against barrier kernel + full grid: pulls
  // win up to 8 MiB per rank (4 MiB: 65-83 against 93-131 us; 16 MiB: 150-160 against 113-147),
  // all_gather up to 1 MiB per rank (8 MiB written), reduce_scatter and the in-place allreduce up
  // to 32 MiB (16 MiB: 83-104 against 106-141 us).  MCCL_PG_COMPACT_MAX_BYTES overrides (0: never).
  size_t compact_max_ = 16u << 20;
  bool allgather_push_ = true;  // MCCL_PG_ALLGATHER_PUSH != 0: all_gather_into_tensor writes into the peers' outputs
  // Bisecting switches of the reference (src/gpu/dpcpp_ccl.cpp:56-85), for rank processes: what
  // does a collective cost without its cross-rank waits, what do the waits cost alone?  Results are
  // NOT valid with either of the first two; they exist for timing.
  //   TORCH_CCL_WORK_ONLY / MCCL_PG_WORK_ONLY=1   data kernels only: no barrier kernel, no waits inside
  //   TORCH_CCL_SYNC_ONLY / MCCL_PG_SYNC_ONLY=1   the cross-rank waits only: no copy-in, no data kernel
  //   TORCH_CCL_DISABLE_ALLREDUCE=1               allreduce enqueues nothing (src/gpu/dpcpp_ccl.cpp:752-756)
  bool work_only_ = false;
  bool sync_only_ = false;
  bool disable_allreduce_ = false;
  unsigned fused_mode_ = 0;     // the same two as flags of mccl_allreduce_fused_replayable
 public:
  // 0 = none, 1 = work only, 2 = sync only, + 4 when allreduce is disabled (for tests of the parsing)
  int bisectMode() const { return (work_only_ ? 1 : 0) | (sync_only_ ? 2 : 0) | (disable_allreduce_ ? 4 : 0); }
  // (collectives that met at the rendezvous of the host threads, collectives that only enqueued)
  // collectives that met at the host rendezvous; that only enqueued; that only enqueued after waiting for
  // single peers (an all-to-all whose piece for or from that peer outgrew the buffer kept for it)
  std::tuple<uint64_t, uint64_t, uint64_t> rendezvousCounts() const { return {rendezvous_count_, enqueue_only_count_, pairwise_wait_count_}; }
  std::string lastPath() const { return last_path_ ? last_path_ : ""; }
 private:
  unsigned waiting_cus_ = 128;  // what all ranks' waiting launches may hold together (MCCL_PG_WAITING_COMPUTE_UNITS)
  bool distinct_pids_ = false;          // every rank is a process of its own
  const char* last_title_ = nullptr;  // the collective this rank enqueued last, for failure reports
  const char* last_path_ = "";
  uint64_t last_seq_ = 0;
  bool comm_stream_for_large_ = false;  // MCCL_PG_COMM_STREAM=1: device-synchronised groups fork large collectives too
  // Decided at start-up, the same on every rank: all ranks are processes of their own (and the
  // environment does not ask for the host barrier), so cross-rank waits can live on the device.
  bool device_sync_ = false;
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
    uint64_t gen = 0;      // bumped whenever the buffer is replaced
    hipIpcMemHandle_t handle{};
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

  // device-side synchronisation: one small arena per rank (flag words, and the staging buffers and
  // tile flags of the one-launch allreduce), mapped by every peer at start-up
  void* arena_ = nullptr;
  std::vector<void*> peer_arena_;           // this process's mapping of rank r's arena
  std::vector<void*> bar_flags_;            // rank r's barrier word
  std::vector<void*> final_flags_;          // rank r's departure word
  std::vector<void*> fused_stage_[2];       // rank r's staging buffer of the one-launch allreduce, per slot
  std::vector<void*> fused_flags_[2];
  void* done_counter_ = nullptr;            // this rank's workgroup counter of the one-launch collectives
  void* fused_state_ = nullptr;             // this rank's device-resident epoch of the one-launch small allreduce
  void* status_dev_ = nullptr;              // device address of shared_->status
  // standing offers: MCCL_PG_STANDING_OFFERS != 0 -- allreduces above the one-launch size exchange
  // where their tensors are on the device and never meet on the host
  bool standing_offers_ = true;
  size_t standing_capacity_ = 0;            // staging of both slots that holds this much on every rank, mapped by every peer
  size_t standing_max_ = 256u << 20;        // larger buffers meet at the rendezvous (MCCL_PG_STANDING_MAX_BYTES): the fallback needs staging of that size
  mccl_import_table_t* import_table_ = nullptr;  // device: the peers' allocations as this rank has mapped them
  void* resolved_ = nullptr;                // device: where the ranks' tensors of the collective under way are
  std::vector<void*> offer_slots_[2];       // rank r's offer slot, per parity of the collective
  std::vector<void*> offer_rows_[2];        // rank r's row of offers (all-to-all), per parity of the collective
  struct OutboxOut {                        // this rank's outbox for rank d (for itself: scratch nobody else maps)
    void* base = nullptr;
    int level = -1;
  } outbox_out_[MCCL_OFFER_RANKS];
  struct OutboxIn {                         // rank r's outbox for this rank, as mapped here
    void* base = nullptr;
    int level = -1;
  } outbox_in_[MCCL_OFFER_RANKS];
  uint64_t big_published_[MCCL_OFFER_RANKS] = {};  // the last BigPiece record written for rank d (its seq)
  uint64_t pairwise_wait_count_ = 0;
  unsigned pairwise_waits_now_ = 0;         // waits for single peers in the all-to-all under way
  std::string last_path_storage_;
  std::vector<mccl_import_update_t> table_updates_;  // mappings that changed since the device table last heard
  uint64_t seen_live_[MCCL_OFFER_RANKS][MCCL_OFFER_ENTRIES] = {};  // peers' export entries as this rank last read them
  uint64_t last_offer_seq_[MCCL_OFFER_ENTRIES] = {};               // 1 + the last collective that offered the entry (0: none)
  std::shared_ptr<GroupShared> shared_;

  // zero-copy exports (this rank's allocations the peers may map) and imports
  struct Export {
    uint64_t base = 0;
    uint64_t size = 0;
    bool valid = false;
  };
  std::vector<Export> exports_;             // mirrors the export table of this rank's control slot
  int export_clock_ = 0;                    // next table entry to evict
  int recent_export_[2] = {-1, -1};         // entries of the last two offers: not evicted
  uint64_t rendezvous_count_ = 0;           // device-synchronised collectives that met at the host rendezvous
  uint64_t enqueue_only_count_ = 0;         // device-synchronised collectives that needed none (recorded ones included)
  struct Import {
    void* base = nullptr;
    uint64_t gen = 0;
  };
  std::vector<std::vector<Import>> imports_;  // [peer][export entry]
 public:
  // Called (under the allocator's lock) when torch's caching allocator returns a segment to the
  // runtime: an export of that segment must not be handed to the peers again.
  void segmentFreed(uint64_t base);
 private:

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
