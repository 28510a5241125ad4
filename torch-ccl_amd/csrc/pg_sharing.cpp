// c10d backend "ccl" for ROCm tensors: staging buffers, allocations shared between the rank processes, standing offers.
#include "pg_internal.hpp"

namespace mccl_pg {

// The tracker is attached once per process and never detached (torch offers no way to), so it only
// touches groups that are still registered here.
std::mutex g_registry_mutex;
std::vector<ProcessGroupCCL*> g_registry;

namespace {
std::once_flag g_tracker_once;
}

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
  int entry = -1;
  if (!st.force_staged && bytes >= kZeroCopyMinBytes) {
    const bool inside = st.block && (const char*)st.buffer >= (const char*)st.block &&
                        (const char*)st.buffer + bytes <= (const char*)st.block + st.block_bytes;
    entry = inside ? exportRange(st.block, st.block_bytes, &off) : exportRange(st.buffer, bytes, &off);
    if (inside && entry >= 0) off += (uint64_t)((const char*)st.buffer - (const char*)st.block);
  }
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

// ---------------------------------------------------------------------------------------------
// all-to-all with standing offers
// ---------------------------------------------------------------------------------------------
// In an all-to-all every rank hands every peer a different piece, and the sizes differ from rank to
// rank: there is no number that all ranks know, so nothing the whole group could agree on without
// meeting -- not "everybody stages", not "the staging buffers grow now".  What two ranks do know in
// common is the length of the piece that goes from one to the other.  So everything is decided pair
// by pair: rank r offers rank d its piece in place when d has mapped the allocation it lives in, and
// through a buffer it keeps for d alone (its outbox for d) otherwise; the outbox has the size class
// of the largest piece that ever went from r to d, so both know when a larger one is due -- r
// creates it on entering that collective, d waits for it there (the only wait of this path, and only
// for that one peer).  Pieces beyond the largest outbox are read in place always: the receiver waits
// until the sender has entered the collective and said where the piece is, and maps it then.
// The offers travel on the device as a row per rank (mccl_rank_barrier_offers_each); each rank pulls
// the column addressed to it (mccl_copy_segments_sync_resolved).
bool ProcessGroupCCL::standingExchangeFits() const {
  return standing_offers_ && device_sync_ && distinct_pids_ && zero_copy_ && !waits_in_data_kernels_ && !work_only_ &&
         !sync_only_ && size_ > 1 && size_ <= MCCL_OFFER_RANKS;
}

// For the all-to-all engine, which has to know before it plans (the fallback moves images larger than
// a staging window in several rounds, this path never does): initialises the group if this is its
// first collective, like run() would a moment later.
bool ProcessGroupCCL::standingExchangeNow(const std::vector<at::Tensor>& inputs, const std::vector<at::Tensor>& outputs) {
  std::lock_guard<std::mutex> lock(mutex_);
  int device = -1;
  for (const auto& t : inputs) if (t.defined()) { device = t.get_device(); break; }
  if (device < 0) for (const auto& t : outputs) if (t.defined()) { device = t.get_device(); break; }
  if (device < 0) return false;
  c10::DeviceGuard guard(c10::Device(at::kCUDA, (c10::DeviceIndex)device));
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HIP_CHECK(hipStreamIsCapturing(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA((c10::DeviceIndex)device).stream(), &capture));
  if (capture != hipStreamCaptureStatusNone) return false;  // run() refuses it with the reason
  ensureInit(device);
  return standingExchangeFits();
}

bool ProcessGroupCCL::acknowledgedBy(int peer, int entry, uint64_t gen, uint64_t seq) const {
  const RankSlot::Ack& a = ctl_->slot[peer].acked[rank_][entry];
  if (a.gen.load(std::memory_order_acquire) != gen) return false;
  const uint64_t from = a.from_seq.load(std::memory_order_acquire);
  return a.gen.load(std::memory_order_acquire) == gen && from <= seq;
}

// A larger outbox for rank `peer` (for this rank itself: scratch).  The old one stays until the group
// goes: the peer's kernels of earlier collectives may still read it.
void ProcessGroupCCL::growOutbox(int peer, int level) {
  TORCH_CHECK(level < kOutboxLevels, "ccl backend: outbox level ", level);
  void* base = nullptr;
  HIP_CHECK(hipMalloc(&base, kOutboxMin << level));
  OutboxOut& out = outbox_out_[peer];
  if (out.base) retired_.push_back(out.base);
  out.base = base;
  out.level = level;
  if (peer == rank_) return;
  RankSlot::OutboxLevel& lv = ctl_->slot[rank_].outbox[peer].level[level];
  HIP_CHECK(hipIpcGetMemHandle(&lv.handle, base));
  lv.ptr = (uint64_t)(uintptr_t)base;
  lv.ready.store(1, std::memory_order_release);
}

// Rank `peer`'s outbox of size class `level` for this rank: the peer creates it when it enters the
// collective whose piece needs it, which is the collective this rank is entering.
void ProcessGroupCCL::mapOutbox(int peer, int level) {
  RankSlot::OutboxLevel& lv = ctl_->slot[peer].outbox[rank_].level[level];
  if (!lv.ready.load(std::memory_order_acquire)) {
    ++pairwise_waits_now_;
    spinUntil([&] { return lv.ready.load(std::memory_order_acquire) != 0; }, peer,
              "the buffer a rank keeps for the pieces of its all-to-alls to this rank (if that rank has entered the same all-to-all, "
              "its inputSplitSizes do not match this rank's outputSplitSizes)",
              [] { return true; });
  }
  OutboxIn& in = outbox_in_[peer];
  if (in.base) {
    quiesce();  // earlier kernels of this rank may still read through the old mapping
    (void)hipIpcCloseMemHandle(in.base);
    in.base = nullptr;
  }
  void* p = nullptr;
  HIP_CHECK(hipIpcOpenMemHandle(&p, lv.handle, hipIpcMemLazyEnablePeerAccess));
  in.base = p;
  in.level = level;
  noteImport((uint32_t)peer, MCCL_OFFER_STAGED, MCCL_OFFER_SLOT_OUTBOX, (uint64_t)(uintptr_t)p, 0);
}

// Step 1 of an exchange: everything this rank has to say, before it waits for anything of anybody's --
// the allocations its pieces live in (where[d]: what rank d can be offered in place), larger
// outboxes where a piece has outgrown the old one, where its oversized pieces are.  Returns whether
// the group's staging buffers had to grow (one piece for all readers only).
bool ProcessGroupCCL::announcePieces(const Plan& plan, uint64_t seq, size_t outbox_max, PieceWhere* where) {
  const Plan::StandingExchange& x = plan.standing_exchange;
  const int W = size_, me = rank_;
  RankSlot& mine_slot = ctl_->slot[me];
  const bool same = x.same_piece;
  bool unshareable_big = false;
  const void* announced_block = nullptr;
  PieceWhere announced;
  for (int d = 0; d < W; ++d) {
    const size_t b = x.send[(size_t)d];
    if (d == me || !b || x.force_staged) continue;
    const bool big = b > outbox_max;
    // (small tensors live in the allocator's 2 MiB segments, many of them: announcing those would turn
    // the table of allocations over all the time, and copying them costs next to nothing)
    if (!big && x.block_bytes[(size_t)d] < kZeroCopyMinBytes) continue;
    PieceWhere& w = where[d];
    if (announced_block == x.block[(size_t)d]) {  // (one tensor, or a flat list: the pieces share a storage)
      w = announced;
    } else {
      w.entry = exportRange(x.block[(size_t)d], x.block_bytes[(size_t)d], &w.off);
      if (w.entry >= 0 && w.entry < kMaxExports) w.gen = mine_slot.exports[w.entry].gen.load(std::memory_order_acquire);
      else w.entry = -1;
      announced_block = x.block[(size_t)d];
      announced = w;
    }
    if (w.entry >= 0) w.off += (uint64_t)((const char*)x.piece[(size_t)d] - (const char*)x.block[(size_t)d]);
  }
  // (pieces in more allocations than the table has free entries: a later one may have taken the entry
  // of an earlier one)
  for (int d = 0; d < W; ++d)
    if (where[d].entry >= 0 && mine_slot.exports[where[d].entry].gen.load(std::memory_order_acquire) != where[d].gen) where[d].entry = -1;
  // (the staging buffers of a group grow when a message exceeds them, which all ranks find at the same
  // collective where all ranks know the sizes; and since they meet there, they also look at what
  // everybody has just announced before anybody decides: see runStanding)
  const bool grow = same && x.unanimous_bytes > standing_capacity_;
  if (grow) growStandingCapacity(x.unanimous_bytes);
  for (int d = 0; d < W && !same; ++d) {
    const size_t b = x.send[(size_t)d];
    if (!b) continue;
    if (b <= outbox_max) {
      const int level = outboxLevel(b);
      const bool needed = d != me || x.force_staged;  // (this rank's piece for itself is copied where it lies, unless that overlaps)
      if (needed && level > outbox_out_[d].level) growOutbox(d, level);
    } else {
      TORCH_CHECK(!x.force_staged, "ccl backend: ", plan.title, ": input and output overlap and the piece for rank ", d, " (", b,
                  " bytes) is larger than the buffers kept for such pieces (", outbox_max, " bytes); set MCCL_PG_STANDING_OFFERS=0");
      if (d == me) continue;  // (copied where it lies)
      RankSlot::BigPiece& rec = mine_slot.big[d];
      if (big_published_[d]) {  // rank d has not read the last such record yet: not overwritten before it has
        const uint64_t last = big_published_[d];
        if (ctl_->slot[d].big_seen[me].load(std::memory_order_acquire) < last) {
          ++pairwise_waits_now_;
          spinUntil([&] { return ctl_->slot[d].big_seen[me].load(std::memory_order_acquire) >= last; }, d,
                    "a rank to take note of an earlier oversized all-to-all piece", [] { return true; });
        }
      }
      rec.entry = where[d].entry;
      rec.gen = where[d].gen;
      rec.seq.store(seq + 1, std::memory_order_release);
      big_published_[d] = seq + 1;
      if (where[d].entry < 0) unshareable_big = true;
    }
  }
  TORCH_CHECK(!unshareable_big, "ccl backend: ", plan.title, ": a piece larger than ", outbox_max,
              " bytes lives in memory that cannot be shared between processes (not from torch's caching allocator, or an allocation of 2 GiB "
              "or more); set MCCL_PG_STANDING_OFFERS=0");
  return grow;
}

// Step 2: what the peers must have said by now, pair by pair -- the outbox of a size class this rank
// has not mapped yet, where an oversized piece is -- and a look at what they have announced.
void ProcessGroupCCL::awaitPeerPieces(const Plan& plan, uint64_t seq, size_t outbox_max, bool grew) {
  const Plan::StandingExchange& x = plan.standing_exchange;
  const int W = size_, me = rank_;
  for (int r = 0; r < W && !x.same_piece; ++r) {
    const size_t b = x.recv[(size_t)r];
    if (r == me || !b) continue;
    if (b <= outbox_max) {
      const int level = outboxLevel(b);
      if (level > outbox_in_[r].level) mapOutbox(r, level);
    } else {
      RankSlot::BigPiece& rec = ctl_->slot[r].big[me];
      if (rec.seq.load(std::memory_order_acquire) != seq + 1) {
        ++pairwise_waits_now_;
        spinUntil([&] { return rec.seq.load(std::memory_order_acquire) >= seq + 1; }, r,
                  "a rank to enter the all-to-all in which it sends this rank an oversized piece", [] { return true; });
      }
      TORCH_CHECK(rec.seq.load(std::memory_order_acquire) == seq + 1, "ccl backend: ", plan.title, ": rank ", r,
                  " is at another oversized all-to-all piece for this rank (the ranks' split sizes do not match)");
    }
  }
  scanPeerExports(seq);
  if (grew) hostBarrier();
  for (int r = 0; r < W; ++r) {
    const size_t b = x.recv[(size_t)r];
    if (r == me || b <= outbox_max) continue;
    RankSlot::BigPiece& rec = ctl_->slot[r].big[me];
    const int64_t entry = rec.entry;
    const uint64_t gen = rec.gen;
    ctl_->slot[me].big_seen[r].store(seq + 1, std::memory_order_release);
    TORCH_CHECK(entry >= 0 && entry < kMaxExports, "ccl backend: ", plan.title, ": rank ", r, " cannot share the memory that holds its piece of ", b,
                " bytes for this rank, which is larger than the buffers kept for such pieces; set MCCL_PG_STANDING_OFFERS=0");
    const Import& im = imports_[(size_t)r][(size_t)entry];
    TORCH_CHECK(im.base && im.gen == gen, "ccl backend: ", plan.title, ": could not map the allocation that holds rank ", r, "'s piece for this rank");
  }
}

void ProcessGroupCCL::runStandingExchange(Plan& plan, hipStream_t s, int slot, uint64_t seq) {
  const Plan::StandingExchange& x = plan.standing_exchange;
  const int W = size_, me = rank_;
  const uint64_t epoch = 4 * seq;
  const bool same = x.same_piece;  // one piece for all readers, sizes known to all: staged through the staging buffer, nothing pairwise
  const size_t outbox_max = same ? ~(size_t)0 : std::min(standing_max_, kOutboxMin << (kOutboxLevels - 1));
  pairwise_waits_now_ = 0;
  PieceWhere where[MCCL_OFFER_RANKS];
  const bool grew = announcePieces(plan, seq, outbox_max, where);
  awaitPeerPieces(plan, seq, outbox_max, grew);
  // 3. This rank's row of offers.
  mccl_offer_t row[MCCL_OFFER_RANKS] = {};
  uint64_t expect[MCCL_OFFER_RANKS] = {};
  std::vector<mccl_segment_t> copy_in;
  int in_place = 0, staged = 0;
  for (int d = 0; d < W; ++d) {
    const size_t b = x.send[(size_t)d];
    mccl_offer_t& o = row[d];
    o.bytes = b;
    o.entry = MCCL_OFFER_STAGED;
    o.slot = same ? (uint32_t)slot : MCCL_OFFER_SLOT_OUTBOX;
    expect[d] = x.recv[(size_t)d];
    if (!b || d == me) continue;
    const PieceWhere& w = where[d];
    if (w.entry >= 0 && (b > outbox_max || acknowledgedBy(d, w.entry, w.gen, seq))) {
      o.entry = (uint32_t)w.entry;
      o.slot = 0;
      o.generation = w.gen;
      o.offset = w.off;
      last_offer_seq_[w.entry] = seq + 1;  // in the units of `entered`: collective `seq` is under way at seq + 1
      ++in_place;
    } else {
      if (!same) copy_in.push_back({x.piece[(size_t)d], outbox_out_[d].base, b});
      else if (copy_in.empty()) copy_in.push_back({x.piece[(size_t)d], stage_[slot].ptr, b});  // once, for all readers that need it
      ++staged;
    }
  }
  const void* my_source = x.piece[(size_t)me];
  if (x.force_staged && x.send[(size_t)me]) {
    void* scratch = same ? stage_[slot].ptr : outbox_out_[me].base;
    if (!same || copy_in.empty()) copy_in.push_back({x.piece[(size_t)me], scratch, x.send[(size_t)me]});
    my_source = scratch;
  }
  // Little to move: ONE launch on this rank's share of half of the compute units, which copies into the
  // outboxes, carries the row and pulls -- with several processes on the GPU every launch waits for
  // its turn at the dispatcher, which costs more than the data at these sizes.  (A matter of this
  // rank alone: the two forms look the same to the peers.)
  size_t moved = 0;
  for (const auto& sg : copy_in) moved += sg.bytes;
  for (int r = 0; r < W; ++r) moved += x.recv[(size_t)r];
  const bool one_launch = !x.reduce && 2.0 * (double)moved <= (double)compact_max_;
  if (!one_launch && !copy_in.empty()) MCCL_CHECK(mccl_copy_segments(copy_in.data(), (int)copy_in.size(), s));
  {
    std::ostringstream os;
    if (same) os << "standing offers, " << (staged ? "this rank staged" : "peers read in place");
    else os << "standing offers, " << in_place << " pieces read in place, " << staged << " through outboxes";
    last_path_storage_ = os.str();
    last_path_ = last_path_storage_.c_str();
  }
  if (verbose_) {
    std::ostringstream os;
    os << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "#" << (seq + 1) << "] " << last_path_;
    std::cout << os.str() << std::endl;
  }
  if (pairwise_waits_now_) ++pairwise_wait_count_;
  else ++enqueue_only_count_;
  // 4. On the device: the rows, then the pulls.
  flushImportTable(s);
  const uint64_t limit_us = (uint64_t)waitLimit(false).count() * 1000ull;
  const int par = (int)(seq & 1);
  if (!one_launch)
    MCCL_CHECK(mccl_rank_barrier_offers_each(bar_flags_.data(), W, me, epoch + 1, limit_us, status_dev_, row, expect, my_source,
                                             offer_rows_[par].data(), import_table_, resolved_, s));
  mccl_xsync_t sync{};
  sync.words = bar_flags_.data();
  sync.n = W;
  sync.rank = me;
  sync.done_epoch = epoch + 3;  // nobody's stream goes on before every rank has pulled what it gets from it
  sync.done_counter = done_counter_;
  sync.timeout_us = limit_us;
  sync.status = status_dev_;
  std::vector<mccl_segment_t> pulls;
  std::vector<int> from;
  for (int r = 0; r < W; ++r) {
    if (!x.recv[(size_t)r]) continue;
    pulls.push_back({nullptr, x.dst[(size_t)r], x.recv[(size_t)r]});
    from.push_back(r);
  }
  if (x.reduce) {
    x.reduce(resolved_, sync, s);
  } else if (one_launch) {
    sync.ready_epoch = epoch + 1;
    sync.max_compute_units = std::max(1u, waiting_cus_ / (unsigned)W);
    MCCL_CHECK(mccl_alltoall_sync_offers(copy_in.data(), (int)copy_in.size(), pulls.data(), from.data(), (int)pulls.size(), &sync, row, expect,
                                         my_source, offer_rows_[par].data(), import_table_, s));
  } else {
    MCCL_CHECK(mccl_copy_segments_sync_resolved(pulls.data(), from.data(), (int)pulls.size(), resolved_, 0u, &sync, s));
  }
}

// ---------------------------------------------------------------------------------------------
// coalesced forms: packed into the staging buffer, which the peers have mapped for good
// ---------------------------------------------------------------------------------------------
// What the rendezvous of a staged collective publishes is the handle of the staging buffer, which
// only changes when the buffer grows.  The coalesced forms pack their tensors into it at offsets
// every rank computes for itself, so once the buffers of both slots are large enough on every rank
// (the sizes of a coalesced call agree, so all ranks find out together: growStandingCapacity) such
// a collective is copy-in, barrier kernel, kernel over the peers' staging buffers -- and no
// meeting of the host threads.  The two slots alternate by collective as ever: every collective
// waits on the device for every peer's start of it, so a slot is free again two collectives on.
bool ProcessGroupCCL::staticStagedFits(const Plan& plan) const {
  return plan.static_staged && standing_offers_ && device_sync_ && distinct_pids_ && !waits_in_data_kernels_ && !work_only_ &&
         !sync_only_ && size_ > 1 && plan.stage_bytes > 0 && plan.stage_bytes <= std::min(stage_max_, standing_max_) && plan.exec &&
         !plan.exec2;
}

void ProcessGroupCCL::runStaticStaged(Plan& plan, hipStream_t s, int slot, uint64_t seq) {
  const uint64_t epoch = 4 * seq;
  if (plan.stage_bytes > standing_capacity_) growStandingCapacity(plan.stage_bytes);
  void* stage = stage_[slot].ptr;
  if (plan.copy_in) plan.copy_in(stage, s);
  last_path_ = "staged, staging buffers mapped for good";
  if (verbose_) {
    std::ostringstream os;
    os << "oneccl_bindings_for_pytorch::" << plan.title << " [" << rank_ << "/" << size_ << "#" << (seq + 1) << "] " << last_path_;
    std::cout << os.str() << std::endl;
  }
  ++enqueue_only_count_;
  deviceBarrier(epoch + 1, s);
  PeerView pv;
  pv.zero_copy = false;
  pv.stage.resize((size_t)size_);
  pv.tables.assign((size_t)size_, nullptr);
  for (int r = 0; r < size_; ++r) pv.stage[(size_t)r] = (r == rank_) ? stage : peers_[(size_t)r].ptr[slot];
  plan.exec(pv, s);
}

void ProcessGroupCCL::closeImports() {
  for (auto& per_peer : imports_)
    for (auto& im : per_peer)
      if (im.base) {
        (void)hipIpcCloseMemHandle(im.base);
        im.base = nullptr;
      }
}

}  // namespace mccl_pg
