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

}  // namespace mccl_pg
