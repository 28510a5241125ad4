// c10d backend "ccl" for ROCm tensors: the collectives.
#include "pg_internal.hpp"

namespace mccl_pg {

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
  if (total && total <= std::min(stage_max_, standing_max_) && standingExchangeNow({t}, {t})) {
    // rank processes: where the root's tensor is travels on the device, nobody meets (runStandingExchange)
    const int W = size_, me = rank_;
    Plan p;
    p.op = c10d::OpType::BROADCAST;
    p.title = "broadcast";
    p.inputs = {t};
    p.outputs = {t};
    Plan::StandingExchange& x = p.standing_exchange;
    x.ok = true;
    x.same_piece = true;
    x.unanimous_bytes = total;
    x.piece.assign((size_t)W, me == root ? t.data_ptr() : nullptr);
    x.send.assign((size_t)W, me == root ? total : 0);
    x.send[(size_t)me] = 0;  // the root keeps what it has
    x.block.assign((size_t)W, t.storage().data());
    x.block_bytes.assign((size_t)W, t.storage().nbytes());
    x.dst.assign((size_t)W, nullptr);
    x.recv.assign((size_t)W, 0);
    if (me != root) {
      x.dst[(size_t)root] = t.data_ptr();
      x.recv[(size_t)root] = total;
    }
    return run(p);
  }
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
      p.standing.block = t.storage().data();
      p.standing.block_bytes = t.storage().nbytes();
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
  p.static_staged = true;
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
        p.standing.block = output.storage().data();
        p.standing.block_bytes = output.storage().nbytes();
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
  const int W = size_;
  if (largest && largest <= standing_max_ && standingExchangeNow({input}, outs)) {
    // rank processes: where the inputs are travels on the device, nobody meets (runStandingExchange:
    // every reader gets the same piece, and every rank knows every rank's size from its output list)
    const int me = rank_;
    TORCH_CHECK(mine == nbytes(outs[(size_t)me]), "allgather: output tensor ", me, " does not match the size rank ", me, " sends");
    Plan p;
    p.op = c10d::OpType::ALLGATHER;
    p.title = "allgather";
    p.inputs = {input};
    p.outputs = outs;
    Plan::StandingExchange& x = p.standing_exchange;
    x.ok = true;
    x.same_piece = true;
    x.unanimous_bytes = largest;
    x.piece.assign((size_t)W, mine ? input.data_ptr() : nullptr);
    x.send.assign((size_t)W, mine);
    x.block.assign((size_t)W, input.storage().data());
    x.block_bytes.assign((size_t)W, input.storage().nbytes());
    x.dst.resize((size_t)W);
    x.recv.resize((size_t)W);
    for (int r = 0; r < W; ++r) {
      x.dst[(size_t)r] = outs[(size_t)r].data_ptr();
      x.recv[(size_t)r] = nbytes(outs[(size_t)r]);
      const bool itself = r == me && outs[(size_t)r].data_ptr() == input.data_ptr();  // gathered into the very tensor it comes from
      if (itself) x.recv[(size_t)r] = 0;
      else if (rangesOverlap(input.data_ptr(), mine, x.dst[(size_t)r], x.recv[(size_t)r])) x.force_staged = true;
    }
    return run(p);
  }
  Plan p;
  p.op = c10d::OpType::ALLGATHER;
  p.title = "allgather";
  p.inputs = {input};
  p.outputs = outs;
  p.stage_bytes = mine;
  p.table = {(int64_t)mine};
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
  p.static_staged = true;
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
        p.standing.block = input.storage().data();
        p.standing.block_bytes = input.storage().nbytes();
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
  size_t largest_slot = 0;
  for (const auto& slot : ins) largest_slot = std::max(largest_slot, nbytes(slot));  // the same on every rank of a valid call
  if (largest_slot <= std::min(standing_max_, kOutboxMin << (kOutboxLevels - 1)) && standingExchangeNow(ins, {out})) {
    // rank processes: where the slots are travels on the device, nobody meets (runStandingExchange: slot d
    // of this rank's list is its piece for rank d, in place or through the outbox kept for rank d)
    TORCH_CHECK(nbytes(out) == nbytes(ins[(size_t)me]), "reduce_scatter: output tensor does not match slot ", me);
    Plan q;
    q.op = c10d::OpType::REDUCE_SCATTER;
    q.title = "reduce_scatter";
    q.inputs = ins;
    q.outputs = {out};
    Plan::StandingExchange& x = q.standing_exchange;
    x.ok = true;
    x.piece.resize((size_t)W);
    x.send.resize((size_t)W);
    x.block.resize((size_t)W);
    x.block_bytes.resize((size_t)W);
    x.dst.assign((size_t)W, out.data_ptr());
    x.recv.assign((size_t)W, nbytes(out));  // every rank's slot for this rank has the size of this rank's output
    for (int d = 0; d < W; ++d) {
      const at::Tensor& slot = ins[(size_t)d];
      x.send[(size_t)d] = nbytes(slot);
      x.piece[(size_t)d] = x.send[(size_t)d] ? slot.data_ptr() : nullptr;
      x.block[(size_t)d] = slot.storage().data();
      x.block_bytes[(size_t)d] = slot.storage().nbytes();
      // (the output may be this rank's own slot for itself, exactly: the reduction reads element i of
      // every input before it writes element i)
      const bool itself = d == me && slot.data_ptr() == out.data_ptr();
      if (!itself && rangesOverlap(slot.data_ptr(), x.send[(size_t)d], out.data_ptr(), nbytes(out))) x.force_staged = true;
    }
    const size_t count = (size_t)out.numel();
    void* const out_ptr = out.data_ptr();
    x.reduce = [=](const void* resolved, const mccl_xsync_t& sync, hipStream_t s) {
      MCCL_CHECK(mccl_reduce_sync_resolved(resolved, 0, out_ptr, count, dtype, op, &sync, s));
    };
    return run(q);
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
  p.static_staged = true;
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
  if (standingExchangeNow(inputs, outputs)) {
    // rank processes that exchange where their pieces are on the device: nothing is published on the
    // host, nobody meets (runStandingExchange)
    Plan p;
    p.op = op;
    p.title = title;
    p.inputs = inputs;
    p.outputs = outputs;
    Plan::StandingExchange& x = p.standing_exchange;
    x.ok = true;
    x.send = image.sizes;
    x.recv = recv;
    x.dst = dst;
    x.piece.assign((size_t)W, nullptr);
    x.block.assign((size_t)W, nullptr);
    x.block_bytes.assign((size_t)W, 0);
    for (int d = 0; d < W; ++d) {
      if (!image.sizes[(size_t)d]) continue;
      x.piece[(size_t)d] = image.flat ? (const void*)((const char*)image.flat + image.offs[(size_t)d]) : image.pieces[(size_t)d].data_ptr();
      // (a flat image is one tensor, or consecutive views of one storage)
      const at::Tensor& holder = image.flat ? (is_base ? inputs[0] : inputs[(size_t)d]) : image.pieces[(size_t)d];
      x.block[(size_t)d] = holder.storage().data();
      x.block_bytes[(size_t)d] = holder.storage().nbytes();
      for (int r = 0; r < W; ++r)
        if (rangesOverlap(x.piece[(size_t)d], image.sizes[(size_t)d], dst[(size_t)r], recv[(size_t)r])) x.force_staged = true;
    }
    return run(p);
  }
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

}  // namespace mccl_pg
