"""Rank body for tests/test_gpu_sync.py: N processes on cuda:0 call the cross-rank entry points of
the C ABI (mccl_rank_barrier, mccl_allreduce_fused) directly.  Staging buffers and flag words are
torch tensors shared between the processes through torch.multiprocessing queues (device IPC)."""
import ctypes
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "torch-ccl_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402
import torch  # noqa: E402

DEV = "cuda:0"
FUSED_MAX_BYTES = 1 << 20
TILE = 1024


def _exchange(rank, world, queues, barrier, mine):
    """Every rank hands its shared tensors to every peer; returns the per-rank lists."""
    for r in range(world):
        if r != rank:
            queues[r].put((rank, mine))
    got = {rank: mine}
    for _ in range(world - 1):
        src, ts = queues[rank].get(timeout=120)
        got[src] = ts
    barrier.wait(timeout=120)  # everybody has opened everything before anyone goes on
    return [got[r] for r in range(world)]


def _status():
    st = torch.zeros(2, dtype=torch.int32).pin_memory()
    return st


def barrier_case(rank, world, queues, barrier):
    """Writes of the kernels before a barrier are visible to the peers' kernels after it, round
    after round, with nothing but the flag kernel between them."""
    from torch_ccl_amd import capi
    L = capi.lib()
    n = 1 << 16
    data = torch.zeros(n, dtype=torch.int32, device=DEV)
    flag = torch.zeros(8, dtype=torch.int64, device=DEV)
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, [data, flag])
    flags = capi.ptr_table([shared[r][1].data_ptr() for r in range(world)])
    st = _status()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ramp = torch.arange(n, dtype=torch.int32, device=DEV)
    epoch = 0
    sums = []
    for it in range(1, 101):
        data.copy_(ramp + (1000 * it + rank))
        epoch += 1
        capi.check(L.mccl_rank_barrier(flags, world, rank, epoch, 5_000_000, st.data_ptr(), stream))
        total = torch.zeros(n, dtype=torch.int32, device=DEV)
        for r in range(world):
            total += shared[r][0]
        sums.append(total)
        epoch += 1  # nobody overwrites its data before everybody has read it
        capi.check(L.mccl_rank_barrier(flags, world, rank, epoch, 5_000_000, st.data_ptr(), stream))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    for it, total in enumerate(sums, start=1):
        want = ramp * world + sum(1000 * it + r for r in range(world))
        assert torch.equal(total, want), (it, total[:4].tolist(), want[:4].tolist())
    barrier.wait(timeout=120)


def fused_case(rank, world, queues, barrier):
    """mccl_allreduce_fused against the oracle, bit for bit: all dtypes and ops, counts with whole
    and partial vectors and tiles, in place and out of place, two alternating staging sets."""
    from helpers import ALL_DTYPES, TORCH_TO_CODE, assert_bits_equal, bits, oracle_reduce_bits, rank_buffer
    from oracle import oracle as O
    from torch_ccl_amd import capi
    L = capi.lib()
    stage = [torch.zeros(FUSED_MAX_BYTES + 64, dtype=torch.uint8, device=DEV) for _ in range(2)]
    tflag = [torch.zeros(FUSED_MAX_BYTES // TILE + 1, dtype=torch.int32, device=DEV) for _ in range(2)]
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, stage + tflag)
    tables = []
    for slot in range(2):
        tables.append((capi.ptr_table([shared[r][slot].data_ptr() for r in range(world)]),
                       capi.ptr_table([shared[r][2 + slot].data_ptr() for r in range(world)])))
    st = _status()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ops = {"SUM": (capi.SUM, O.SUM), "PROD": (capi.PROD, O.PROD), "MIN": (capi.MIN, O.MIN), "MAX": (capi.MAX, O.MAX),
           "AVG": (capi.AVG, O.AVG)}
    cases = []
    for dtype in ALL_DTYPES:
        es = torch.empty(0, dtype=dtype).element_size()
        for count in (1, 7, 16 // es, 16 // es + 1, 1024 // es, 1024 // es + 3, 5 * 1024 // es - 1, 40_000):
            for name in ops:
                if name == "AVG" and not dtype.is_floating_point:
                    continue  # an addition of this library, floats only
                cases.append((dtype, count, name))
    cases.append((torch.bfloat16, 131072, "SUM"))       # the 256 KiB decode message
    cases.append((torch.float32, FUSED_MAX_BYTES // 4, "SUM"))
    # the same on few compute units: exactly four tiles per wavefront, an uneven split, one workgroup
    forced = {}
    for dtype, count, units in ((torch.bfloat16, 131072, 4), (torch.float32, FUSED_MAX_BYTES // 4, 16), (torch.float32, FUSED_MAX_BYTES // 4 - 5, 17),
                                (torch.bfloat16, 131072 - 9, 5), (torch.int8, 64 << 10, 1), (torch.float64, 3 * 1024 + 1, 1)):
        forced[len(cases)] = units
        cases.append((dtype, count, "SUM"))
    pending = []
    epoch = 0
    for i, (dtype, count, name) in enumerate(cases):
        seed = 4000 + i
        scale = 1.0 if name == "PROD" else 0.02
        cpu_in = [rank_buffer(count, dtype, r, seed=seed, scale=scale) for r in range(world)]
        want = oracle_reduce_bits(cpu_in, ops[name][1])
        x = cpu_in[rank].to(DEV)
        in_place = i % 2 == 0
        out = x if in_place else torch.empty_like(x)
        epoch += 1
        slot = epoch & 1
        # every third call as many workgroups as the message has 16 KiB pieces, the others limited to
        # 128 / world of them (the limit bites from 256 KiB on) or to what the message just fits in
        units = forced.get(i, (0, 128 // world, max(1, -(-count * dtype.itemsize // (64 << 10))))[i % 3])
        if units == 0 and count * dtype.itemsize * world > (2 << 20):
            units = 256 // world  # all ranks' launches must be resident together, with room to spare
        capi.check(L.mccl_allreduce_fused(x.data_ptr(), out.data_ptr(), count, TORCH_TO_CODE[dtype], ops[name][0],
                                          tables[slot][0], tables[slot][1], world, rank, epoch, 5_000_000,
                                          st.data_ptr(), units, stream))
        pending.append((out, want, (str(dtype), count, name, in_place)))
        if len(pending) >= 64:
            torch.cuda.synchronize()
            assert st.tolist() == [0, 0], st.tolist()
            for o, w, what in pending:
                assert_bits_equal(bits(o), w, what)
            pending = []
    torch.cuda.synchronize()
    for o, w, what in pending:
        assert_bits_equal(bits(o), w, what)
    assert st.tolist() == [0, 0], st.tolist()
    # the same message many times back to back (the decode loop): every call sees the current inputs
    count = 131072
    base = [rank_buffer(count, torch.bfloat16, r, seed=77) for r in range(world)]
    x = base[rank].to(DEV)
    outs = []
    for it in range(50):
        epoch += 1
        slot = epoch & 1
        out = torch.empty_like(x)
        capi.check(L.mccl_allreduce_fused(x.data_ptr(), out.data_ptr(), count, capi.BF16, capi.SUM,
                                          tables[slot][0], tables[slot][1], world, rank, epoch, 5_000_000,
                                          st.data_ptr(), (0, 4)[it & 1], stream))
        outs.append(out)
        x = out  # the next round reduces the previous result: any stale read changes every later round
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    cur = base
    for it in range(50):
        want = oracle_reduce_bits(cur, O.SUM)
        assert_bits_equal(bits(outs[it]), want, "chained round %d" % it)
        red = torch.from_numpy(want.view(np.int16).copy()).view(torch.bfloat16)
        cur = [red for _ in range(world)]
    barrier.wait(timeout=120)


def fused_replay_case(rank, world, queues, barrier):
    """mccl_allreduce_fused_replayable -- the epoch and the choice of buffer set live on the device and
    are advanced by the launch itself -- against the oracle, bit for bit: eager calls, then launches
    recorded in a HIP graph and replayed with fresh inputs, with eager calls between the replays."""
    from helpers import TORCH_TO_CODE, assert_bits_equal, bits, oracle_reduce_bits, rank_buffer
    from oracle import oracle as O
    from torch_ccl_amd import capi
    L = capi.lib()
    stage_stride = FUSED_MAX_BYTES + 64
    flags_stride = (FUSED_MAX_BYTES // TILE + 1) * 4
    stage = torch.zeros(2 * stage_stride, dtype=torch.uint8, device=DEV)          # both sets, one allocation
    tflag = torch.zeros(2 * flags_stride // 4, dtype=torch.int32, device=DEV)
    state = torch.zeros(capi.FUSED_STATE_BYTES // 4, dtype=torch.int32, device=DEV)  # this rank's own
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, [stage, tflag])
    stages = capi.ptr_table([shared[r][0].data_ptr() for r in range(world)])
    flags = capi.ptr_table([shared[r][1].data_ptr() for r in range(world)])
    st = _status()

    def call(x, out, count, dtype, op, units=0, flags_=0):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        capi.check(L.mccl_allreduce_fused_replayable(x.data_ptr(), out.data_ptr(), count, TORCH_TO_CODE[dtype], op, stages, flags,
                                                     stage_stride, flags_stride, state.data_ptr(), world, rank, 5_000_000,
                                                     st.data_ptr(), units, flags_, stream))

    ops = {"SUM": (capi.SUM, O.SUM), "AVG": (capi.AVG, O.AVG), "MAX": (capi.MAX, O.MAX)}
    launches = 0
    pending = []
    for i, (dtype, count, name, units) in enumerate([(torch.bfloat16, 131072, "SUM", 128 // world), (torch.float32, 7, "SUM", 0), (torch.bfloat16, 1025, "AVG", 0),
                                                    (torch.float32, FUSED_MAX_BYTES // 4, "SUM", 128 // world), (torch.int8, 40_001, "MAX", 1),
                                                    (torch.float16, 5 * 512 - 1, "AVG", 2), (torch.float64, 3 * 1024 + 1, "SUM", 1),
                                                    (torch.bfloat16, 131072 - 9, "SUM", 5), (torch.int64, 129, "SUM", 0)]):
        cpu_in = [rank_buffer(count, dtype, r, seed=6000 + i) for r in range(world)]
        x = cpu_in[rank].to(DEV)
        out = x if i % 2 == 0 else torch.empty_like(x)
        call(x, out, count, dtype, ops[name][0], units)
        launches += 1
        pending.append((out, oracle_reduce_bits(cpu_in, ops[name][1]), ("eager", str(dtype), count, name)))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    for o, w, what in pending:
        assert_bits_equal(bits(o), w, what)
    assert state.cpu().tolist()[0] == launches and state.cpu().tolist()[16] == 0, state.cpu().tolist()

    # recorded: K launches of the decode message with a small kernel of the caller's between them
    K, count, replays = 6, 131072, 12
    pool = [rank_buffer(count + 4096, torch.bfloat16, r, seed=6100) for r in range(world)]
    pool_dev = pool[rank].to(DEV)
    xs = [torch.zeros(count, dtype=torch.bfloat16, device=DEV) for _ in range(K)]
    ticks = torch.zeros(8, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # (a first pass outside the capture, as torch asks for; every rank does the same)
        for k in range(K):
            call(xs[k], xs[k], count, torch.bfloat16, capi.SUM, 128 // world)
            launches += 1
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for k in range(K):
            call(xs[k], xs[k], count, torch.bfloat16, capi.SUM, 128 // world)
            ticks.add_(1.0)
    results = []
    for p in range(replays):
        for k in range(K):
            off = (p * K + k) * 7 % 4096
            xs[k].copy_(pool_dev[off:off + count])
        graph.replay()
        launches += K
        results.append(torch.stack(xs).clone())
        if p % 3 == 2:  # an eager call between two replays: the same counter serves both
            e_in = [rank_buffer(3000 + p, torch.float32, r, seed=6200 + p) for r in range(world)]
            e = e_in[rank].to(DEV)
            call(e, e, 3000 + p, torch.float32, capi.SUM, 0)
            launches += 1
            pending.append((e, oracle_reduce_bits(e_in, O.SUM), ("eager between replays", p)))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    assert ticks.cpu().tolist() == [float(K * replays)] * 8
    for p in range(replays):
        got = results[p].cpu()
        for k in range(K):
            off = (p * K + k) * 7 % 4096
            want = oracle_reduce_bits([pool[r][off:off + count] for r in range(world)], O.SUM)
            assert_bits_equal(bits(got[k]), want, ("replay", p, k))
    for o, w, what in pending:
        assert_bits_equal(bits(o), w, what)
    assert state.cpu().tolist()[0] == launches and state.cpu().tolist()[16] == 0, (state.cpu().tolist(), launches)
    # the bisecting forms run to their end and keep the counter going; their output is not a result
    y = torch.ones(4096, device=DEV)
    call(y, y, 4096, torch.float32, capi.SUM, 0, capi.FUSED_WORK_ONLY)
    call(y, y, 4096, torch.float32, capi.SUM, 0, capi.FUSED_SYNC_ONLY)
    z_in = [rank_buffer(4096, torch.float32, r, seed=6300) for r in range(world)]
    z = z_in[rank].to(DEV)
    call(z, z, 4096, torch.float32, capi.SUM, 0)
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    assert_bits_equal(bits(z), oracle_reduce_bits(z_in, O.SUM), "after the bisecting forms")
    assert state.cpu().tolist()[0] == launches + 3
    barrier.wait(timeout=120)


def offers_case(rank, world, queues, barrier):
    """mccl_rank_barrier_offers + mccl_allreduce_sync_resolved: where each rank's tensor is travels on
    the device.  Every rank has two "allocations" the peers have mapped (entries 3 and 17 of its
    table, with generations of their own) and two staging buffers; from call to call a rank offers
    a range at another offset of one of them, or its staging buffer.  Bit for bit against the
    oracle, call after call with nothing but the kernels' own waits between them; then an offer at
    a generation the peers have not mapped: reported, nothing written."""
    from helpers import assert_bits_equal, bits, oracle_reduce_bits, rank_buffer
    from oracle import oracle as O
    from torch_ccl_amd import capi
    L = capi.lib()
    BUF = 10 << 20
    allocs = [torch.zeros(BUF, dtype=torch.uint8, device=DEV) for _ in range(2)]   # entries 3 and 17
    stages = [torch.zeros(BUF, dtype=torch.uint8, device=DEV) for _ in range(2)]
    # [0]: the flag word, [8..12) and [16..20): the two offer slots, [64..96) and [96..128): the two rows of offers (alltoall)
    ctl = torch.zeros(128, dtype=torch.int64, device=DEV)
    OUTBOX = 1 << 20
    outbox = torch.zeros(world * OUTBOX, dtype=torch.uint8, device=DEV)  # piece d of this rank's, when it is not offered in place
    counter = torch.zeros(1024, dtype=torch.int32, device=DEV)
    table = torch.zeros(ctypes.sizeof(capi.ImportTable) // 8, dtype=torch.int64, device=DEV)
    resolved = torch.zeros(8, dtype=torch.int64, device=DEV)
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, allocs + stages + [ctl, outbox])
    flags = capi.ptr_table([shared[r][4].data_ptr() for r in range(world)])
    slots = [capi.ptr_table([shared[r][4].data_ptr() + 8 * (8 + 8 * sl) for r in range(world)]) for sl in range(2)]
    rows = [capi.ptr_table([shared[r][4].data_ptr() + 8 * (64 + 32 * sl) for r in range(world)]) for sl in range(2)]
    st = _status()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    entries = (3, 17)

    def gen_of(r, which):
        return 100 * (r + 1) + which

    # this rank's table of the peers' mappings, in stream order, at most eight entries per call
    ups = []
    for r in range(world):
        if r == rank:
            continue
        for which in range(2):
            ups.append(capi.ImportUpdate(r, entries[which], 0, 0, shared[r][which].data_ptr(), gen_of(r, which)))
            ups.append(capi.ImportUpdate(r, capi.OFFER_STAGED, which, 0, shared[r][2 + which].data_ptr(), 0))
        ups.append(capi.ImportUpdate(r, capi.OFFER_STAGED, capi.OFFER_SLOT_OUTBOX, 0, shared[r][5].data_ptr() + rank * OUTBOX, 0))  # rank r's outbox for this rank
    for at in range(0, len(ups), 8):
        chunk = (capi.ImportUpdate * len(ups[at:at + 8]))(*ups[at:at + 8])
        capi.check(L.mccl_import_table_update(table.data_ptr(), chunk, len(ups[at:at + 8]), stream))

    ops = {"SUM": (capi.SUM, O.SUM), "AVG": (capi.AVG, O.AVG), "MAX": (capi.MAX, O.MAX)}
    from helpers import TORCH_TO_CODE
    pending = []
    call = 0
    for i, (dtype, count, name) in enumerate([(torch.bfloat16, (1 << 20) + 77, "SUM"), (torch.float32, 100003, "SUM"), (torch.int8, (3 << 20) + 5, "MAX"),
                                              (torch.float64, 7, "SUM"), (torch.bfloat16, 3, "SUM"), (torch.float16, 1 << 21, "AVG"),
                                              (torch.bfloat16, 4096 * 1024, "SUM"), (torch.float32, 1025, "AVG"), (torch.bfloat16, (2 << 20) + 9, "SUM")]):
        es = torch.empty(0, dtype=dtype).element_size()
        host = [rank_buffer(count, dtype, r, seed=900 + i, scale=0.02) for r in range(world)]
        call += 1
        # what this rank offers this time: by call and rank, so that every mixture occurs
        kind = (call + rank) % 3            # 0, 1: one of its allocations, 2: its staging buffer
        off = ((call * 37 + rank * 11) % 64) * es
        if kind < 2:
            where = allocs[kind][off:off + count * es].view(dtype)
            offer = capi.Offer(entries[kind], 0, gen_of(rank, kind), off, 0)
        else:
            where = stages[call & 1][off:off + count * es].view(dtype)
            offer = capi.Offer(capi.OFFER_STAGED, call & 1, 0, off, 0)
        where.copy_(host[rank])
        if i % 2 == 0:  # a barrier kernel that carries the offers, then the allreduce over the resolved addresses
            capi.check(L.mccl_rank_barrier_offers(flags, world, rank, 4 * call + 1, 5_000_000, st.data_ptr(), ctypes.byref(offer),
                                                  where.data_ptr(), slots[call & 1], table.data_ptr(), resolved.data_ptr(), stream))
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 0, 4 * call + 3, counter.data_ptr(), 5_000_000, st.data_ptr(), 0, 0)
            capi.check(L.mccl_allreduce_sync_resolved(resolved.data_ptr(), count, TORCH_TO_CODE[dtype], ops[name][0], ctypes.byref(sy), stream))
        else:           # one launch that does both, on few compute units
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 4 * call + 1, 4 * call + 3, counter.data_ptr(), 5_000_000,
                            st.data_ptr(), (16, 3)[i % 4 == 1], 0)
            capi.check(L.mccl_allreduce_sync_offers(count, TORCH_TO_CODE[dtype], ops[name][0], ctypes.byref(sy), ctypes.byref(offer),
                                                    where.data_ptr(), slots[call & 1], table.data_ptr(), stream))
        pending.append((where.clone(), oracle_reduce_bits(host, ops[name][1]), (str(dtype), count, name, kind, i % 2)))
    # the shard reduction (reduce_scatter: rank r reduces slice r of every rank's offered input) and the
    # push (allgather: rank r writes its contribution into slice r of every rank's offered output)
    # over the same offers, in both forms
    from helpers import to_carrier
    for i, (dtype, m, name) in enumerate([(torch.bfloat16, 70001, "SUM"), (torch.float32, 4099, "MAX"), (torch.float16, 1 << 17, "AVG"),
                                          (torch.int8, 300007, "SUM"), (torch.float64, 1027, "SUM"), (torch.bfloat16, 1 << 19, "SUM")]):
        es = torch.empty(0, dtype=dtype).element_size()
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(world * m, dtype, r, seed=950 + i, scale=0.02) for r in range(world)]
        call += 1
        kind = (call + rank) % 3
        off = ((call * 37 + rank * 11) % 64) * es
        nbytes = world * m * es
        if kind < 2:
            where = allocs[kind][off:off + nbytes].view(dtype)
            offer = capi.Offer(entries[kind], 0, gen_of(rank, kind), off, 0)
        else:
            where = stages[call & 1][off:off + nbytes].view(dtype)
            offer = capi.Offer(capi.OFFER_STAGED, call & 1, 0, off, 0)
        where.copy_(host[rank])
        out = torch.zeros(m, dtype=dtype, device=DEV)
        if i % 2 == 0:
            capi.check(L.mccl_rank_barrier_offers(flags, world, rank, 4 * call + 1, 5_000_000, st.data_ptr(), ctypes.byref(offer),
                                                  where.data_ptr(), slots[call & 1], table.data_ptr(), resolved.data_ptr(), stream))
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 0, 4 * call + 3, counter.data_ptr(), 5_000_000, st.data_ptr(), 0, 0)
            capi.check(L.mccl_reduce_sync_resolved(resolved.data_ptr(), rank * m * es, out.data_ptr(), m, code, ops[name][0], ctypes.byref(sy), stream))
        else:
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 4 * call + 1, 4 * call + 3, counter.data_ptr(), 5_000_000,
                            st.data_ptr(), 16, 0)
            capi.check(L.mccl_reduce_sync_offers(rank * m * es, out.data_ptr(), m, code, ops[name][0], ctypes.byref(sy), ctypes.byref(offer),
                                                 where.data_ptr(), slots[call & 1], table.data_ptr(), stream))
        want = O.reduce_scatter([to_carrier(h) for h in host], code, ops[name][1], shard_first=rank, shard_num=1)[0]
        pending.append((out, want.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[want.dtype.itemsize]), ("reduce_scatter", str(dtype), m, name, kind, i % 2)))
        # the push: what is offered is the OUTPUT (world * nb bytes), rank r's contribution is nb bytes
        nb = m * es + (i % 3)  # not always a whole number of vectors or elements: bytes
        parts = [rank_buffer(nb, torch.uint8, r, seed=970 + i) for r in range(world)]
        call += 1
        kind = (call + rank) % 3
        off = (call * 5 + rank) % 32
        if kind < 2:
            dest = allocs[kind][off:off + world * nb]
            offer = capi.Offer(entries[kind], 0, gen_of(rank, kind), off, 0)
        else:
            dest = stages[call & 1][off:off + world * nb]
            offer = capi.Offer(capi.OFFER_STAGED, call & 1, 0, off, 0)
        dest.zero_()
        in_place = i % 3 == 1  # the contribution already sits in this rank's slice of its own output
        src = parts[rank].to(DEV)
        if in_place:
            dest[rank * nb:(rank + 1) * nb].copy_(src)
            src = dest[rank * nb:(rank + 1) * nb]
        if i % 2 == 1:
            capi.check(L.mccl_rank_barrier_offers(flags, world, rank, 4 * call + 1, 5_000_000, st.data_ptr(), ctypes.byref(offer),
                                                  dest.data_ptr(), slots[call & 1], table.data_ptr(), resolved.data_ptr(), stream))
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 0, 4 * call + 3, counter.data_ptr(), 5_000_000, st.data_ptr(), 0, 0)
            capi.check(L.mccl_fanout_sync_resolved(src.data_ptr(), resolved.data_ptr(), rank * nb, nb, int(in_place), ctypes.byref(sy), stream))
        else:
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 4 * call + 1, 4 * call + 3, counter.data_ptr(), 5_000_000,
                            st.data_ptr(), 16, 0)
            capi.check(L.mccl_fanout_sync_offers(src.data_ptr(), rank * nb, nb, int(in_place), ctypes.byref(sy), ctypes.byref(offer),
                                                 dest.data_ptr(), slots[call & 1], table.data_ptr(), stream))
        pending.append((dest.clone(), np.concatenate([bits(p) for p in parts]), ("allgather", nb, kind, in_place, i % 2)))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    for got, want, what in pending:
        assert_bits_equal(bits(got), want, what)
    assert int(counter.abs().sum()) == 0
    # alltoall(v): every rank publishes a row of offers -- piece d in place (somewhere in one of its
    # allocations) or in its outbox for rank d -- and pulls the column addressed to it
    def alltoall_round(call, seed, break_length=False):
        rng = np.random.default_rng(seed)
        S = rng.integers(0, 3, size=(world, world)) * rng.integers(1, 200000, size=(world, world)) + rng.integers(0, 2, size=(world, world)) * 13
        S[rng.integers(0, world)][rng.integers(0, world)] = 0
        pieces = [[rng.integers(0, 256, size=int(S[r][d]), dtype=np.uint8) for d in range(world)] for r in range(world)]
        displ = np.concatenate([[0], np.cumsum(S[rank])[:-1]])
        total = int(S[rank].sum())
        kind = (call + rank) % 2
        off = (call * 7 + rank * 3) % 61
        image = allocs[kind][off:off + total]
        if total:
            image.copy_(torch.from_numpy(np.concatenate(pieces[rank])).to(DEV))
        one_launch = (call + rank) % 3 != 0  # the two forms mix among the ranks of one collective
        mine = (capi.Offer * world)()
        stage = []
        for d in range(world):
            nb = int(S[rank][d])
            told = nb + 16 if (break_length and rank == 0 and d == 1) else nb
            if (call + rank + d) % 3 == 0:  # through the outbox for rank d
                if one_launch:
                    stage.append(capi.Segment(image.data_ptr() + int(displ[d]), outbox.data_ptr() + d * OUTBOX, nb))
                else:
                    outbox[d * OUTBOX:d * OUTBOX + nb].copy_(image[int(displ[d]):int(displ[d]) + nb])
                mine[d] = capi.Offer(capi.OFFER_STAGED, capi.OFFER_SLOT_OUTBOX, 0, 0, told)
            else:
                mine[d] = capi.Offer(entries[kind], 0, gen_of(rank, kind), off + int(displ[d]), told)
        expect = (ctypes.c_uint64 * world)(*[int(S[r][rank]) for r in range(world)])
        odispl = np.concatenate([[0], np.cumsum(S[:, rank])[:-1]])
        out = torch.full((int(S[:, rank].sum()) + 64,), 0xee, dtype=torch.uint8, device=DEV)
        segs = (capi.Segment * world)(*[capi.Segment(0, out.data_ptr() + int(odispl[r]), int(S[r][rank])) for r in range(world)])
        src_rank = (ctypes.c_int * world)(*range(world))
        my_source = image.data_ptr() + int(displ[rank])
        if one_launch:
            stage_segs = (capi.Segment * max(1, len(stage)))(*stage)
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 4 * call + 1, 4 * call + 3, counter.data_ptr(), 5_000_000,
                            st.data_ptr(), (16, 2)[call % 2], 0)
            capi.check(L.mccl_alltoall_sync_offers(stage_segs, len(stage), segs, src_rank, world, ctypes.byref(sy), mine, expect, my_source,
                                                   rows[call & 1], table.data_ptr(), stream))
        else:
            capi.check(L.mccl_rank_barrier_offers_each(flags, world, rank, 4 * call + 1, 5_000_000, st.data_ptr(), mine, expect,
                                                        my_source, rows[call & 1], table.data_ptr(), resolved.data_ptr(), stream))
            sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 0, 4 * call + 3, counter.data_ptr(), 5_000_000, st.data_ptr(), 0, 0)
            capi.check(L.mccl_copy_segments_sync_resolved(segs, src_rank, world, resolved.data_ptr(), 0, ctypes.byref(sy), stream))
        want = np.concatenate([pieces[r][rank] for r in range(world)] + [np.full(64, 0xee, dtype=np.uint8)])
        return out, want, S

    pending = []
    for i in range(9):
        call += 1
        out, want, S = alltoall_round(call, seed=1000 + i)
        pending.append((out, want, ("alltoall", i, S.tolist())))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    for got, want, what in pending:
        assert_bits_equal(bits(got), want, what)
    assert int(counter.abs().sum()) == 0
    if world > 1:
        # rank 0 tells rank 1 a length that rank 1 does not expect: rank 1 reports it and leaves that piece alone
        barrier.wait(timeout=120)
        call += 1
        out, want, S = alltoall_round(call, seed=1100, break_length=True)
        torch.cuda.synchronize()
        if rank == 1 and S[0][1] + 16 != S[0][1]:
            assert st.tolist()[0] == 1 and (st.tolist()[1] & 0xffffffff) == capi.STATUS_MISMATCH, st.tolist()
            lo = int(S[:0, 1].sum())
            want[lo:lo + int(S[0][1])] = 0xee
            st.zero_()
        else:
            assert st.tolist() == [0, 0], st.tolist()
        assert_bits_equal(bits(out), want, ("alltoall with a wrong length", rank))
        barrier.wait(timeout=120)
    # rank 0 offers an allocation at a generation nobody has mapped: every other rank reports it
    # and leaves all tensors alone, and every launch still ends
    barrier.wait(timeout=120)
    call += 1
    count = 70001
    where = allocs[0][:count * 4].view(torch.float32)
    where.fill_(float(rank + 1))
    offer = capi.Offer(entries[0], 0, gen_of(rank, 0) + (7 if rank == 0 else 0), 0, 0)
    capi.check(L.mccl_rank_barrier_offers(flags, world, rank, 4 * call + 1, 5_000_000, st.data_ptr(), ctypes.byref(offer),
                                          where.data_ptr(), slots[call & 1], table.data_ptr(), resolved.data_ptr(), stream))
    sy = capi.XSync(ctypes.cast(flags, ctypes.c_void_p), world, rank, 0, 4 * call + 3, counter.data_ptr(), 5_000_000, st.data_ptr(), 0, 0)
    capi.check(L.mccl_allreduce_sync_resolved(resolved.data_ptr(), count, capi.F32, capi.SUM, ctypes.byref(sy), stream))
    torch.cuda.synchronize()
    if rank == 0:
        assert st.tolist() == [0, 0], st.tolist()
    else:
        assert st.tolist()[0] == 1 and (st.tolist()[1] & 0xffffffff) == capi.STATUS_UNMAPPED, st.tolist()
    barrier.wait(timeout=120)
    # (rank 0 itself resolved everybody and reduced its shard: only that shard of the tensors has changed)
    shard = L.mccl_allreduce_sync_shard(count, world)
    assert bool((where[shard:] == float(rank + 1)).all())
    barrier.wait(timeout=120)


def xrank_case(rank, world, queues, barrier):
    """The one-launch collectives that read the peers' buffers in place -- mccl_reduce_sync
    (reduce_scatter shard), mccl_allreduce_sync (in-place allreduce) and mccl_copy_segments_sync
    (alltoallv pull) -- against the oracle, bit for bit, call after call on the same shared buffers
    with nothing but the kernels' own waits between them."""
    from helpers import TORCH_TO_CODE, assert_bits_equal, bits, oracle_reduce_bits, rank_buffer, to_carrier
    from oracle import oracle as O
    from torch_ccl_amd import capi
    L = capi.lib()
    BUF = 24 << 20
    shared_in = torch.zeros(BUF, dtype=torch.uint8, device=DEV)      # what the peers read in place
    word = torch.zeros(8, dtype=torch.int64, device=DEV)             # [0]: the sync word
    counter = torch.zeros(1024, dtype=torch.int32, device=DEV)  # MCCL_SYNC_COUNTER_BYTES
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, [shared_in, word])
    words = capi.ptr_table([shared[r][1].data_ptr() for r in range(world)])
    st = _status()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    call = [0]

    def sync(done=True):
        call[0] += 1
        # every third call as single wavefronts all over the GPU, the others as at most 16 or 2
        # workgroups of sixteen wavefronts
        return capi.XSync(ctypes.cast(words, ctypes.c_void_p), world, rank, 4 * call[0] + 1, 4 * call[0] + 3 if done else 0,
                          counter.data_ptr(), 5_000_000, st.data_ptr(), (0, 16, 2)[call[0] % 3], 0)

    def mine(dtype, count, off):
        return shared_in[off:off + count * torch.empty(0, dtype=dtype).element_size()].view(dtype)

    ops = {"SUM": (capi.SUM, O.SUM), "PROD": (capi.PROD, O.PROD), "MIN": (capi.MIN, O.MIN), "MAX": (capi.MAX, O.MAX),
           "AVG": (capi.AVG, O.AVG)}
    checks = []
    # reduce_scatter shard: rank r reduces slice r of every rank's buffer
    for i, (dtype, m, name, off) in enumerate([(torch.bfloat16, 70001, "SUM", 0), (torch.float32, 4099, "MAX", 4), (torch.int8, 300007, "SUM", 1),
                                              (torch.float64, 1, "PROD", 8), (torch.float16, 1 << 19, "SUM", 16), (torch.int64, 33, "MIN", 0),
                                              (torch.bfloat16, 1 << 20, "SUM", 2), (torch.bfloat16, 70001, "AVG", 2), (torch.float32, 4099, "AVG", 0),
                                              (torch.float16, 515, "AVG", 6), (torch.float64, 1027, "AVG", 8)]):
        es = torch.empty(0, dtype=dtype).element_size()
        off = off // es * es
        host = [rank_buffer(world * m, dtype, r, seed=300 + i, scale=1.0 if name == "PROD" else 0.02) for r in range(world)]
        mine(dtype, world * m, off).copy_(host[rank])
        out = torch.empty(m, dtype=dtype, device=DEV)
        ins = capi.ptr_table([shared[r][0].data_ptr() + off + rank * m * es for r in range(world)])
        sy = sync()
        capi.check(L.mccl_reduce_sync(ins, out.data_ptr(), m, TORCH_TO_CODE[dtype], ops[name][0], ctypes.byref(sy), stream))
        want = oracle_reduce_bits([h[rank * m:(rank + 1) * m] for h in host], ops[name][1])
        checks.append((out, want, ("reduce_sync", str(dtype), m, name)))
    # allreduce in place on the shared buffer: every owner writes its finished shard into every
    # rank's tensor; the clone behind it reads what the peers wrote
    for i, (dtype, count, name, off) in enumerate([(torch.bfloat16, (2 << 20) + 77, "SUM", 0), (torch.float32, 1025, "SUM", 4), (torch.int8, (3 << 20) + 5, "MAX", 3),
                                                  (torch.float64, 7, "SUM", 8), (torch.bfloat16, 3, "MIN", 2), (torch.float16, 1 << 21, "SUM", 0),
                                                  (torch.int32, 100003, "PROD", 4), (torch.bfloat16, 4096 * 1024, "SUM", 0), (torch.uint8, 1, "SUM", 5),
                                                  (torch.bfloat16, 4096 * 1024, "SUM", 6), (torch.bfloat16, (1 << 20) + 77, "AVG", 0),
                                                  (torch.float32, 100003, "AVG", 4), (torch.float16, 1025, "AVG", 2), (torch.float64, 4097, "AVG", 8)]):
        es = torch.empty(0, dtype=dtype).element_size()
        off = off // es * es
        host = [rank_buffer(count, dtype, r, seed=450 + i, scale=1.0 if name == "PROD" else 0.02) for r in range(world)]
        t = mine(dtype, count, off)
        t.copy_(host[rank])
        sy = sync()
        capi.check(L.mccl_allreduce_sync(capi.ptr_table([shared[r][0].data_ptr() + off for r in range(world)]),
                                         count, TORCH_TO_CODE[dtype], ops[name][0], ctypes.byref(sy), stream))
        want = oracle_reduce_bits(host, ops[name][1])
        checks.append((t.clone(), want, ("allreduce_sync", str(dtype), count, name)))
    # alltoallv pull: rank d copies its segment out of every rank's buffer
    rng = np.random.default_rng(99)
    for i in range(4):
        S = rng.integers(0, 4000, size=(world, world))
        S[rng.integers(0, world), rng.integers(0, world)] = 0
        row = (16, 96, 2, 1024)[i]
        host = [rank_buffer(int(S[r].sum()) * row, torch.uint8, r, seed=500 + i) for r in range(world)]
        mine(torch.uint8, host[rank].numel(), 0).copy_(host[rank])
        out = torch.zeros(int(S[:, rank].sum()) * row, dtype=torch.uint8, device=DEV)
        segs, roff = [], 0
        for r in range(world):
            b = int(S[r, rank]) * row
            if b:
                segs.append(capi.Segment(shared[r][0].data_ptr() + int(S[r, :rank].sum()) * row, out.data_ptr() + roff, b))
            roff += b
        arr = (capi.Segment * max(1, len(segs)))(*segs)
        sy = sync()
        capi.check(L.mccl_copy_segments_sync(arr, len(segs), i & 1, ctypes.byref(sy), stream))  # both load flavours
        want = O.alltoallv([to_carrier(h) for h in host], S, row)[rank]
        checks.append((out, want, ("copy_segments_sync", row, i)))
    # allgather as pushes: every rank writes its contribution into slice `rank` of every rank's shared
    # buffer; the clone behind the call reads what the peers wrote.  Odd lengths and offsets included.
    for i, (nbytes, src_off, dst_off) in enumerate([(1 << 20, 0, 0), (70001, 3, 5), (15, 1, 0), (16, 0, 16), (1, 0, 7), ((2 << 20) + 48, 16, 32),
                                                    (1024, 0, 0), (0, 0, 0), (333333, 8, 1)]):
        host = [rank_buffer(max(nbytes, 1), torch.uint8, r, seed=700 + i)[:nbytes] for r in range(world)]
        own = torch.empty(nbytes + 64, dtype=torch.uint8, device=DEV)[src_off:src_off + nbytes]
        own.copy_(host[rank])
        dst = capi.ptr_table([shared[r][0].data_ptr() + dst_off + rank * nbytes for r in range(world)])
        sy = sync()
        capi.check(L.mccl_fanout_sync(own.data_ptr(), dst, world, nbytes, ctypes.byref(sy), stream))
        got = shared_in[dst_off:dst_off + world * nbytes].clone()
        want = O.allgather([to_carrier(h) for h in host]) if nbytes else np.zeros(0, np.uint8)
        checks.append((got, want, ("fanout_sync", nbytes, src_off, dst_off)))
    torch.cuda.synchronize()
    assert st.tolist() == [0, 0], st.tolist()
    assert not counter.cpu().any()  # every counter is back at zero
    for o, w, what in checks:
        assert_bits_equal(bits(o), np.asarray(w).view(bits(o).dtype) if np.asarray(w).dtype != bits(o).dtype else w, what)
    barrier.wait(timeout=120)


def timeout_case(rank, world, queues, barrier):
    """A peer that never signals: the waiting kernels end by themselves at their (tiny) limit, name
    the late rank, and leave the output alone.  Rank 1 simply does not call."""
    from torch_ccl_amd import capi
    L = capi.lib()
    flag = torch.zeros(8, dtype=torch.int64, device=DEV)
    stage = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    tflag = torch.zeros(8, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    shared = _exchange(rank, world, queues, barrier, [flag, stage, tflag])
    if rank != 1:
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        st = _status()
        flags = capi.ptr_table([shared[r][0].data_ptr() for r in range(world)])
        capi.check(L.mccl_rank_barrier(flags, world, rank, 5, 200_000, st.data_ptr(), stream))
        torch.cuda.synchronize()
        assert st.tolist() == [2, 5], st.tolist()  # 1 + the late rank, the epoch
        st.zero_()
        x = torch.full((256,), float(rank + 1), device=DEV)
        out = torch.full((256,), -7.0, device=DEV)
        capi.check(L.mccl_allreduce_fused(
            x.data_ptr(), out.data_ptr(), 256, capi.F32, capi.SUM,
            capi.ptr_table([shared[r][1].data_ptr() for r in range(world)]),
            capi.ptr_table([shared[r][2].data_ptr() for r in range(world)]), world, rank, 9, 200_000,
            st.data_ptr(), 0, stream))
        torch.cuda.synchronize()
        assert st.tolist() == [2, 9], st.tolist()
        assert out.cpu().tolist() == [-7.0] * 256
    barrier.wait(timeout=120)


def run_rank(rank, world, queues, barrier, mode):
    torch.set_num_threads(max(1, (os.cpu_count() or 16) // world))  # the ranks share the host's cores
    torch.cuda.set_device(0)
    {"barrier": barrier_case, "fused": fused_case, "fused_replay": fused_replay_case, "timeout": timeout_case,
     "xrank": xrank_case, "offers": offers_case}[mode](rank, world, queues, barrier)
    torch.cuda.synchronize()
