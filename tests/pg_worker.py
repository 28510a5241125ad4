"""Rank body for the backend tests: N ranks (processes or threads) share cuda:0 and replay the
reference's functional cases (tests/test_c10d_ccl.py, via tests/golden/c10d_kats.json) plus
seeded random cases checked bit for bit against the CPU oracle."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "torch-ccl_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402
import torch  # noqa: E402
import torch.distributed as dist  # noqa: E402
import torch.distributed.distributed_c10d as c10d  # noqa: E402

DEV = "cuda:0"


def _kats(world):
    with open(os.path.join(ROOT, "tests", "golden", "c10d_kats.json")) as f:
        return json.load(f)["world_sizes"][str(world)]


def _dev(x, dtype=None):
    return torch.tensor(x, dtype=dtype).to(DEV)


def reference_cases(pg, rank, world):
    """The closed-form cases of the reference's ProcessGroupCCLTest, on GPU tensors."""
    K = _kats(world)
    ops = {"SUM": c10d.ReduceOp.SUM, "PRODUCT": c10d.ReduceOp.PRODUCT, "MIN": c10d.ReduceOp.MIN,
           "MAX": c10d.ReduceOp.MAX}
    # allreduce basics (:173-187)
    for name, want in K["allreduce"]["expected"].items():
        opts = c10d.AllreduceOptions()
        opts.reduceOp = ops[name]
        t = _dev(K["allreduce"]["inputs"][rank])
        pg.allreduce([t], opts).wait()
        assert t.cpu().tolist() == want, (name, t.cpu().tolist(), want)
    # allreduce_coalesced (:200-209)
    ts = [_dev(v, torch.float32) for v in K["allreduce_coalesced"]["inputs"][rank]]
    opts = c10d.AllreduceCoalescedOptions()
    opts.reduceOp = c10d.ReduceOp.SUM
    pg.allreduce_coalesced(ts, opts).wait()
    for t, want in zip(ts, K["allreduce_coalesced"]["expected"]):
        assert t.cpu().tolist() == want
    # _reduce_scatter_base (:550-566)
    out = torch.empty(1, device=DEV)
    pg._reduce_scatter_base(out, _dev(K["reduce_scatter_base"]["inputs"][rank], torch.float32)).wait()
    assert out.cpu().tolist() == K["reduce_scatter_base"]["expected"][rank]
    # reduce_scatter, list form (:579-610) and variable-length slots (:623-653)
    for key in ("reduce_scatter_list", "reduce_scatter_list_variable"):
        want = K[key]["expected"][rank]
        out = [_dev([0] * len(want))]
        ins = [[_dev(v) for v in K[key]["inputs"][rank]]]
        opts = c10d.ReduceScatterOptions()
        opts.reduceOp = c10d.ReduceOp.SUM
        pg.reduce_scatter(out, ins, opts).wait()
        assert out[0].cpu().tolist() == want, (key, out[0].cpu().tolist(), want)
    # _allgather_base (:377-391) and its error strings (:404-429)
    out = torch.empty(world, dtype=torch.int64, device=DEV)
    pg._allgather_base(out, _dev(K["allgather_base"]["inputs"][rank])).wait()
    assert out.cpu().tolist() == K["allgather_base"]["expected"]
    try:
        pg._allgather_base(torch.empty(world + 1, dtype=torch.int64, device=DEV), _dev([rank]))
        raise AssertionError("size check did not fire")
    except RuntimeError as e:
        assert "output tensor size must be equal to world_size times input tensor size" in str(e)
    try:
        pg._allgather_base(torch.empty(world + 1, dtype=torch.int64, device=DEV), _dev([rank], torch.float32))
        raise AssertionError("dtype check did not fire")
    except RuntimeError as e:
        assert "Tensors are not equal in data type" in str(e)
    # allgather, list form (:345-364)
    for sub in K["allgather_list"]:
        outs = [[_dev([-1]) for _ in range(world)]]
        pg.allgather(outs, [_dev(sub["inputs"][rank])]).wait()
        assert [t.cpu().tolist() for t in outs[0]] == sub["expected"]
    # alltoall_base, equal (:443-456) and uneven (:458-473) splits
    out = torch.ones(world, world, device=DEV) * -1
    pg.alltoall_base(out, _dev(K["alltoall_base_equal"]["inputs"][rank], torch.float32), [], []).wait()
    assert out.cpu().tolist() == K["alltoall_base_equal"]["expected"][rank]
    U = K["alltoall_base_unequal"]
    out = torch.ones((rank + 1) * world, world, device=DEV)
    pg.alltoall_base(out, _dev(U["inputs"][rank], torch.float32), U["out_splits"][rank], U["in_splits"][rank]).wait()
    assert out.cpu().tolist() == U["expected"][rank]
    # alltoall, list form (:498-518)
    L = K["alltoall_list"]
    outs = [torch.ones(rank + 1, world, device=DEV) for _ in range(world)]
    pg.alltoall(outs, [_dev(v, torch.float32) for v in L["inputs"][rank]]).wait()
    assert [t.cpu().tolist() for t in outs] == L["expected"][rank]
    # reduce to each root in turn (:221-237): the allreduce closed forms, on the root only
    for name, want in K["reduce"]["expected"].items():
        for root in K["reduce"]["roots"]:
            opts = c10d.ReduceOptions()
            opts.reduceOp = ops[name]
            opts.rootRank = root
            t = _dev(K["reduce"]["inputs"][rank])
            pg.reduce([t], opts).wait()
            if rank == root:
                assert t.cpu().tolist() == want, (name, root, t.cpu().tolist(), want)
            else:
                assert t.cpu().tolist() == K["reduce"]["inputs"][rank]  # untouched off the root
    # gather, every rank root in turn, work items collected first (:254-277)
    outputs = [_dev([-1]) for _ in range(world)]
    work = []
    for root in K["gather"]["roots"]:
        opts = c10d.GatherOptions()
        opts.rootRank = root
        work.append(pg.gather([outputs] if root == rank else [], [_dev(K["gather"]["inputs"][rank])], opts))
    for w in work:
        w.wait()
    assert [t.cpu().tolist() for t in outputs] == K["gather"]["expected"]
    try:
        opts = c10d.GatherOptions()
        opts.rootRank = (rank + 1) % world
        pg.gather([outputs], [_dev([rank])], opts)
        raise AssertionError("non-root output check did not fire")
    except RuntimeError as e:
        assert "gather: number of output tensors should be 0 for non-root" in str(e)
    # scatter from each root in turn (:290-308)
    for root in K["scatter"]["roots"]:
        opts = c10d.ScatterOptions()
        opts.rootRank = root
        output = [_dev([-1])]
        pg.scatter(output, [[_dev(v) for v in K["scatter"]["inputs"]]] if root == rank else [], opts).wait()
        assert output[0].cpu().tolist() == K["scatter"]["expected"][rank]
    try:
        opts = c10d.ScatterOptions()
        opts.rootRank = rank
        pg.scatter([_dev([-1])], [[_dev([0])] * (world + 1)], opts)
        raise AssertionError("input list check did not fire")
    except ValueError as e:
        assert "Incorrect input list size" in str(e)
    # broadcast root check (:109-113)
    try:
        opts = c10d.BroadcastOptions()
        opts.rootRank = -1
        opts.rootTensor = 0
        pg.broadcast([torch.zeros(1, device=DEV)], opts)
        raise AssertionError("rank check did not fire")
    except ValueError as e:
        assert "unexpected rank" in str(e)
    # broadcast data (each root in turn)
    for root in range(world):
        opts = c10d.BroadcastOptions()
        opts.rootRank = root
        opts.rootTensor = 0
        t = torch.full((1000,), float(rank), device=DEV)
        pg.broadcast([t], opts).wait()
        assert t.cpu().tolist() == [float(root)] * 1000
    pg.barrier().wait()


def oracle_cases(pg, rank, world):
    """Seeded random buffers: every rank rebuilds all ranks' inputs on the CPU, runs the oracle
    and compares its own GPU result bit for bit."""
    from helpers import TORCH_TO_CODE, bits, rank_buffer, to_carrier
    from oracle import oracle as O

    def bits_np(arr):
        return arr.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[arr.dtype.itemsize])

    for dtype in (torch.bfloat16, torch.float16, torch.float32, torch.int32):
        code = TORCH_TO_CODE[dtype]
        for count in (1, 1000, 131072, (1 << 20) + 3):
            host = [rank_buffer(count, dtype, r, seed=99) for r in range(world)]
            t = host[rank].to(DEV)
            pg.allreduce([t], c10d.AllreduceOptions()).wait()
            want = bits_np(O.reduce([to_carrier(h) for h in host], code, O.SUM))
            assert np.array_equal(bits(t), want), ("allreduce", dtype, count)
        # reduce_scatter_tensor
        m = 4099
        host = [rank_buffer(world * m, dtype, r, seed=7) for r in range(world)]
        out = torch.empty(m, dtype=dtype, device=DEV)
        pg._reduce_scatter_base(out, host[rank].to(DEV)).wait()
        want = O.reduce_scatter([to_carrier(h) for h in host], code, O.SUM, shard_first=rank, shard_num=1)[0]
        assert np.array_equal(bits(out), bits_np(want)), ("reduce_scatter", dtype)
        # all_gather_into_tensor
        host = [rank_buffer(m, dtype, r, seed=8) for r in range(world)]
        out = torch.empty(world * m, dtype=dtype, device=DEV)
        pg._allgather_base(out, host[rank].to(DEV)).wait()
        assert np.array_equal(bits(out), np.concatenate([bits(h) for h in host])), ("allgather", dtype)
        out.zero_()
        n_in = host[rank].numel()
        out[rank * n_in:(rank + 1) * n_in].copy_(host[rank])
        pg._allgather_base(out, out[rank * n_in:(rank + 1) * n_in]).wait()  # in place
        assert np.array_equal(bits(out), np.concatenate([bits(h) for h in host])), ("allgather in place", dtype)
    # two-shot path (>= 4 MiB, >= 4 ranks): ragged counts, every dtype width, same bits as the oracle
    for dtype, count in ((torch.bfloat16, (4 << 20) + 777), (torch.float32, (2 << 20) + 5), (torch.int8, (8 << 20) + 3),
                         (torch.float64, (1 << 20) + 1)):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(count, dtype, r, seed=21) for r in range(world)]
        t = host[rank].to(DEV)
        pg.allreduce([t], c10d.AllreduceOptions()).wait()
        want = bits_np(O.reduce([to_carrier(h) for h in host], code, O.SUM))
        assert np.array_equal(bits(t), want), ("two-shot allreduce", dtype, count)
    # MIN / MAX / PRODUCT / AVG on floats
    for opname, op, ocode in (("min", c10d.ReduceOp.MIN, O.MIN), ("max", c10d.ReduceOp.MAX, O.MAX),
                              ("prod", c10d.ReduceOp.PRODUCT, O.PROD)):
        host = [rank_buffer(5000, torch.float32, r, seed=11, scale=1.0) for r in range(world)]
        t = host[rank].to(DEV)
        opts = c10d.AllreduceOptions()
        opts.reduceOp = op
        pg.allreduce([t], opts).wait()
        assert np.array_equal(bits(t), bits_np(O.reduce([to_carrier(h) for h in host], O.F32, ocode))), opname
    # AVG against the oracle's (sum in ascending rank order at the accumulation width, one division,
    # one rounding): through the one-launch small allreduce, the in-place allreduce of the peers'
    # tensors (from 1 MiB on), the two-shot form and reduce_scatter_tensor
    for dtype, count in ((torch.bfloat16, 131072), (torch.float32, 1000), (torch.bfloat16, (1 << 20) + 77), (torch.float32, (1 << 19) + 3),
                         (torch.float16, (3 << 20) + 1), (torch.float64, (1 << 20) + 5), (torch.bfloat16, (4 << 20) + 777)):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(count, dtype, r, seed=12, scale=1.0) for r in range(world)]
        t = host[rank].to(DEV)
        opts = c10d.AllreduceOptions()
        opts.reduceOp = c10d.ReduceOp.AVG
        pg.allreduce([t], opts).wait()
        assert np.array_equal(bits(t), bits_np(O.reduce([to_carrier(h) for h in host], code, O.AVG))), ("avg", dtype, count)
    for dtype, m in ((torch.bfloat16, 70001), (torch.float32, (1 << 18) + 9)):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(world * m, dtype, r, seed=13, scale=1.0) for r in range(world)]
        out = torch.empty(m, dtype=dtype, device=DEV)
        opts = c10d.ReduceScatterOptions()
        opts.reduceOp = c10d.ReduceOp.AVG
        pg._reduce_scatter_base(out, host[rank].to(DEV), opts).wait()
        want = O.reduce_scatter([to_carrier(h) for h in host], code, O.AVG, shard_first=rank, shard_num=1)[0]
        assert np.array_equal(bits(out), bits_np(want)), ("reduce_scatter avg", dtype)
    # rooted reduce: only the root's tensor changes, to the oracle's bits
    for dtype, count, op, ocode in ((torch.bfloat16, 300001, c10d.ReduceOp.SUM, O.SUM), (torch.float32, 77, c10d.ReduceOp.MAX, O.MAX),
                                    (torch.int64, 4097, c10d.ReduceOp.PRODUCT, O.PROD)):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(count, dtype, r, seed=31) for r in range(world)]
        root = count % world
        t = host[rank].to(DEV)
        opts = c10d.ReduceOptions()
        opts.reduceOp = op
        opts.rootRank = root
        pg.reduce([t], opts).wait()
        want = bits_np(O.reduce([to_carrier(h) for h in host], code, ocode)) if rank == root else bits(host[rank])
        assert np.array_equal(bits(t), want), ("reduce", dtype, count)
    # gather and scatter of odd-sized byte tensors, byte for byte
    root = world - 1
    host = [rank_buffer(10007, torch.int8, r, seed=41) for r in range(world)]
    outs = [torch.zeros(10007, dtype=torch.int8, device=DEV) for _ in range(world)]
    opts = c10d.GatherOptions()
    opts.rootRank = root
    pg.gather([outs] if rank == root else [], [host[rank].to(DEV)], opts).wait()
    if rank == root:
        for r in range(world):
            assert np.array_equal(bits(outs[r]), bits(host[r])), ("gather", r)
    out = torch.zeros(10007, dtype=torch.int8, device=DEV)
    opts = c10d.ScatterOptions()
    opts.rootRank = root
    pg.scatter([out], [[h.to(DEV) for h in host]] if rank == root else [], opts).wait()
    assert np.array_equal(bits(out), bits(host[rank])), "scatter"
    # uneven all_to_all_single: a seeded split matrix every rank agrees on
    rng = np.random.default_rng(1234)
    S = rng.integers(0, 300, size=(world, world))
    S[0, world - 1] = 0
    hidden = 96
    host = [rank_buffer(int(S[r].sum()) * hidden, torch.bfloat16, r, seed=5).view(-1, hidden) for r in range(world)]
    out = torch.zeros(int(S[:, rank].sum()), hidden, dtype=torch.bfloat16, device=DEV)
    pg.alltoall_base(out, host[rank].to(DEV), S[:, rank].tolist(), S[rank].tolist()).wait()
    want = O.alltoallv([to_carrier(h) for h in host], S, hidden * 2)[rank]
    assert np.array_equal(out.cpu().view(torch.uint8).numpy().reshape(-1), want), "alltoallv"
    pg.barrier().wait()


def dist_api_cases(rank, world):
    """The public torch.distributed entry points on the default group (backend "ccl")."""
    t = torch.full((1 << 16,), float(rank + 1), device=DEV)
    dist.all_reduce(t)
    assert torch.equal(t.cpu(), torch.full((1 << 16,), world * (world + 1) / 2.0))
    w = dist.all_reduce(t, async_op=True)
    w.wait()
    torch.cuda.synchronize()
    assert float(t[0]) == world * world * (world + 1) / 2.0
    fut = dist.all_reduce(t, async_op=True).get_future()
    fut.wait()
    assert float(t[123]) == world ** 2 * world * (world + 1) / 2.0
    # reduce_scatter_tensor / all_gather_into_tensor / all_to_all_single
    inp = torch.arange(world * 4, dtype=torch.float32, device=DEV)
    out = torch.empty(4, device=DEV)
    dist.reduce_scatter_tensor(out, inp)
    assert out.cpu().tolist() == [world * (rank * 4 + j) for j in range(4)]
    gathered = torch.empty(world * 3, device=DEV)
    dist.all_gather_into_tensor(gathered, torch.full((3,), float(rank), device=DEV))
    assert gathered.cpu().tolist() == [float(r) for r in range(world) for _ in range(3)]
    a2a = torch.empty(world * 2, device=DEV)
    dist.all_to_all_single(a2a, torch.full((world * 2,), float(rank), device=DEV))
    assert a2a.cpu().tolist() == [float(r) for r in range(world) for _ in range(2)]
    # AVG
    t = torch.full((100,), float(rank), device=DEV)
    dist.all_reduce(t, op=dist.ReduceOp.AVG)
    assert torch.equal(t.cpu(), torch.full((100,), (world - 1) / 2.0))  # small integers over W: exact in fp32 for these world sizes
    # coalescing manager (:667-693): two 8-element allreduces equal one 16-element allreduce
    small = [torch.ones(8, device=DEV) for _ in range(2)]
    with c10d._coalescing_manager(device=torch.device(DEV)):
        for s in small:
            dist.all_reduce(s)
    torch.cuda.synchronize()
    big = torch.ones(16, device=DEV)
    dist.all_reduce(big)
    for i in range(2):
        assert torch.equal(small[i].cpu(), big[i * 8:(i + 1) * 8].cpu())
    # reduce_scatter_tensor of ones (:716-733)
    o = torch.zeros(2, 2, device=DEV)
    dist.reduce_scatter_tensor(o, torch.ones(world * 2, 2, device=DEV))
    assert torch.equal(o.cpu(), torch.full((2, 2), float(world)))
    # many asynchronous all_reduces of mixed sizes in flight before the first wait: small ones run on
    # the caller's stream, large ones on the communication stream, the two staging slots alternate
    rng = np.random.default_rng(77)
    sizes = [int(x) for x in rng.choice([1, 300, 70_000, 300_000, 1_100_000, 2_500_000], size=40)]
    ts = [torch.full((n,), float(rank + 1 + i % 3), device=DEV) for i, n in enumerate(sizes)]
    works = [dist.all_reduce(t, async_op=True) for t in ts]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for i, t in enumerate(ts):
        want = float(sum(r + 1 + i % 3 for r in range(world)))
        assert float(t.min()) == want == float(t.max()), ("async all_reduce", i, sizes[i])
    del ts, works
    # rooted collectives through the public API
    t = torch.full((10,), float(rank + 1), device=DEV)
    dist.reduce(t, dst=world - 1)
    if rank == world - 1:
        assert t.cpu().tolist() == [world * (world + 1) / 2.0] * 10
    got = [torch.zeros(3, device=DEV) for _ in range(world)] if rank == 0 else None
    dist.gather(torch.full((3,), float(rank), device=DEV), got, dst=0)
    if rank == 0:
        assert [g.cpu().tolist() for g in got] == [[float(r)] * 3 for r in range(world)]
    piece = torch.zeros(2, device=DEV)
    dist.scatter(piece, [torch.full((2,), float(10 + r), device=DEV) for r in range(world)] if rank == 1 else None, src=1)
    assert piece.cpu().tolist() == [float(10 + rank)] * 2
    # point to point through the public API: blocking pair, then isend / irecv round the ring
    if rank == 0:
        dist.send(torch.arange(6, dtype=torch.float32, device=DEV), dst=1)
    elif rank == 1:
        r = torch.zeros(6, device=DEV)
        dist.recv(r, src=0)
        assert r.cpu().tolist() == [0.0, 1.0, 2.0, 3.0, 4.0, 5.0]
    r = torch.zeros(4, device=DEV)
    reqs = [dist.irecv(r, src=(rank - 1) % world), dist.isend(torch.full((4,), float(rank), device=DEV), dst=(rank + 1) % world)]
    for q in reqs:
        q.wait()
    assert r.cpu().tolist() == [float((rank - 1) % world)] * 4
    # unsupported reduce op and collectives outside the path
    try:
        dist.all_reduce(torch.ones(4, dtype=torch.int32, device=DEV), op=dist.ReduceOp.BAND)
        raise AssertionError("BAND accepted")
    except RuntimeError as e:
        assert "Cannot use ReduceOp.BAND" in str(e)
    dist.barrier()


def p2p_cases(pg, rank, world):
    """send / recv: ring exchange, several messages in flight each way, waits out of posting order,
    more messages than the sender has buffers, empty and odd sizes; byte for byte."""
    from helpers import bits, rank_buffer
    nxt, prv = (rank + 1) % world, (rank - 1) % world

    def payload(src, dst, i, count, dtype=torch.uint8):
        return rank_buffer(count, dtype, src * 64 + dst, seed=1000 + i)

    # ring: everybody sends to the next rank and receives from the previous one
    for i, count in enumerate((1, 0, 4097, (1 << 20) + 3)):
        got = torch.full((count,), 7, dtype=torch.uint8, device=DEV)
        w = pg.recv([got], prv, 0)
        pg.send([payload(rank, nxt, i, count).to(DEV)], nxt, 0).wait()
        w.wait()
        assert np.array_equal(bits(got), bits(payload(prv, rank, i, count))), ("ring", count)
    # two receives and two sends posted each way, then waited receive-first (neither side may block)
    sizes = (300001, 12)
    gots = [torch.zeros(c, dtype=torch.bfloat16, device=DEV) for c in sizes]
    works = [pg.recv([g], prv, 0) for g in gots]
    works += [pg.send([payload(rank, nxt, 10 + j, c, torch.bfloat16).to(DEV)], nxt, 0) for j, c in enumerate(sizes)]
    assert works[2].is_completed() and works[3].is_completed()  # the data has left the tensors
    works[1].wait()  # second receive first: the first one is completed on the way
    assert works[0].is_completed()
    for w in works:
        w.wait()
    for j, c in enumerate(sizes):
        assert np.array_equal(bits(gots[j]), bits(payload(prv, rank, 10 + j, c, torch.bfloat16))), ("batch", j)
    # ten messages to one destination: more than the sender has buffers, so it has to wait for the receiver
    if rank == 0:
        for i in range(10):
            pg.send([payload(0, 1, 20 + i, 1000 + i).to(DEV)], 1, 0).wait()
    elif rank == 1:
        for i in range(10):
            got = torch.zeros(1000 + i, dtype=torch.uint8, device=DEV)
            pg.recv([got], 0, 0).wait()
            assert np.array_equal(bits(got), bits(payload(0, 1, 20 + i, 1000 + i))), ("burst", i)
    # a growing message reuses and then replaces the buffers (the receiver must re-map them)
    for i, count in enumerate((100, 70000, 100, 300000)):
        got = torch.zeros(count, dtype=torch.uint8, device=DEV)
        w = pg.recv([got], nxt, 0)
        pg.send([payload(rank, prv, 40 + i, count).to(DEV)], prv, 0).wait()
        w.wait()
        assert np.array_equal(bits(got), bits(payload(nxt, rank, 40 + i, count))), ("grow", count)
    # a receive posted before a collective, waited for after it: the sender may need more buffers
    # than it has before it can join the collective, so the receiver has to take messages in
    # while it waits in the collective's barrier
    count = 300000
    if rank == 0:
        got = torch.zeros(count, dtype=torch.uint8, device=DEV)
        w = pg.recv([got], 1, 0)
    elif rank == 1:
        pg.send([payload(1, 0, 60, count).to(DEV)], 0, 0).wait()
    t = torch.ones(8, device=DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    assert t.cpu().tolist() == [float(world)] * 8
    if rank == 0:
        w.wait()
        assert np.array_equal(bits(got), bits(payload(1, 0, 60, count))), "receive across a collective"
    # three ranks: 0 posts a receive from 2 and then blocks on one from 1; 2 sends 0 a long tensor
    # before it sends 1 what 1 needs to send 0 its message - 0 must take 2's messages in while it
    # waits for 1
    if world >= 3:
        count = 200000
        if rank == 0:
            a = torch.zeros(count, dtype=torch.uint8, device=DEV)
            b = torch.zeros(16, dtype=torch.uint8, device=DEV)
            wa = pg.recv([a], 2, 0)
            pg.recv([b], 1, 0).wait()
            wa.wait()
            assert np.array_equal(bits(a), bits(payload(2, 0, 70, count))) and np.array_equal(bits(b), bits(payload(2, 1, 71, 16)))
        elif rank == 1:
            b = torch.zeros(16, dtype=torch.uint8, device=DEV)
            pg.recv([b], 2, 0).wait()
            pg.send([b], 0, 0).wait()
        elif rank == 2:
            pg.send([payload(2, 0, 70, count).to(DEV)], 0, 0).wait()
            pg.send([payload(2, 1, 71, 16).to(DEV)], 1, 0).wait()
    # polling: is_completed turns true once the sender has published, without a wait
    got = torch.zeros(5, dtype=torch.uint8, device=DEV)
    w = pg.recv([got], prv, 0)
    pg.send([payload(rank, nxt, 50, 5).to(DEV)], nxt, 0).wait()
    import time
    deadline = time.time() + 60.0
    while not w.is_completed() and time.time() < deadline:
        pass
    assert w.is_completed() and np.array_equal(bits(got), bits(payload(prv, rank, 50, 5)))
    pg.barrier().wait()


def list_window_cases(pg, rank, world):
    """List and rooted forms whose staging image exceeds the (shrunk) window: they fall back to
    windowed broadcasts, rooted reduces or point-to-point messages and must give the same results."""
    n = 3001  # 12 KB of fp32: three windows of 4 KiB
    val = lambda r, i=0: float(r * 3 + i + 1)
    # allgather (list)
    outs = [torch.zeros(n, device=DEV) for _ in range(world)]
    pg.allgather([outs], [torch.full((n,), val(rank), device=DEV)]).wait()
    torch.cuda.synchronize()
    for r in range(world):
        assert float(outs[r].min()) == val(r) == float(outs[r].max()), ("allgather", r)
    # reduce_scatter (list): slot d of every rank's list is summed into rank d's output
    ins = [torch.full((n,), val(rank, d), device=DEV) for d in range(world)]
    keep = [t.clone() for t in ins]
    out = torch.zeros(n, device=DEV)
    o = c10d.ReduceScatterOptions()
    o.reduceOp = c10d.ReduceOp.SUM
    pg.reduce_scatter([out], [ins], o).wait()
    torch.cuda.synchronize()
    want = sum(val(r, rank) for r in range(world))
    assert float(out.min()) == want == float(out.max()), "reduce_scatter"
    assert all(torch.equal(a, b) for a, b in zip(ins, keep)), "reduce_scatter must not touch its inputs"
    # all_to_all (list), uneven sizes: rank r sends rank d a tensor of 1000 + 97 r + 13 d floats
    size = lambda r, d: 1000 + 97 * r + 13 * d
    a_in = [torch.full((size(rank, d),), val(rank, d), device=DEV) for d in range(world)]
    a_out = [torch.zeros(size(r, rank), device=DEV) for r in range(world)]
    pg.alltoall(a_out, a_in).wait()
    torch.cuda.synchronize()
    for r in range(world):
        assert float(a_out[r].min()) == val(r, rank) == float(a_out[r].max()), ("alltoall", r)
    # gather and scatter, every rank root in turn
    for root in range(world):
        go = c10d.GatherOptions()
        go.rootRank = root
        got = [torch.zeros(n, device=DEV) for _ in range(world)]
        pg.gather([got] if rank == root else [], [torch.full((n,), val(rank, root), device=DEV)], go).wait()
        torch.cuda.synchronize()
        if rank == root:
            for r in range(world):
                assert float(got[r].min()) == val(r, root) == float(got[r].max()), ("gather", root, r)
        so = c10d.ScatterOptions()
        so.rootRank = root
        piece = torch.zeros(n, device=DEV)
        src = [[torch.full((n,), val(r, root) + 0.5, device=DEV) for r in range(world)]] if rank == root else []
        pg.scatter([piece], src, so).wait()
        torch.cuda.synchronize()
        assert float(piece.min()) == val(rank, root) + 0.5 == float(piece.max()), ("scatter", root)
    pg.barrier().wait()


def large_message_case(pg, rank, world):
    """A message larger than one staging window (1 GiB) is cut into windows."""
    count = (1 << 28) + 12345  # 1 GiB + a bit of fp32
    t = torch.arange(count, dtype=torch.float32, device=DEV) * 0 + float(rank + 1)
    t[-1] = 7.0 * (rank + 1)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    torch.cuda.synchronize()
    s = world * (world + 1) / 2.0
    assert float(t[0]) == s and float(t[count // 2]) == s and float(t[-2]) == s and float(t[-1]) == 7.0 * s
    assert float(t.min()) == s
    del t
    # uneven all_to_all_single with inputs beyond one staging window (1200 and 1300 MiB): rows of
    # 1 MiB tagged with (source rank, row), so every output row names where it came from
    S = [[300, 900], [1100, 200]]
    row = 1 << 20
    def tagged(r, nrows):
        tag = (torch.arange(nrows, device=DEV) * 7 + r * 97) % 251
        return tag.to(torch.uint8).view(-1, 1).expand(nrows, row).contiguous()
    inp = tagged(rank, sum(S[rank]))
    out = torch.zeros(S[0][rank] + S[1][rank], row, dtype=torch.uint8, device=DEV)
    pg.alltoall_base(out, inp, [S[0][rank], S[1][rank]], S[rank]).wait()
    torch.cuda.synchronize()
    pos = 0
    for r in range(2):
        first = sum(S[r][:rank])
        want = ((torch.arange(first, first + S[r][rank], device=DEV) * 7 + r * 97) % 251).to(torch.uint8)
        got = out[pos:pos + S[r][rank]]
        assert torch.equal(got[:, 0], want) and torch.equal(got[:, -1], want) and torch.equal(got[:, row // 2], want), r
        pos += S[r][rank]
    del inp, out
    # coalesced forms whose staging image would exceed one window fall back to one collective per tensor
    ts = [torch.full((160 << 20,), float(rank + 1 + i), device=DEV) for i in range(2)]  # 2 x 640 MiB
    o = c10d.AllreduceCoalescedOptions()
    o.reduceOp = c10d.ReduceOp.SUM
    pg.allreduce_coalesced(ts, o).wait()
    torch.cuda.synchronize()
    for i, t in enumerate(ts):
        want = sum(r + 1 + i for r in range(world))
        assert float(t[0]) == want and float(t[-1]) == want and float(t.min()) == want == float(t.max())
    del ts
    # point to point across the 1 GiB window: two chunks travel as two messages
    count = (1 << 30) + 5
    if rank == 0:
        big = torch.arange(count, dtype=torch.int64, device=DEV).to(torch.uint8)
        pg.send([big], 1, 0).wait()
    elif rank == 1:
        got = torch.zeros(count, dtype=torch.uint8, device=DEV)
        pg.recv([got], 0, 0).wait()
        want = torch.arange(count, dtype=torch.int64, device=DEV).to(torch.uint8)
        assert torch.equal(got, want)
    pg.barrier().wait()


def missing_rank_case(pg, rank, world):
    """Rank 1 never joins the second collective: the others must get an error, not hang.  (A gather
    to rank 0, 2 MiB per rank: a collective whose host threads meet first in every mode -- the staging
    buffers' handles are published per call -- so the call itself raises.)"""
    t = torch.ones(1 << 19, device=DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    if rank == 1:
        return
    try:
        opts = c10d.GatherOptions()
        opts.rootRank = 0
        pg.gather([[torch.empty(1 << 19, device=DEV) for _ in range(world)]] if rank == 0 else [], [t], opts).wait()
        raise AssertionError("collective with a missing rank returned")
    except RuntimeError as e:
        assert ("timed out waiting for rank 1" in str(e) or "reported a failure" in str(e)
                or "rank 1 left the group" in str(e)), str(e)


def zero_copy_cases(pg, rank, world):
    """Large single-tensor collectives between rank processes read the peers' tensors in place.
    Same bits as the oracle: tensors that are views at odd offsets of larger allocations, a tensor
    reused call after call (cached mappings), an allocation that is freed and handed out again at
    the same address with other contents (a stale mapping would read the old bytes), and a rank
    whose tensor cannot be shared (everybody stages instead)."""
    from helpers import TORCH_TO_CODE, bits, rank_buffer, to_carrier
    from oracle import oracle as O

    def bits_np(arr):
        return arr.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[arr.dtype.itemsize])

    def view_of(host, pad):
        """The tensor as a view `pad` elements into a larger device allocation."""
        big = torch.empty(host.numel() + 2 * pad + 64, dtype=host.dtype, device=DEV)
        v = big[pad:pad + host.numel()]
        v.copy_(host)
        return v

    def allreduce_check(dtype, count, seed, pad=0, keep=None):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(count, dtype, r, seed=seed) for r in range(world)]
        t = keep if keep is not None else view_of(host[rank], pad)
        if keep is not None:
            t.copy_(host[rank])
        pg.allreduce([t], c10d.AllreduceOptions()).wait()
        want = bits_np(O.reduce([to_carrier(h) for h in host], code, O.SUM))
        assert np.array_equal(bits(t), want), ("allreduce", dtype, count, seed, pad)
        return t

    # allreduce: odd counts and offsets, every element width
    for dtype, count, pad in ((torch.bfloat16, (3 << 20) + 7, 3), (torch.float32, (1 << 20) + 1, 1), (torch.int8, (5 << 20) + 13, 5),
                              (torch.float64, (1 << 19) + 3, 0), (torch.bfloat16, 1 << 19, 0)):
        allreduce_check(dtype, count, seed=61, pad=pad)
    # the same tensor again and again: the peers' mappings are cached
    t = None
    for i in range(6):
        t = allreduce_check(torch.bfloat16, 2 << 20, seed=70 + i, keep=t)
    # freed and allocated again: torch returns the segment to the runtime, the next allocation of
    # the same size usually lands on the same address, with new contents
    for i in range(3):
        x = allreduce_check(torch.float32, (3 << 20) + 11, seed=80 + i)
        del x
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    # reduce_scatter_tensor, all_gather_into_tensor, broadcast, uneven all_to_all_single
    for dtype, m, pad in ((torch.bfloat16, 300007, 1), (torch.float32, 262144, 0)):
        code = TORCH_TO_CODE[dtype]
        host = [rank_buffer(world * m, dtype, r, seed=91) for r in range(world)]
        out = torch.empty(m, dtype=dtype, device=DEV)
        pg._reduce_scatter_base(out, view_of(host[rank], pad)).wait()
        want = O.reduce_scatter([to_carrier(h) for h in host], code, O.SUM, shard_first=rank, shard_num=1)[0]
        assert np.array_equal(bits(out), bits_np(want)), ("reduce_scatter", dtype, m)
        # in place: the output is this rank's slice of its input, which no other rank reads
        x = view_of(host[rank], pad)
        pg._reduce_scatter_base(x[rank * m:(rank + 1) * m], x).wait()
        assert np.array_equal(bits(x[rank * m:(rank + 1) * m]), bits_np(want)), ("reduce_scatter in place", dtype, m)
        host = [rank_buffer(m * 4, dtype, r, seed=92) for r in range(world)]
        out = torch.empty(world * m * 4, dtype=dtype, device=DEV)
        pg._allgather_base(out, view_of(host[rank], pad)).wait()
        assert np.array_equal(bits(out), np.concatenate([bits(h) for h in host])), ("allgather", dtype, m)
        # the output as a view at an odd offset of a larger allocation, which the peers write into:
        # the bytes either side of it stay as they were
        big = torch.full((world * m * 4 + 2 * pad + 64,), 7, dtype=dtype, device=DEV)
        out = big[pad + 3:pad + 3 + world * m * 4]
        pg._allgather_base(out, view_of(host[rank], pad)).wait()
        assert np.array_equal(bits(out), np.concatenate([bits(h) for h in host])), ("allgather into a view", dtype, m)
        assert bool((big[:pad + 3] == 7).all()) and bool((big[pad + 3 + world * m * 4:] == 7).all()), ("allgather wrote outside its output", dtype)
        # in place, as FSDP calls it: the input is this rank's slice of the output
        full = torch.zeros(world * m * 4, dtype=dtype, device=DEV)
        full[rank * m * 4:(rank + 1) * m * 4].copy_(host[rank])
        pg._allgather_base(full, full[rank * m * 4:(rank + 1) * m * 4]).wait()
        assert np.array_equal(bits(full), np.concatenate([bits(h) for h in host])), ("allgather in place", dtype, m)
        # aliased, but not the in-place form: the output of reduce_scatter_tensor inside ANOTHER rank's
        # slice of the input (which that rank reads), the input of all_gather_into_tensor inside another
        # rank's slice of the output (which that rank writes).  Such calls must be staged, where the
        # copy-in comes first: the results are those of the calls on separate tensors.
        other = (rank + 1) % world
        host = [rank_buffer(world * m, dtype, r, seed=94) for r in range(world)]
        x = view_of(host[rank], pad)
        want = O.reduce_scatter([to_carrier(h) for h in host], code, O.SUM, shard_first=rank, shard_num=1)[0]
        pg._reduce_scatter_base(x[other * m:(other + 1) * m], x).wait()
        assert np.array_equal(bits(x[other * m:(other + 1) * m]), bits_np(want)), ("reduce_scatter into a foreign slice", dtype, m)
        host = [rank_buffer(m * 4, dtype, r, seed=95) for r in range(world)]
        full = torch.zeros(world * m * 4, dtype=dtype, device=DEV)
        full[other * m * 4:(other + 1) * m * 4].copy_(host[rank])
        pg._allgather_base(full, full[other * m * 4:(other + 1) * m * 4]).wait()
        assert np.array_equal(bits(full), np.concatenate([bits(h) for h in host])), ("allgather from a foreign slice", dtype, m)
        root = m % world
        src = rank_buffer(m * 4 + 3, dtype, root, seed=93)
        t = view_of(src if rank == root else torch.zeros_like(src), pad)
        opts = c10d.BroadcastOptions()
        opts.rootRank = root
        pg.broadcast([t], opts).wait()
        assert np.array_equal(bits(t), bits(src)), ("broadcast", dtype, m)
    rng = np.random.default_rng(4321)
    S = rng.integers(0, 3000, size=(world, world))
    S[world - 1, 0] = 0
    hidden = 256
    host = [rank_buffer(int(S[r].sum()) * hidden, torch.bfloat16, r, seed=6).view(-1, hidden) for r in range(world)]
    out = torch.zeros(int(S[:, rank].sum()), hidden, dtype=torch.bfloat16, device=DEV)
    pg.alltoall_base(out, host[rank].to(DEV), S[:, rank].tolist(), S[rank].tolist()).wait()
    want = O.alltoallv([to_carrier(h) for h in host], S, hidden * 2)[rank]
    assert np.array_equal(out.cpu().view(torch.uint8).numpy().reshape(-1), want), "alltoallv"
    # List forms.  A list that is consecutive views of one tensor is read in place; any other list
    # is packed.  flat_on(r) decides per rank which it is, so that "every rank flat", "no rank
    # flat" and "some ranks flat" (every rank must then stage) all run.
    def as_list(host_pieces, flat):
        if flat:
            whole = torch.cat([h.reshape(-1) for h in host_pieces]).to(DEV) if host_pieces else None
            out, at = [], 0
            for h in host_pieces:
                out.append(whole[at:at + h.numel()].view(h.shape))
                at += h.numel()
            return out
        return [h.to(DEV) for h in host_pieces]

    for name, flat_on in (("all flat", lambda r: True), ("none flat", lambda r: False), ("mixed", lambda r: r % 2 == 0)):
        for scale in (1, 64):  # a few KiB per piece, and pieces large enough to be shared
            # alltoall(list) with uneven pieces (one of them empty)
            S = np.random.default_rng(777 + scale).integers(1, 40, size=(world, world)) * 129 * scale
            S[0, world - 1] = 0
            host = [[rank_buffer(int(S[r, d]), torch.bfloat16, r * world + d, seed=7) for d in range(world)] for r in range(world)]
            ins = as_list(host[rank], flat_on(rank))
            outs = as_list([torch.zeros(int(S[r, rank]), dtype=torch.bfloat16) for r in range(world)], flat_on(rank + 1))
            pg.alltoall(outs, ins).wait()
            for r in range(world):
                assert np.array_equal(bits(outs[r]), bits(host[r][rank])), ("alltoall list", name, scale, r)
            assert all(np.array_equal(bits(ins[d]), bits(host[rank][d])) for d in range(world)), "alltoall list: inputs changed"
            # reduce_scatter(list): slot d of every rank's list is reduced into rank d's output
            m = 1031 * scale * 8
            host = [[rank_buffer(m, torch.float32, r * world + d, seed=8) for d in range(world)] for r in range(world)]
            ins = as_list(host[rank], flat_on(rank))
            out = torch.zeros(m, dtype=torch.float32, device=DEV)
            pg.reduce_scatter([out], [ins]).wait()
            want = bits_np(O.reduce([to_carrier(host[r][rank]) for r in range(world)], O.F32, O.SUM))
            assert np.array_equal(bits(out), want), ("reduce_scatter list", name, scale)
            # allgather(list): every rank contributes a tensor of its own size
            sizes = [(517 + 3 * r) * scale * 16 for r in range(world)]
            host = [rank_buffer(sizes[r], torch.bfloat16, r, seed=9) for r in range(world)]
            outs = as_list([torch.zeros(sizes[r], dtype=torch.bfloat16) for r in range(world)], flat_on(rank))
            pg.allgather([outs], [host[rank].to(DEV)]).wait()
            for r in range(world):
                assert np.array_equal(bits(outs[r]), bits(host[r])), ("allgather list", name, scale, r)
    # rank 1's tensor lives in an allocation too large to be shared between processes: every rank
    # stages, results are the same
    count = (2 << 20) + 5
    host = [rank_buffer(count, torch.bfloat16, r, seed=99) for r in range(world)]
    if rank == 1:
        big = torch.empty((2 << 30) // 2 + 4096, dtype=torch.bfloat16, device=DEV)
        t = big[4096:4096 + count]
        t.copy_(host[rank])
    else:
        t = host[rank].to(DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    want = bits_np(O.reduce([to_carrier(h) for h in host], O.BF16, O.SUM))
    assert np.array_equal(bits(t), want), "allreduce with an unshareable tensor on rank 1"
    pg.barrier().wait()


def baseline_config_cases(pg, rank, world):
    """The benchmark configurations at their full size through the drop-in API, 8 rank processes:
    C3 (allreduce of 64 MiB bf16 per rank), C4's shape at a quarter of its size (reduce_scatter_tensor of
    256 MiB bf16 per rank) and C5 (all_to_all_single of 4096 tokens x top-8 x 7168 bf16 per rank with
    the routing counts of a seeded top-8-of-256 gate).  Every rank regenerates all ranks' inputs
    on the device and checks its result bit for bit against an fp32 chain in ascending rank order
    (one rounding at the end), respectively against the rows it must have received."""
    def rank_input(r, count, seed):
        g = torch.Generator(device=DEV)
        g.manual_seed(seed * 1000 + r)
        return (torch.randn(count, generator=g, device=DEV, dtype=torch.float32) * 0.02).to(torch.bfloat16)

    def chain(inputs):
        acc = inputs[0].float()
        for x in inputs[1:]:
            acc += x.float()
        return acc.to(torch.bfloat16)

    # C3
    count = 4096 * 8192
    xs = [rank_input(r, count, 3) for r in range(world)]
    want = chain(xs)
    t = xs[rank].clone()
    for _ in range(2):  # the second call reduces fresh contents in the same tensor (same mappings)
        t.copy_(xs[rank])
        pg.allreduce([t], c10d.AllreduceOptions()).wait()
        assert torch.equal(t.view(torch.int16), want.view(torch.int16)), "C3 through the backend"
    del xs, want, t
    # C4 shape, 256 MiB per rank
    m = (128 << 20) // world
    xs = [rank_input(r, m * world, 4) for r in range(world)]
    want = chain([x[rank * m:(rank + 1) * m] for x in xs])
    out = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    pg._reduce_scatter_base(out, xs[rank]).wait()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16)), "C4 shape through the backend"
    assert torch.equal(xs[rank].view(torch.int16), rank_input(rank, m * world, 4).view(torch.int16)), "reduce_scatter changed its input"
    del xs, want, out
    # C5: rows tagged with (source rank, row index) in their first eight bytes
    tokens, hidden, topk, experts = 4096, 7168, 8, 256
    S = torch.zeros(world, world, dtype=torch.int64)
    for r in range(world):
        g = torch.Generator()
        g.manual_seed(5000 + r)
        picks = torch.topk(torch.randn(tokens, experts, generator=g), topk, dim=1).indices
        S[r] = torch.bincount(picks.reshape(-1) // (experts // world), minlength=world)
    rows = tokens * topk
    inp = torch.empty(rows, hidden, dtype=torch.bfloat16, device=DEV)
    tags = inp.view(torch.int16).view(rows, hidden)
    tags.copy_((torch.arange(rows, device=DEV).view(-1, 1) * 31 + torch.arange(hidden, device=DEV).view(1, -1) * 7 + rank * 1009) % 30011)
    out = torch.zeros(int(S[:, rank].sum()), hidden, dtype=torch.bfloat16, device=DEV)
    pg.alltoall_base(out, inp, S[:, rank].tolist(), S[rank].tolist()).wait()
    got = out.view(torch.int16).view(-1, hidden)
    pos = 0
    for r in range(world):
        n = int(S[r, rank])
        first = int(S[r, :rank].sum())
        want = ((torch.arange(first, first + n, device=DEV).view(-1, 1) * 31 + torch.arange(hidden, device=DEV).view(1, -1) * 7 + r * 1009) % 30011).to(torch.int16)
        assert torch.equal(got[pos:pos + n], want), ("C5 through the backend", r)
        pos += n
    pg.barrier().wait()


def heavy_predecessor_case(rank, world):
    """A late rank with register-heavy kernels of its own (GEMMs) queued in front of its collective,
    while all other ranks are already waiting on the device: the waiting kernels must leave room
    for the GEMMs to start, or the group would wait for a rank that cannot get there."""
    import time
    a = torch.randn(4096, 4096, dtype=torch.bfloat16, device=DEV)
    b = torch.randn(4096, 4096, dtype=torch.bfloat16, device=DEV)
    c = torch.mm(a, b)  # warm the GEMM up
    t = torch.full((8 << 20,), 1.0, dtype=torch.bfloat16, device=DEV)
    dist.all_reduce(t)
    torch.cuda.synchronize()
    for it in range(3):
        t.fill_(float(rank + it))
        dist.barrier()
        if rank == (it % world):
            time.sleep(0.003)  # the others have launched and wait on the device
            for _ in range(20):
                c = torch.mm(a, b)
        dist.all_reduce(t)
        torch.cuda.synchronize()
        want = float(sum(r + it for r in range(world)))
        assert float(t[0]) == want and float(t[-1]) == want, (it, float(t[0]), want)
    # the same with small and medium messages, whose single launch waits itself, limited to its
    # share of half of the compute units
    for it, elems in enumerate((1 << 17, 1 << 19, 8, 1 << 21)):
        small = torch.full((elems,), float(rank + it), dtype=torch.bfloat16, device=DEV)
        dist.barrier()
        if rank == ((it + 3) % world):
            time.sleep(0.003)
            for _ in range(20):
                c = torch.mm(a, b)
        dist.all_reduce(small)
        torch.cuda.synchronize()
        want = float(sum(r + it for r in range(world)))
        assert float(small[0]) == want and float(small[-1]) == want, (elems, float(small[0]), want)
    # the pulls and the shard reduction at 4 MiB per rank, a late rank each
    n = (1 << 21) // world * world
    src = torch.full((n,), float(rank), dtype=torch.bfloat16, device=DEV)
    for it, what in enumerate(("all_to_all_single", "reduce_scatter_tensor", "all_gather_into_tensor")):
        dist.barrier()
        if rank == ((it + 5) % world):
            time.sleep(0.003)
            for _ in range(20):
                c = torch.mm(a, b)
        if what == "all_to_all_single":
            got = torch.empty_like(src)
            dist.all_to_all_single(got, src)
            want = [float(r) for r in range(world)]
            have = got.view(world, -1)[:, 0].tolist()
        elif what == "reduce_scatter_tensor":
            got = torch.empty(n // world, dtype=torch.bfloat16, device=DEV)
            dist.reduce_scatter_tensor(got, src)
            want = [float(sum(range(world)))] * 2
            have = [float(got[0]), float(got[-1])]
        else:
            got = torch.empty(n * world, dtype=torch.bfloat16, device=DEV)
            dist.all_gather_into_tensor(got, src)
            want = [float(r) for r in range(world)]
            have = got.view(world, -1)[:, -1].tolist()
        torch.cuda.synchronize()
        assert have == want, (what, have, want)
    out = torch.empty(world * 1024, dtype=torch.float32, device=DEV)
    if rank == 1:
        for _ in range(20):
            c = torch.mm(a, b)
    dist.all_gather_into_tensor(out, torch.full((1024,), float(rank), device=DEV))
    torch.cuda.synchronize()
    assert out.view(world, 1024)[:, 0].tolist() == [float(r) for r in range(world)]
    del c


def missing_rank_device_case(pg, rank, world):
    """Device-side waits: rank 1 never joins the second collective.  The survivors' kernel gives up
    by itself at the (shortened) limit and names the late rank; their Work reports the failure
    instead of success, the group refuses further collectives, and (one-launch form) the tensor is
    left alone.  MCCL_TEST_ELEMS floats: 16, or 2^18 (1 MiB: the largest message of this form,
    four tiles per wavefront when the launch is limited to few compute units)."""
    elems = int(os.environ.get("MCCL_TEST_ELEMS", "16"))
    t = torch.ones(elems, device=DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    torch.cuda.synchronize()
    assert t[:16].cpu().tolist() == [float(world)] * 16
    if rank == 1:
        return
    blocking = os.environ.get("CCL_BLOCKING_WAIT") == "1"
    before = t.clone()
    w = pg.allreduce([t], c10d.AllreduceOptions())
    if blocking:
        try:
            w.wait()
            raise AssertionError("blocking wait on a collective with a missing rank returned")
        except RuntimeError as e:
            # (the one-launch allreduce counts its own launches on the device: this is the group's second)
            assert "timed out waiting for rank 1 on the device (one-launch allreduce #2 of this group" in str(e), str(e)
    else:
        w.wait()  # stream-ordered: returns at once, the failure shows when the device gets there
        torch.cuda.synchronize()
    assert w.is_completed()
    assert not w.is_success()
    assert torch.equal(t, before)  # the kernel skips the sum when its wait gives up
    try:
        pg.allreduce([t], c10d.AllreduceOptions())
        raise AssertionError("a failed group accepted another collective")
    except RuntimeError as e:
        assert "timed out waiting for rank 1 on the device (one-launch allreduce #2 of this group" in str(e), str(e)


def late_peer_case(pg, rank, world):
    """wait(timeout) in blocking mode: rank 1 joins 1.5 s late, the others wait with a 200 ms limit
    and get the reference's "Caught collective operation timeout"; the collective itself still
    completes once the late rank arrives, with the right result."""
    import datetime
    import time
    t = torch.ones(1 << 18, device=DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    if rank == 1:
        time.sleep(1.5)
    w = pg.allreduce([t], c10d.AllreduceOptions())
    if rank != 1:
        try:
            w.wait(datetime.timedelta(milliseconds=200))
            raise AssertionError("wait(timeout) did not time out")
        except RuntimeError as e:
            assert "Caught collective operation timeout" in str(e), str(e)
    w.wait(datetime.timedelta(seconds=20))
    assert w.is_completed() and w.is_success()
    assert float(t[0]) == float(world * world) and float(t[-1]) == float(world * world)
    # a receive honours its timeout too
    if rank == 0:
        r = pg.recv([torch.zeros(4, device=DEV)], 1, 0)
        t0 = time.time()
        try:
            r.wait(datetime.timedelta(milliseconds=300))
            raise AssertionError("recv wait(timeout) did not time out")
        except RuntimeError as e:
            assert "timed out waiting for a message" in str(e), str(e)
        assert time.time() - t0 < 5.0
    else:
        time.sleep(1.0)  # stay in the group while rank 0 waits: it must run into its own limit


def missing_sender_case(pg, rank, world):
    """Rank 0 posts a receive for a message rank 1 never sends: the wait must raise, not hang; a
    mismatched size raises on the receiver as well."""
    t = torch.ones(16, device=DEV)
    pg.allreduce([t], c10d.AllreduceOptions()).wait()
    if rank == 1:
        pg.send([torch.ones(8, device=DEV)], 0, 0).wait()
        return
    got = torch.zeros(4, device=DEV)
    try:
        pg.recv([got], 1, 0).wait()  # 16 bytes expected, 32 sent
        raise AssertionError("size mismatch accepted")
    except RuntimeError as e:
        assert "recv expects 16 bytes from rank 1 but the message holds 32" in str(e), str(e)
    w = pg.recv([torch.zeros(4, device=DEV)], 1, 0)
    assert not w.is_completed()
    try:
        w.wait()
        raise AssertionError("receive without a sender returned")
    except RuntimeError as e:
        assert ("timed out waiting for a message" in str(e) or "reported a failure" in str(e)
                or "left the group" in str(e)), str(e)


def env_switch_case(pg, rank, world):
    """CCL_SAME_STREAM / CCL_BLOCKING_WAIT (src/ProcessGroupCCL.hpp:96-102): results are the same,
    a blocking wait leaves the Work completed, a same-stream op is ordered on the caller's stream."""
    t = torch.full((1 << 20,), float(rank + 1), device=DEV)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        t2 = t * 2  # produced on a side stream; the collective must be ordered after it
        w = pg.allreduce([t2], c10d.AllreduceOptions())
        w.wait()
        if os.environ.get("CCL_BLOCKING_WAIT") == "1":
            assert w.is_completed()
            # a Work answers for its own collective, not for what the caller enqueues behind it
            w2 = pg.allreduce([t2.clone()], c10d.AllreduceOptions())
            w2.wait()
            a = torch.ones(4096, 4096, device=DEV)
            for _ in range(40):
                a = (a @ a) * 1e-4
            assert w2.is_completed() and w2.is_success()
            del a
        r = t2 + 1
    side.synchronize()
    assert float(r[0]) == world * (world + 1) + 1 and float(r[-1]) == world * (world + 1) + 1
    pg.barrier().wait()


def ddp_case(rank, world):
    """A real caller: DistributedDataParallel over backend "ccl" (the reference's demo/demo.py trains
    nn.Linear under DDP).  Gradients after backward must equal the average of the per-rank
    gradients computed without DDP."""
    import torch.nn as nn
    from torch.nn.parallel import DistributedDataParallel as DDP
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(64, 128), nn.ReLU(), nn.Linear(128, 10)).to(DEV)
    ref = nn.Sequential(nn.Linear(64, 128), nn.ReLU(), nn.Linear(128, 10)).to(DEV)
    ref.load_state_dict(model.state_dict())
    ddp = DDP(model, device_ids=[0])
    xs = [torch.randn(32, 64, generator=torch.Generator().manual_seed(100 + r)) for r in range(world)]
    ys = [torch.randn(32, 10, generator=torch.Generator().manual_seed(200 + r)) for r in range(world)]
    loss = ((ddp(xs[rank].to(DEV)) - ys[rank].to(DEV)) ** 2).mean()
    loss.backward()
    torch.cuda.synchronize()
    # reference: every rank's gradient on the same weights, averaged in fp32 in rank order
    grads = None
    for r in range(world):
        ref.zero_grad()
        ((ref(xs[r].to(DEV)) - ys[r].to(DEV)) ** 2).mean().backward()
        g = [p.grad.detach().clone() for p in ref.parameters()]
        grads = g if grads is None else [a + b for a, b in zip(grads, g)]
    for p, g in zip(ddp.module.parameters(), grads):
        assert torch.allclose(p.grad, g / world, rtol=1e-5, atol=1e-6), float((p.grad - g / world).abs().max())
    # FSDP-style step: all_gather_into_tensor of parameter shards, reduce_scatter_tensor of gradients
    flat = torch.cat([p.detach().reshape(-1) for p in ref.parameters()])
    pad = (-flat.numel()) % world
    flat = torch.cat([flat, flat.new_zeros(pad)])
    shard = flat.view(world, -1)[rank].contiguous()
    full = torch.empty_like(flat)
    dist.all_gather_into_tensor(full, shard)
    assert torch.equal(full, flat)
    gshard = torch.empty_like(shard)
    dist.reduce_scatter_tensor(gshard, flat * (rank + 1))
    want = flat.view(world, -1)[rank] * (world * (world + 1) / 2)
    assert torch.allclose(gshard, want, rtol=1e-6)


def reference_p2p_cases(rank, world):
    """The four cases of the reference's tests/test_c10d_p2p.py (world size 6), from the fixture:
    cubes of rank+1 elements per side filled with rank+1; a pair, a relay 1 -> 3 -> 5, every rank
    sending to all others in turn, and the same with tags."""
    with open(os.path.join(ROOT, "tests", "golden", "c10d_kats.json")) as f:
        P = json.load(f)["p2p"]
    assert world == P["world_size"]

    def cube(r, fill=None):
        side = P["cube"][r]["side"]
        return torch.full((side, side, side), P["cube"][r]["value"] if fill is None else fill)

    dist.all_reduce(torch.zeros(1, device=DEV))  # the reference's tests start with one, too
    mine = cube(rank).to(DEV)
    for hop in [P["pair"]] + P["relay"] + P["all_pairs"]:
        if rank == hop["src"]:
            dist.send(mine, hop["dst"])
        elif rank == hop["dst"]:
            out = cube(hop["src"], -1.0).to(DEV)
            dist.recv(out, hop["src"])
            assert torch.equal(out.cpu(), cube(hop["src"])), hop
    side = P["tagged"]["side"]
    tagged = torch.full((side, side, side), float(rank), device=DEV)
    for m in P["tagged"]["messages"]:
        if rank == m["src"]:
            dist.send(tagged, m["dst"], tag=m["tag"])
        elif rank == m["dst"]:
            out = torch.full((side, side, side), -1.0, device=DEV)
            dist.recv(out, m["src"], tag=m["tag"])
            assert bool(out.eq(m["value"]).all()), m
    dist.barrier()


def identity_replay_case(rank, world):
    """The reference's tests/test_allreduce.py in small: fp16 data of 0.1 is allreduced and divided
    by the (power-of-two) world size round after round, interleaved with elementwise kernels that
    consume it on the caller's stream.  x*W/W == x exactly, so data must keep its bits and the
    accumulator must equal a replay without any collective; a collective that ran before its
    input was ready, or let its consumer start early, breaks that.  Two sizes: one staged on the
    caller's stream (28 KiB), one on the communication stream (2 MiB)."""
    assert world & (world - 1) == 0
    for count, rounds in ((14336, 150), (1 << 20, 40)):
        data = (torch.ones(count, dtype=torch.float16) * 0.1).to(DEV)
        keep = data.clone()
        a = torch.zeros(8, count, dtype=torch.float16, device=DEV)
        want = torch.zeros(8, count, dtype=torch.float16, device=DEV)
        for _ in range(rounds):
            a[0] += data * 0.1
            for _ in range(4):
                a += 0.01
            dist.all_reduce(data)
            data /= world
        for _ in range(rounds):
            want[0] += keep * 0.1
            for _ in range(4):
                want += 0.01
        torch.cuda.synchronize()
        assert torch.equal(data.view(torch.int16), keep.view(torch.int16)), count
        assert torch.equal(a.view(torch.int16), want.view(torch.int16)), count
    dist.barrier()


def standing_offer_cases(pg, rank, world):
    """all_reduce above the one-launch size between rank processes: the ranks' host threads never
    wait for each other.  Where each rank's tensor is travels on the device; a rank whose allocation
    the peers have not mapped yet copies through its staging buffer meanwhile.  Every result is the
    oracle's, bit for bit."""
    import time
    from helpers import TORCH_TO_CODE, bits, rank_buffer, to_carrier
    from oracle import oracle as O

    def bits_np(arr):
        return arr.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[arr.dtype.itemsize])

    def check(t, host, what, op=O.SUM):
        want = bits_np(O.reduce([to_carrier(h) for h in host], TORCH_TO_CODE[t.dtype], op))
        assert np.array_equal(bits(t), want), what

    # the same tensor again and again: after the first calls nobody rendezvous, everybody reads in place
    count = (2 << 20) + 5
    t = torch.empty(count, dtype=torch.bfloat16, device=DEV)
    paths = []
    for i in range(12):
        host = [rank_buffer(count, torch.bfloat16, r, seed=500 + i) for r in range(world)]
        t.copy_(host[rank])
        if i == 4:
            torch.cuda.synchronize()
            before = pg._rendezvous_counts()
        pg.allreduce([t], c10d.AllreduceOptions()).wait()
        paths.append(pg._last_path())
        check(t, host, ("same tensor", i, paths[-1]))
    after = pg._rendezvous_counts()
    assert after[0] == before[0] and after[1] == before[1] + 8, (before, after)  # no rendezvous, eight that only enqueued
    assert all(p.startswith("standing offers") for p in paths), paths
    assert paths[-1] == "standing offers, peers read in place", paths  # (the first calls are staged until every peer has mapped the allocation)
    # a message larger than any before: the ranks meet once to enlarge their staging buffers, and since
    # they meet they map each other's new tensors there and then -- in place from the first call on
    count = (10 << 20) + 3  # 40 MiB of int32
    big = torch.empty(count, dtype=torch.int32, device=DEV)
    for i in range(2):
        host = [rank_buffer(count, torch.int32, r, seed=520 + i) for r in range(world)]
        big.copy_(host[rank])
        pg.allreduce([big], c10d.AllreduceOptions()).wait()
        assert pg._last_path() == "standing offers, peers read in place", (i, pg._last_path())
        check(big, host, ("larger than any before", i))
    del big
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    # a new allocation per call (each tensor fills a segment of its own), all alive at once, more of
    # them than the table of announced allocations holds: entries are reused, results stay right
    keep = []
    for i in range(40):
        n = (12 << 20) // 4 + i
        x = torch.full((n,), float(rank + 1 + i), device=DEV)
        keep.append(x)
        pg.allreduce([x], c10d.AllreduceOptions()).wait()
    for again in range(2):
        for i, x in enumerate(keep):
            if again:
                x.fill_(float(rank + 1 + i))
                pg.allreduce([x], c10d.AllreduceOptions()).wait()
            want = float(sum(r + 1 + i for r in range(world)))
            assert float(x.min()) == want == float(x.max()), ("many allocations", again, i, float(x.min()), want)
    del keep
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    # odd counts, offsets into an allocation, every element width, AVG and MAX
    for dtype, n, pad, op, oop in ((torch.float32, (1 << 20) + 1, 1, c10d.ReduceOp.SUM, O.SUM), (torch.int8, (5 << 20) + 13, 5, c10d.ReduceOp.MAX, O.MAX),
                                   (torch.float64, (1 << 19) + 3, 0, c10d.ReduceOp.SUM, O.SUM), (torch.bfloat16, (3 << 20) + 7, 3, c10d.ReduceOp.AVG, O.AVG),
                                   (torch.float16, (1 << 20) + 9, 2, c10d.ReduceOp.SUM, O.SUM)):
        host = [rank_buffer(n, dtype, r, seed=540) for r in range(world)]
        whole = torch.zeros(n + 2 * pad + 8, dtype=dtype, device=DEV)
        view = whole[pad:pad + n]
        for rep in range(3):  # staged at first, in place once the peers have mapped the allocation
            view.copy_(host[rank])
            opts = c10d.AllreduceOptions()
            opts.reduceOp = op
            pg.allreduce([view], opts).wait()
            check(view, host, ("view", dtype, n, rep, pg._last_path()), oop)
            assert bool((whole[:pad] == 0).all()) and bool((whole[pad + n:] == 0).all()), ("wrote outside the tensor", dtype)
    # rank 1's tensor lives in an allocation too large to be shared: that rank stages every time,
    # the others read and write its staging buffer, everybody else is read in place
    n = (2 << 20) + 5
    host = [rank_buffer(n, torch.bfloat16, r, seed=560) for r in range(world)]
    if rank == 1:
        huge = torch.empty((2 << 30) + 64, dtype=torch.uint8, device=DEV)
        x = huge[64:64 + 2 * n].view(torch.bfloat16)
    else:
        x = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    for rep in range(4):
        x.copy_(host[rank])
        pg.allreduce([x], c10d.AllreduceOptions()).wait()
        check(x, host, ("unshareable on rank 1", rep))
    assert pg._last_path() == ("standing offers, this rank staged" if rank == 1 else "standing offers, peers read in place"), pg._last_path()
    del x
    if rank == 1:
        del huge
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    # freed and allocated again between the calls (usually the same address, new contents)
    for i in range(4):
        host = [rank_buffer((3 << 20) + 11, torch.float32, r, seed=580 + i) for r in range(world)]
        y = host[rank].to(DEV)
        pg.allreduce([y], c10d.AllreduceOptions()).wait()
        check(y, host, ("freed and allocated again", i))
        del y
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    # reduce_scatter_tensor and all_gather_into_tensor the same way: no rendezvous in steady state, small
    # and large, in place and not, rank 1 staging for good (its tensors sit in an allocation too large
    # to share), and the forms whose tensors overlap outside the rank's own slice
    for dtype, m in ((torch.bfloat16, 300007), (torch.float32, 1 << 20), (torch.float32, 33)):
        code = TORCH_TO_CODE[dtype]
        es = torch.empty(0, dtype=dtype).element_size()
        if rank == 1:
            huge = torch.empty((2 << 30) + 64, dtype=torch.uint8, device=DEV)
            x = huge[64:64 + world * m * es].view(dtype)
            full = huge[(1 << 30):(1 << 30) + world * m * es].view(dtype)
        else:
            x = torch.empty(world * m, dtype=dtype, device=DEV)
            full = torch.empty(world * m, dtype=dtype, device=DEV)
        out = torch.empty(m, dtype=dtype, device=DEV)
        for rep in range(4):
            host = [rank_buffer(world * m, dtype, r, seed=600 + rep) for r in range(world)]
            want = bits_np(O.reduce_scatter([to_carrier(h) for h in host], code, O.SUM, shard_first=rank, shard_num=1)[0])
            x.copy_(host[rank])
            if rep == 2:
                before = pg._rendezvous_counts()
            pg._reduce_scatter_base(out, x).wait()
            assert np.array_equal(bits(out), want), ("reduce_scatter", dtype, m, rep, pg._last_path())
            x.copy_(host[rank])
            pg._reduce_scatter_base(x[rank * m:(rank + 1) * m], x).wait()  # in place
            assert np.array_equal(bits(x[rank * m:(rank + 1) * m]), want), ("reduce_scatter in place", dtype, m, rep)
            other = (rank + 1) % world
            x.copy_(host[rank])
            pg._reduce_scatter_base(x[other * m:(other + 1) * m], x).wait()  # output in a foreign slice: this rank stages
            assert np.array_equal(bits(x[other * m:(other + 1) * m]), want), ("reduce_scatter into a foreign slice", dtype, m, rep)
            assert pg._last_path() == "standing offers, this rank staged", pg._last_path()
            parts = [rank_buffer(m, dtype, r, seed=650 + rep) for r in range(world)]
            whole = np.concatenate([bits(h) for h in parts])
            full.zero_()
            pg._allgather_base(full, parts[rank].to(DEV)).wait()
            assert np.array_equal(bits(full), whole), ("allgather", dtype, m, rep, pg._last_path())
            full.zero_()
            full[rank * m:(rank + 1) * m].copy_(parts[rank])
            pg._allgather_base(full, full[rank * m:(rank + 1) * m]).wait()  # in place
            assert np.array_equal(bits(full), whole), ("allgather in place", dtype, m, rep)
            full.zero_()
            full[other * m:(other + 1) * m].copy_(parts[rank])
            pg._allgather_base(full, full[other * m:(other + 1) * m]).wait()  # input in a foreign slice: this rank stages
            assert np.array_equal(bits(full), whole), ("allgather from a foreign slice", dtype, m, rep)
        after = pg._rendezvous_counts()
        assert after[0] == before[0] and after[1] == before[1] + 12, (before, after)
        large = world * m * es >= (1 << 20)
        assert pg._last_path() == "standing offers, this rank staged"  # (the foreign-slice form was last)
        del x, full, out
        if rank == 1:
            del huge
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    # the coalesced forms pack their tensors into the staging buffer, which every peer has mapped since
    # it last grew: after the first call of a size nobody meets
    for rep in range(3):
        ts = [torch.full((5000 + 300 * i,), float(rank + 1 + i), device=DEV) for i in range(6)] + [torch.full((1 << 20,), float(rank + 1), device=DEV)]
        o = c10d.AllreduceCoalescedOptions()
        o.reduceOp = c10d.ReduceOp.SUM
        before = pg._rendezvous_counts()
        pg.allreduce_coalesced(ts, o).wait()
        mid = pg._rendezvous_counts()
        for i, t in enumerate(ts[:6]):
            want = float(sum(r + 1 + i for r in range(world)))
            assert float(t.min()) == want == float(t.max()), ("allreduce_coalesced", rep, i)
        assert float(ts[6].min()) == world * (world + 1) / 2 == float(ts[6].max())
        assert pg._last_path() == "staged, staging buffers mapped for good", pg._last_path()
        if rep:
            assert mid[0] == before[0], (rep, before, mid)
    # a rank that comes 50 ms late: the others' calls return at once (nobody's host thread waits
    # for anybody), their Works complete when the late rank's kernels have run
    z = torch.full((1 << 20,), float(rank + 1), device=DEV)  # 4 MiB
    pg.allreduce([z], c10d.AllreduceOptions()).wait()
    pg.allreduce([z], c10d.AllreduceOptions()).wait()  # (mapped by every peer now)
    torch.cuda.synchronize()
    pg.barrier().wait()
    z.fill_(float(rank + 1))
    torch.cuda.synchronize()
    if rank == 1:
        time.sleep(0.05)
    t0 = time.perf_counter()
    w = pg.allreduce([z], c10d.AllreduceOptions())
    call_ms = (time.perf_counter() - t0) * 1e3
    w.wait()
    torch.cuda.synchronize()
    total_ms = (time.perf_counter() - t0) * 1e3
    assert float(z[0]) == world * (world + 1) / 2 == float(z[-1])
    print("standing offers: rank %d of %d, all_reduce(4 MiB) with rank 1 50 ms late: call %.3f ms, call + synchronize %.3f ms" % (
        rank, world, call_ms, total_ms), flush=True)
    assert call_ms < 5.0, call_ms  # (measured: below 0.1 ms; the late rank itself included)
    if rank != 1:
        assert total_ms > 30.0, total_ms  # the result did wait for the late rank
    pg.barrier().wait()
    # the same for reduce_scatter_tensor and all_gather_into_tensor of 8 MiB per rank's buffer
    inp = torch.full((world << 18,), float(rank + 1), device=DEV)
    shard = torch.empty(1 << 18, device=DEV)
    gathered = torch.empty(world << 18, device=DEV)
    for _ in range(2):
        pg._reduce_scatter_base(shard, inp).wait()
        pg._allgather_base(gathered, shard).wait()
    torch.cuda.synchronize()
    pg.barrier().wait()
    if rank == 1:
        time.sleep(0.05)
    t0 = time.perf_counter()
    w1 = pg._reduce_scatter_base(shard, inp)
    w2 = pg._allgather_base(gathered, shard)
    call_ms = (time.perf_counter() - t0) * 1e3
    w1.wait()
    w2.wait()
    torch.cuda.synchronize()
    assert float(gathered.min()) == world * (world + 1) / 2 == float(gathered.max())
    print("standing offers: rank %d of %d, reduce_scatter_tensor + all_gather_into_tensor with rank 1 50 ms late: both calls %.3f ms" % (
        rank, world, call_ms), flush=True)
    assert call_ms < 5.0, call_ms
    pg.barrier().wait()


def standing_alltoall_cases(pg, rank, world):
    """all_to_all_single / all_to_all between rank processes without a rendezvous of the host threads: the
    ranks' pieces are offered on the device, pair by pair in place or through the outbox a rank keeps
    for that one peer.  Every result is the index map's (oracle), byte for byte."""
    import time
    from helpers import bits, rank_buffer, to_carrier
    from oracle import oracle as O

    def a2a(S, hidden, seed, dtype=torch.bfloat16, inp=None, out=None, overlapping=False):
        es = torch.empty(0, dtype=dtype).element_size()
        host = [rank_buffer(int(S[r].sum()) * hidden, dtype, r, seed=seed).view(int(S[r].sum()), hidden) for r in range(world)]
        if inp is None:
            inp = torch.empty(int(S[rank].sum()), hidden, dtype=dtype, device=DEV)
        if out is None:
            out = torch.empty(int(S[:, rank].sum()), hidden, dtype=dtype, device=DEV)
        if not overlapping:
            out.zero_()
        inp.copy_(host[rank])
        pg.alltoall_base(out, inp, S[:, rank].tolist(), S[rank].tolist()).wait()
        want = O.alltoallv([to_carrier(h) for h in host], S, hidden * es)[rank]
        assert np.array_equal(out.cpu().view(torch.uint8).numpy().reshape(-1), want), ("alltoallv", seed, pg._last_path())
        if not overlapping:
            assert np.array_equal(bits(inp.view(-1)), bits(host[rank].view(-1))), ("alltoallv changed its input", seed)
        return inp, out

    rng = np.random.default_rng(4321)
    hidden = 512
    # the same tensors again and again (1 KiB rows, up to 600 per piece): after the first calls every piece is
    # read in place and nobody waits for anybody
    S = rng.integers(0, 600, size=(world, world))
    S[0, world - 1] = 0
    S[world - 1, 0] = 0
    inp = out = None
    for i in range(8):
        if i == 3:
            torch.cuda.synchronize()
            before = pg._rendezvous_counts()
        inp, out = a2a(S, hidden, 700 + i, inp=inp, out=out)
    after = pg._rendezvous_counts()
    assert after[0] == before[0] and after[2] == before[2] and after[1] == before[1] + 5, (before, after)
    if int(S[rank].sum()) * hidden * 2 >= (1 << 20):
        sent = sum(1 for d in range(world) if d != rank and S[rank][d])
        assert pg._last_path() == "standing offers, %d pieces read in place, 0 through outboxes" % sent, pg._last_path()
    # new tensors per call, pieces that grow from call to call (each growth: the pair meets, nobody else)
    for i, top in enumerate((40, 700, 3000, 3000, 300, 9000)):
        S = rng.integers(0, top, size=(world, world))
        S[i % world, (i + 1) % world] = top  # (one pair grows for sure)
        a2a(S, hidden, 720 + i)
    # rows of odd widths and element sizes, empty pieces, a rank that sends nothing, one that gets nothing
    for i, (dtype, hid) in enumerate(((torch.uint8, 333), (torch.float64, 17), (torch.float32, 1), (torch.int16, 4099))):
        S = rng.integers(0, 400, size=(world, world))
        S[rng.integers(0, world)] = 0
        S[:, rng.integers(0, world)] = 0
        a2a(S, hid, 740 + i, dtype=dtype)
    # input and output in one tensor, overlapping: every piece is copied out of the way first
    S = np.full((world, world), 200)
    whole = torch.empty(world * 200 + 100, hidden, dtype=torch.bfloat16, device=DEV)
    for i in range(2):
        a2a(S, hidden, 760 + i, inp=whole[:world * 200], out=whole[100:100 + world * 200], overlapping=True)
        assert pg._last_path().endswith("0 pieces read in place, %d through outboxes" % (world - 1)), pg._last_path()
    # the list form: pieces in tensors of their own (small ones through outboxes, large ones in place once mapped)
    for i in range(3):
        sizes = [[(37 + 11 * r + 5 * d) * (1 if (r + d) % 3 else 9000) for d in range(world)] for r in range(world)]
        sizes[0][world - 1] = 0
        host = [[rank_buffer(sizes[r][d], torch.float32, r * world + d, seed=780 + i) for d in range(world)] for r in range(world)]
        ins = [h.to(DEV) for h in host[rank]]
        outs = [torch.zeros(sizes[r][rank], device=DEV) for r in range(world)]
        pg.alltoall(outs, ins).wait()
        for r in range(world):
            assert np.array_equal(bits(outs[r]), bits(host[r][rank])), ("alltoall list", i, r, pg._last_path())
    # all_gather into a list (every rank's size is known to all from the output list: sizes may differ) and
    # broadcast: the same piece for every reader, staged through the rank's staging buffer when it is
    # not offered in place
    for i in range(4):
        sizes = [((3 << 18) + 1000 * r + 7) * (1 if i % 2 else 3) for r in range(world)]  # floats: 3 and 9 MiB and a bit
        sizes[world - 1] = 0 if i == 2 else sizes[world - 1]
        host = [rank_buffer(sizes[r], torch.float32, r, seed=820 + i) for r in range(world)]
        mine_t = host[rank].to(DEV)
        outs = [torch.zeros(sizes[r], device=DEV) for r in range(world)]
        if i == 3:
            outs[rank] = mine_t  # gathered into the very tensor it comes from
        before = pg._rendezvous_counts()
        pg.allgather([outs], [mine_t]).wait()
        after = pg._rendezvous_counts()
        assert after[0] == before[0] or i == 0, (i, before, after)  # (the first one enlarges the staging buffers: the ranks meet)
        for r in range(world):
            assert np.array_equal(bits(outs[r]), bits(host[r])), ("allgather list", i, r, pg._last_path())
    # reduce_scatter from a list: slot d of every rank's list is reduced into rank d's output; slots of
    # different sizes, in tensors of their own or views of one, the output one of the slots
    from helpers import TORCH_TO_CODE
    for i, (dtype, base_n, op, oop) in enumerate(((torch.bfloat16, 300007, c10d.ReduceOp.SUM, O.SUM), (torch.float32, 1 << 19, c10d.ReduceOp.MAX, O.MAX),
                                                    (torch.float32, 33, c10d.ReduceOp.SUM, O.SUM), (torch.float16, (1 << 20) + 5, c10d.ReduceOp.AVG, O.AVG))):
        sizes = [base_n + 17 * d for d in range(world)]
        host = [[rank_buffer(sizes[d], dtype, r * world + d, seed=860 + i) for d in range(world)] for r in range(world)]
        for rep in range(3):
            if rep == 2:  # one storage, slots back to back
                flat = torch.cat([h.view(-1) for h in host[rank]]).to(DEV)
                ins = list(flat.split(sizes))
            else:
                ins = [h.to(DEV) for h in host[rank]]
            out = ins[rank] if rep == 1 else torch.zeros(sizes[rank], dtype=dtype, device=DEV)
            opts = c10d.ReduceScatterOptions()
            opts.reduceOp = op
            before = pg._rendezvous_counts()
            pg.reduce_scatter([out], [ins], opts).wait()
            after = pg._rendezvous_counts()
            assert after[0] == before[0], (i, rep, before, after)
            want = O.reduce([to_carrier(host[r][rank]) for r in range(world)], TORCH_TO_CODE[dtype], oop)
            want = want.view({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[want.dtype.itemsize])
            assert np.array_equal(bits(out), want), ("reduce_scatter list", dtype, i, rep, pg._last_path())
            for d in range(world):
                if d != rank or rep != 1:
                    assert np.array_equal(bits(ins[d]), bits(host[rank][d])), ("reduce_scatter list changed slot", d)
    small = [torch.zeros(100 + r, dtype=torch.int16, device=DEV) for r in range(world)]
    pg.allgather([small], [torch.full((100 + rank,), rank + 1, dtype=torch.int16, device=DEV)]).wait()
    for r in range(world):
        assert int(small[r].min()) == r + 1 == int(small[r].max()), ("allgather list, small", r)
    keep = torch.empty((5 << 20) + 3, dtype=torch.uint8, device=DEV)
    for i in range(6):
        root = i % world
        n = ((5 << 20) + 3) if i < 4 else 4099
        want = rank_buffer(n, torch.uint8, root, seed=840 + i)
        t = keep[:n] if i % 2 else torch.empty(n, dtype=torch.uint8, device=DEV)
        t.copy_(want if rank == root else torch.zeros(n, dtype=torch.uint8))
        opts = c10d.BroadcastOptions()
        opts.rootRank = root
        opts.rootTensor = 0
        before = pg._rendezvous_counts()
        pg.broadcast([t], opts).wait()
        after = pg._rendezvous_counts()
        assert after[0] == before[0], (i, before, after)
        assert np.array_equal(bits(t), bits(want)), ("broadcast", i, root, pg._last_path())
    # a rank that comes 50 ms late: the others' calls return at once
    S = rng.integers(100, 600, size=(world, world))
    inp = out = None
    for i in range(3):
        inp, out = a2a(S, hidden, 800 + i, inp=inp, out=out)
    torch.cuda.synchronize()
    pg.barrier().wait()
    if rank == 1:
        time.sleep(0.05)
    t0 = time.perf_counter()
    w = pg.alltoall_base(out, inp, S[:, rank].tolist(), S[rank].tolist())
    call_ms = (time.perf_counter() - t0) * 1e3
    w.wait()
    torch.cuda.synchronize()
    total_ms = (time.perf_counter() - t0) * 1e3
    print("standing offers: rank %d of %d, all_to_all_single with rank 1 50 ms late: call %.3f ms, call + synchronize %.3f ms" % (
        rank, world, call_ms, total_ms), flush=True)
    assert call_ms < 5.0, call_ms
    if rank != 1:
        assert total_ms > 30.0, total_ms
    pg.barrier().wait()


def standing_alltoall_big_case(pg, rank, world):
    """Pieces larger than any outbox (the limit shrunk by MCCL_PG_STANDING_MAX_BYTES) are read in place
    always: the receiver waits for the sender to enter the collective, and for nobody else."""
    from helpers import rank_buffer, to_carrier
    from oracle import oracle as O
    rng = np.random.default_rng(99)
    hidden = 1024
    for i in range(4):
        S = rng.integers(0, 200, size=(world, world))
        S[0, 1] = 3000 + i  # 3 MiB and more at one byte per element: above the 2 MiB limit of this run
        S[1, 0] = 0 if i % 2 else 2500
        host = [rank_buffer(int(S[r].sum()) * hidden, torch.uint8, r, seed=900 + i).view(-1, hidden) for r in range(world)]
        out = torch.zeros(int(S[:, rank].sum()), hidden, dtype=torch.uint8, device=DEV)
        before = pg._rendezvous_counts()
        pg.alltoall_base(out, host[rank].to(DEV), S[:, rank].tolist(), S[rank].tolist()).wait()
        after = pg._rendezvous_counts()
        assert after[0] == before[0], (before, after)
        want = O.alltoallv([to_carrier(h) for h in host], S, hidden)[rank]
        assert np.array_equal(out.cpu().numpy().reshape(-1), want), ("alltoallv with an oversized piece", i, pg._last_path())
    pg.barrier().wait()


def alltoall_mismatch_case(pg, rank, world):
    """Split sizes that do not match between two ranks (rank 1 expects less from rank 0 than rank 0
    sends): with the offers on the device nobody's host thread can notice, so the reader's kernel does --
    it leaves that piece alone, reports, and rank 1's next call raises with the reason."""
    rows, hidden = 64, 256
    S = np.full((world, world), rows)
    out_splits = S[:, rank].tolist()
    if rank == 1:
        out_splits[0] = rows - 8
    inp = torch.full((rows * world, hidden), float(rank + 1), device=DEV)
    out = torch.zeros(sum(out_splits), hidden, device=DEV)
    said = None
    try:
        pg.alltoall_base(out, inp, out_splits, S[rank].tolist()).wait()
    except RuntimeError as e:  # (the kernel may have run and reported by the time wait() looks)
        said = str(e)
    torch.cuda.synchronize()
    if rank == 1:
        assert float(out[:rows - 8].abs().max()) == 0.0  # the piece of the wrong length was not copied
        assert float(out[rows - 8:rows - 8 + rows].min()) == 2.0  # its own piece was
        if said is None:
            try:
                pg.allreduce([inp], c10d.AllreduceOptions()).wait()
                raise AssertionError("the call after a mismatch returned")
            except RuntimeError as e:
                said = str(e)
        assert "does not have the length this rank expects" in said and "rank 0" in said, said
    else:
        assert said is None, said
        for r in range(world):
            assert float(out[r * rows:(r + 1) * rows].min()) == float(r + 1) == float(out[r * rows:(r + 1) * rows].max()), r


def standing_mix_case(pg, rank, world):
    """A seeded mixture of the collectives that only enqueue -- all-to-alls with pieces of every size class
    (and beyond the largest, when the limit is shrunk), all_reduce, reduce_scatter / all_gather in both
    forms, broadcast -- on new and on reused tensors, with every rank late at random: the offers, the
    acknowledgements, the outboxes and their growth have to keep in step whatever the order in which
    the host threads get there.  Values are chosen so that every result has a closed form."""
    import random
    import time
    ops = random.Random(2024)       # the same sequence on every rank
    lag = random.Random(77 + rank)  # this rank's own delays
    kept = {}
    for it in range(250):
        op = ops.choice(("a2a", "a2a", "a2a", "allreduce", "rs", "ag", "ag_list", "rs_list", "bcast"))
        scale = ops.choice((1, 1, 40, 700, 3000))  # KiB: pieces from a few bytes to several MiB
        reuse = ops.random() < 0.5
        root = ops.randrange(world)
        S = [[ops.randrange(0, scale * 256 + 2) for _ in range(world)] for _ in range(world)]  # floats
        n = ops.randrange(1, scale * 256 + 2)
        if lag.random() < 0.3:
            time.sleep(lag.random() * 0.002)
        def tensor(key, numel, value):
            if reuse and key in kept and kept[key].numel() >= numel:
                t = kept[key][:numel]
            else:
                t = torch.empty(numel, device=DEV)
                kept[key] = t
            t.fill_(value)
            return t
        if op == "a2a":
            inp = tensor("a2a_in", sum(S[rank]), 0.0)
            pos = 0
            for d in range(world):
                inp[pos:pos + S[rank][d]] = float(rank * 16 + d + it)
                pos += S[rank][d]
            out = tensor("a2a_out", sum(S[r][rank] for r in range(world)), -1.0)
            pg.alltoall_base(out, inp, [S[r][rank] for r in range(world)], S[rank]).wait()
            pos = 0
            for r in range(world):
                piece = out[pos:pos + S[r][rank]]
                if S[r][rank]:
                    assert float(piece.min()) == float(r * 16 + rank + it) == float(piece.max()), ("a2a", it, r, pg._last_path())
                pos += S[r][rank]
        elif op == "allreduce":
            t = tensor("ar", n + (1 << 18), float(rank + it))
            pg.allreduce([t], c10d.AllreduceOptions()).wait()
            want = float(sum(r + it for r in range(world)))
            assert float(t.min()) == want == float(t.max()), ("allreduce", it, pg._last_path())
        elif op == "rs":
            t = tensor("rs_in", n * world, float(rank + 1))
            out = tensor("rs_out", n, 0.0)
            pg._reduce_scatter_base(out, t).wait()
            assert float(out.min()) == world * (world + 1) / 2 == float(out.max()), ("rs", it, pg._last_path())
        elif op == "ag":
            t = tensor("ag_in", n, float(rank + it))
            out = tensor("ag_out", n * world, -1.0)
            pg._allgather_base(out, t).wait()
            for r in range(world):
                assert float(out[r * n:(r + 1) * n].min()) == float(r + it) == float(out[r * n:(r + 1) * n].max()), ("ag", it, r)
        elif op == "ag_list":
            sizes = [S[0][r] + 1 for r in range(world)]
            t = tensor("agl_in", sizes[rank], float(rank + it))
            outs = [torch.full((sizes[r],), -1.0, device=DEV) for r in range(world)]
            pg.allgather([outs], [t]).wait()
            for r in range(world):
                assert float(outs[r].min()) == float(r + it) == float(outs[r].max()), ("ag_list", it, r, pg._last_path())
        elif op == "rs_list":
            sizes = [S[0][d] + 1 for d in range(world)]
            ins = [torch.full((sizes[d],), float(rank + d), device=DEV) for d in range(world)]
            out = torch.zeros(sizes[rank], device=DEV)
            pg.reduce_scatter([out], [ins], c10d.ReduceScatterOptions()).wait()
            want = float(sum(r + rank for r in range(world)))
            assert float(out.min()) == want == float(out.max()), ("rs_list", it, pg._last_path())
        else:
            t = tensor("bc", n, float(it) if rank == root else -1.0)
            o = c10d.BroadcastOptions()
            o.rootRank = root
            o.rootTensor = 0
            pg.broadcast([t], o).wait()
            assert float(t.min()) == float(it) == float(t.max()), ("bcast", it, root, pg._last_path())
    torch.cuda.synchronize()
    pg.barrier().wait()


def graph_capture_case(rank, world):
    """A decode loop from a HIP graph: every rank records K dist.all_reduce of the 256 KiB bf16
    message with a small kernel of the caller's between them, then replays the graph with fresh
    inputs, with eager collectives and synchronisations between the replays.  Every result of
    every replay is compared bit for bit with the oracle's.  What cannot be recorded is refused
    with a message, and the capture survives the refusal."""
    from helpers import assert_bits_equal, bits, oracle_reduce_bits, rank_buffer
    from oracle import oracle as O
    K, count, replays, windows = 32, 131072, 50, 8
    pool = [rank_buffer(count + 64 * windows, torch.bfloat16, r, seed=7000) for r in range(world)]
    want = torch.stack([torch.from_numpy(oracle_reduce_bits([pool[r][64 * w:64 * w + count] for r in range(world)], O.SUM).view(np.int16).copy())
                        for w in range(windows)]).to(DEV)                       # (windows, count) bit patterns
    mine = torch.stack([pool[rank][64 * w:64 * w + count] for w in range(windows)]).to(DEV)
    warm = torch.ones(1, device=DEV)
    dist.all_reduce(warm)  # the group's buffers are allocated and exchanged at its first collective
    assert float(warm[0]) == world
    X = torch.zeros(K, count, dtype=torch.bfloat16, device=DEV)
    ticks = torch.zeros(8, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # one pass outside the capture, as torch asks for
        for k in range(K):
            dist.all_reduce(X[k])
            ticks.add_(1.0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    big = torch.ones(1 << 20, device=DEV)  # 4 MiB: needs the host rendezvous
    with torch.cuda.graph(graph, stream=side):  # (every further stream would be another hardware queue of this process)
        for k in range(K):
            w = dist.all_reduce(X[k], async_op=True)
            w.wait()
            assert w.is_completed()
            ticks.add_(1.0)
        if rank == 0:  # (no other rank enters this collective: the refusal comes before anything is exchanged)
            for refused in (lambda: dist.all_reduce(big), lambda: dist.all_gather_into_tensor(torch.empty(world * 4, device=DEV), torch.ones(4, device=DEV))):
                try:
                    refused()
                    raise AssertionError("recorded a collective that cannot be replayed")
                except RuntimeError as e:
                    assert "cannot be recorded into a HIP graph" in str(e), str(e)
    ticks.zero_()
    wrong = torch.zeros((), dtype=torch.int64, device=DEV)
    eager = []
    gen = torch.Generator().manual_seed(7100)  # the same on every rank
    for p in range(replays):
        which = torch.randint(0, windows, (K,), generator=gen).to(DEV)
        X.copy_(mine[which])
        graph.replay()
        wrong += (X.view(torch.int16) != want[which]).sum()
        if p % 10 == 9:  # eager work of this backend and a synchronisation between two replays
            e_in = [rank_buffer(5000 + p, torch.float32, r, seed=7200 + p) for r in range(world)]
            e = e_in[rank].to(DEV)
            dist.all_reduce(e)
            eager.append((e, oracle_reduce_bits(e_in, O.SUM), p))
            big2 = torch.full((1 << 20,), float(rank + 1), device=DEV)
            dist.all_reduce(big2)
            torch.cuda.synchronize()
            assert float(big2[0]) == world * (world + 1) / 2 == float(big2[-1])
    torch.cuda.synchronize()
    assert int(wrong) == 0, int(wrong)
    assert ticks.cpu().tolist() == [float(K * replays)] * 8
    for e, w, p in eager:
        assert_bits_equal(bits(e), w, ("eager between replays", p))
    dist.barrier()


def graph_late_rank_case(rank, world):
    """A rank that does not replay its graph: the bounded waits of the recorded launches on the other
    ranks run into their (shortened) limit, every kernel ends by itself, and the group reports the
    late rank at its next call."""
    warm = torch.ones(1, device=DEV)
    dist.all_reduce(warm)
    X = torch.ones(2, 131072, dtype=torch.bfloat16, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for k in range(2):
            dist.all_reduce(X[k])
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for k in range(2):
            dist.all_reduce(X[k])
    X.fill_(1.0)
    graph.replay()
    torch.cuda.synchronize()
    assert float(X[0, 0]) == world == float(X[1, -1])
    if rank == 1:
        import time
        time.sleep(6.0)  # stays in the group, replays nothing
        return
    X.fill_(1.0)
    graph.replay()
    torch.cuda.synchronize()  # both launches have given up by now
    assert float(X[0, 0]) == 1.0 == float(X[1, -1])  # left alone
    try:
        dist.all_reduce(warm)
        raise AssertionError("a failed group accepted another collective")
    except RuntimeError as e:
        assert "timed out waiting for rank 1 on the device (one-launch allreduce #" in str(e), str(e)


def coalesced_window_cases(rank, world):
    """Coalesced forms on the default group whose staging image exceeds the (shrunk) window: they
    fall back to one windowed collective per tensor and must give the same results."""
    pg = c10d._get_default_group()
    n = 50_000  # 200 KB of fp32 per tensor: several 64 KiB windows each
    ts = [torch.full((n + i,), float(rank + 1 + i), device=DEV) for i in range(3)]
    o = c10d.AllreduceCoalescedOptions()
    o.reduceOp = c10d.ReduceOp.SUM
    pg.allreduce_coalesced(ts, o).wait()
    torch.cuda.synchronize()
    for i, t in enumerate(ts):
        want = float(sum(r + 1 + i for r in range(world)))
        assert float(t.min()) == want == float(t.max()), ("allreduce_coalesced", i)
    ins = [torch.full((world * (n + i),), float(rank + 1), device=DEV) for i in range(2)]
    outs = [torch.empty(n + i, device=DEV) for i in range(2)]
    pg.reduce_scatter_tensor_coalesced(outs, ins, c10d.ReduceScatterOptions()).wait()
    torch.cuda.synchronize()
    for t in outs:
        assert float(t.min()) == world * (world + 1) / 2.0 == float(t.max())
    gin = [torch.full((n + i,), float(rank * 10 + i), device=DEV) for i in range(2)]
    gout = [torch.empty(world * (n + i), device=DEV) for i in range(2)]
    pg.allgather_into_tensor_coalesced(gout, gin).wait()
    torch.cuda.synchronize()
    for i, t in enumerate(gout):
        got = t.view(world, n + i)
        for r in range(world):
            assert float(got[r].min()) == float(r * 10 + i) == float(got[r].max())
    dist.barrier()


def subgroup_case(rank, world):
    """Subgroups as the reference's tests/ds_subgroup_allreduce.py builds them: a one-rank group, then
    strided groups of `sub` ranks; plus a rooted op and a send / recv addressed by global rank inside
    a subgroup."""
    sub = 2
    warm = torch.ones(1, dtype=torch.bfloat16, device=DEV)
    dist.all_reduce(warm)
    assert float(warm[0]) == world
    x = torch.ones(2048, dtype=torch.bfloat16, device=DEV)
    g1 = dist.new_group([0])
    if rank == 0:
        dist.all_reduce(x, group=g1)
        assert torch.equal(x.cpu(), torch.ones(2048, dtype=torch.bfloat16))
    members = [[i + (world // sub) * j for j in range(sub)] for i in range(world // sub)]
    groups = [dist.new_group(m) for m in members]
    for m, g in zip(members, groups):
        if rank in m:
            dist.all_reduce(x, group=g)
            assert torch.equal(x.cpu(), torch.full((2048,), float(sub), dtype=torch.bfloat16))
            t = torch.full((5,), float(rank), device=DEV)
            dist.broadcast(t, src=m[-1], group=g)
            assert t.cpu().tolist() == [float(m[-1])] * 5
            got = torch.zeros(3, device=DEV)
            peer = m[1 - m.index(rank)]
            reqs = [dist.irecv(got, src=peer, group=g), dist.isend(torch.full((3,), float(rank), device=DEV), dst=peer, group=g)]
            for q in reqs:
                q.wait()
            assert got.cpu().tolist() == [float(peer)] * 3
    dist.barrier()


def run_rank(rank, world, store_path, mode):
    # the expected values are computed on the host by every rank: share the cores instead of
    # letting every rank process start a thread per core
    torch.set_num_threads(max(1, (os.cpu_count() or 16) // world))
    torch.cuda.set_device(0)
    import torch_ccl_amd  # noqa: F401  registers the backend
    if mode == "dist":
        store = dist.FileStore(store_path, world)
        dist.init_process_group("ccl", store=store, rank=rank, world_size=world)
        try:
            dist_api_cases(rank, world)
        finally:
            dist.destroy_process_group()
        return
    if mode in ("subgroup", "replay", "reference_p2p", "coalesced_windows", "heavy_predecessor", "graph", "graph_late"):
        store = dist.FileStore(store_path, world)
        dist.init_process_group("ccl", store=store, rank=rank, world_size=world)
        try:
            {"subgroup": subgroup_case, "replay": identity_replay_case, "reference_p2p": reference_p2p_cases,
             "coalesced_windows": coalesced_window_cases, "heavy_predecessor": heavy_predecessor_case,
             "graph": graph_capture_case, "graph_late": graph_late_rank_case}[mode](rank, world)
        finally:
            dist.destroy_process_group()
        return
    if mode == "ddp":
        store = dist.FileStore(store_path, world)
        dist.init_process_group("ccl", store=store, rank=rank, world_size=world)
        try:
            ddp_case(rank, world)
        finally:
            dist.destroy_process_group()
        return
    store = dist.FileStore(store_path, world)
    pg = dist.ProcessGroupCCL(store, rank, world)
    assert pg.name() == "ccl" and pg.rank() == rank and pg.size() == world
    if mode == "reference":
        reference_cases(pg, rank, world)
    elif mode == "oracle":
        oracle_cases(pg, rank, world)
    elif mode == "p2p":
        p2p_cases(pg, rank, world)
    elif mode == "list_windows":
        list_window_cases(pg, rank, world)
    elif mode == "large":
        large_message_case(pg, rank, world)
    elif mode == "env":
        env_switch_case(pg, rank, world)
    elif mode == "missing":
        missing_rank_case(pg, rank, world)
    elif mode == "missing_sender":
        missing_sender_case(pg, rank, world)
    elif mode == "zero_copy":
        zero_copy_cases(pg, rank, world)
    elif mode == "baseline_configs":
        baseline_config_cases(pg, rank, world)
    elif mode == "missing_device":
        missing_rank_device_case(pg, rank, world)
    elif mode == "late_peer":
        late_peer_case(pg, rank, world)
    elif mode == "standing":
        standing_offer_cases(pg, rank, world)
    elif mode == "standing_alltoall":
        standing_alltoall_cases(pg, rank, world)
    elif mode == "standing_mix":
        standing_mix_case(pg, rank, world)
    elif mode == "alltoall_mismatch":
        alltoall_mismatch_case(pg, rank, world)
    elif mode == "standing_big":
        standing_alltoall_big_case(pg, rank, world)
    else:
        raise ValueError(mode)
    torch.cuda.synchronize()
    del pg
