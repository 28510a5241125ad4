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
    ops = {"SUM": (capi.SUM, O.SUM), "PROD": (capi.PROD, O.PROD), "MIN": (capi.MIN, O.MIN), "MAX": (capi.MAX, O.MAX)}
    cases = []
    for dtype in ALL_DTYPES:
        es = torch.empty(0, dtype=dtype).element_size()
        for count in (1, 7, 16 // es, 16 // es + 1, 1024 // es, 1024 // es + 3, 5 * 1024 // es - 1, 40_000):
            for name in ops:
                cases.append((dtype, count, name))
    cases.append((torch.bfloat16, 131072, "SUM"))       # the 256 KiB decode message
    cases.append((torch.float32, FUSED_MAX_BYTES // 4, "SUM"))
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
        capi.check(L.mccl_allreduce_fused(x.data_ptr(), out.data_ptr(), count, TORCH_TO_CODE[dtype], ops[name][0],
                                          tables[slot][0], tables[slot][1], world, rank, epoch, 5_000_000,
                                          st.data_ptr(), stream))
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
                                          st.data_ptr(), stream))
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
            st.data_ptr(), stream))
        torch.cuda.synchronize()
        assert st.tolist() == [2, 9], st.tolist()
        assert out.cpu().tolist() == [-7.0] * 256
    barrier.wait(timeout=120)


def run_rank(rank, world, queues, barrier, mode):
    torch.cuda.set_device(0)
    {"barrier": barrier_case, "fused": fused_case, "timeout": timeout_case}[mode](rank, world, queues, barrier)
    torch.cuda.synchronize()
