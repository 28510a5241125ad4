#!/usr/bin/env python3
"""Headline benchmark: 8-rank bf16 allreduce local-reduce on one MI355X.

A "step" is one pass of the hot path over one batch: one N-buffer reduction of the
headline workload (8 rank buffers of bf16 [4096 x 8192], 64 MiB each, already resident
in HBM, reduced with fp32 accumulation into one bf16 output).  The line printed at the end
carries the whole-job throughput in algorithmic GB/s ((N+1) * S bytes per step), the HBM
roofline fraction of the kernel measured with HIP events on the launch stream, the p50/p99
latency of the 256 KiB decode-sized allreduce, and a CPU baseline (the oracle port, OpenMP)
timed on this host's cores on the same workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extras all|none|c1,c2,c4,c5,variants]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "torch-ccl_amd"))
sys.path.insert(0, os.path.join(ROOT, "bench"))

PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, published peak
SEED = 1234
# HBM bytes of one launch of the headline kernel come from rocprofv3 FETCH_SIZE + WRITE_SIZE runs of
# this script, each counter scaled by its reading for a 512 MiB copy of known size; the summary of
# those runs is this file, and the figure is read from its "Calibrated traffic" line.
C3_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "reduce_bf16_8rank_64MiB_stream.md")


def profiled_traffic_bytes(path=C3_TRAFFIC_PROFILE):
    """Bytes per launch from the committed counter summary (None when the file or the line is
    missing, so that a stale or absent profile shows as null instead of a made-up number)."""
    import re
    try:
        with open(path) as f:
            for line in f:
                m = re.search(r"Calibrated traffic of one reduce launch:.*?=\s*([0-9][0-9 ,_]*)\s*B\b", line)
                if m:
                    return int(re.sub(r"[ ,_]", "", m.group(1)))
    except OSError:
        pass
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def rank_generator(torch, seed, rank, device="cpu"):
    return torch.Generator(device=device).manual_seed(seed * 1_000_003 + rank)


def make_rank_buffers(torch, n, count, dtype, std, dev, on_device=False):
    """One buffer per rank: fp32 N(0, std) from the (seed, rank) generator, rounded to dtype."""
    bufs = []
    for r in range(n):
        if on_device:
            g = rank_generator(torch, SEED, r, dev)
            x = torch.empty(count, dtype=dtype, device=dev)
            step = 1 << 26
            for lo in range(0, count, step):
                hi = min(count, lo + step)
                x[lo:hi] = (torch.randn(hi - lo, generator=g, dtype=torch.float32, device=dev) * std).to(dtype)
            bufs.append(x)
        else:
            g = rank_generator(torch, SEED, r)
            bufs.append((torch.randn(count, generator=g, dtype=torch.float32) * std).to(dtype).to(dev))
    return bufs


def percentile(sorted_vals, q):
    i = min(len(sorted_vals) - 1, max(0, int(round(q * (len(sorted_vals) - 1)))))
    return sorted_vals[i]


def cpu_baseline(torch, host_inputs, n, count):
    """The oracle port (plain C, OpenMP) on this host: same workload, bounded to about 12 s."""
    import numpy as np
    from oracle import oracle as O
    threads = min(16, O.max_threads(), len(os.sched_getaffinity(0)))
    O.set_threads(threads)
    ins = [t.view(torch.int16).numpy().view(np.uint16) for t in host_inputs]
    t0 = time.perf_counter()
    O.reduce(ins, O.BF16, O.SUM)  # warm-up pass, also gives a cost estimate
    one = time.perf_counter() - t0
    passes = max(3, min(1000, int(12.0 / max(one, 1e-3))))  # about 12 s of CPU work
    t0 = time.perf_counter()
    for _ in range(passes):
        out = O.reduce(ins, O.BF16, O.SUM)
    dt = (time.perf_counter() - t0) / passes
    O.set_threads(1)
    gbs = (n + 1) * count * 2 / dt / 1e9
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d full-size passes of the headline workload (8 x 64 MiB bf16 -> 64 MiB) through "
                      "oracle/mccl_oracle.c with %d OpenMP threads; %.1f ms per pass" % (passes, threads, dt * 1e3),
            "ms_per_step": round(dt * 1e3, 3)}, out


def c5_split_matrix(torch, world, tokens=4096, topk=8, experts=256):
    """S[src][dst]: rows rank src sends to rank dst when each of its tokens goes to its top-k experts
    (router logits N(0,1) per (seed, rank)) and rank d holds experts [d * experts/world, ...)."""
    S = torch.zeros(world, world, dtype=torch.int64)
    for r in range(world):
        g = rank_generator(torch, SEED, r)
        chosen = torch.topk(torch.randn(tokens, experts, generator=g), topk, dim=1).indices
        S[r] = torch.bincount(chosen.reshape(-1) // (experts // world), minlength=world)
    return S


def _gloo_rank(rank, world, store_path, backend, cases, out_path, keep_path):
    """One host process of the N-process CPU baseline: same op, same (seed, rank) data, CPU tensors.
    A case that this backend cannot run is reported as such, not dropped."""
    os.dup2(2, 1)  # keep the parent's stdout clean for the one JSON line (gloo prints connection notes)
    import torch
    import torch.distributed as dist
    torch.set_num_threads(max(1, len(os.sched_getaffinity(0)) // world))
    store = dist.FileStore(store_path, world)
    dist.init_process_group(backend, store=store, rank=rank, world_size=world)
    res = {}
    for case in cases:
        name, op, count, dtype_name, warm, iters = case["name"], case["op"], case["count"], case["dtype"], case["warm"], case["iters"]
        dtype = getattr(torch, dtype_name)
        try:
            g = rank_generator(torch, SEED, rank)
            if case.get("dist") == "uniform":
                x = (torch.rand(count, generator=g, dtype=torch.float32) * 2 - 1).to(dtype)
            else:  # in pieces: the fp32 samples of a 1 GiB bf16 gradient would take 2 GiB per process
                x = torch.empty(count, dtype=dtype)
                for o in range(0, count, 1 << 26):
                    n = min(1 << 26, count - o)
                    x[o:o + n] = (torch.randn(n, generator=g, dtype=torch.float32) * case["std"]).to(dtype)
            if op == "all_reduce":
                t = x.clone()

                def prepare():
                    t.copy_(x)

                def run():
                    dist.all_reduce(t)
            elif op == "reduce_scatter_tensor":
                t = torch.empty(count // world, dtype=dtype)
                prepare = lambda: None  # noqa: E731

                def run():
                    dist.reduce_scatter_tensor(t, x)
            elif op == "all_to_all_single":
                S = c5_split_matrix(torch, world)
                hidden = case["hidden"]
                x = x.view(-1, hidden)
                t = torch.empty(int(S[:, rank].sum()), hidden, dtype=dtype)
                prepare = lambda: None  # noqa: E731

                def run():
                    dist.all_to_all_single(t, x, S[:, rank].tolist(), S[rank].tolist())
            else:
                raise ValueError(op)
            for _ in range(warm):
                prepare()
                run()
            ts = []
            for _ in range(iters):
                prepare()
                dist.barrier()
                t0 = time.perf_counter()
                run()
                ts.append(time.perf_counter() - t0)
            ts.sort()
            res[name] = {"p50_us": ts[len(ts) // 2] * 1e6, "p99_us": percentile(ts, 0.99) * 1e6, "iters": iters}
            if case.get("keep") and rank == 0:
                torch.save(t, keep_path)
            del x, t
        except Exception as e:  # e.g. an op this backend does not implement for CPU tensors
            res[name] = {"error": "%s on the %s backend: %s" % (op, backend, repr(e)[:200])}
    if rank == 0:
        with open(out_path, "w") as f:
            json.dump(res, f)
    dist.destroy_process_group()


def _backend_rank(rank, world, store_path, cases, out_path, large=True):
    """One rank process of the drop-in path: dist.all_reduce through backend "ccl" on cuda:0."""
    os.dup2(2, 1)
    sys.path.insert(0, os.path.join(ROOT, "torch-ccl_amd"))
    import torch
    import torch.distributed as dist
    import torch_ccl_amd  # noqa: F401
    torch.cuda.set_device(0)
    dist.init_process_group("ccl", store=dist.FileStore(store_path, world), rank=rank, world_size=world)
    res = {}
    for name, count, warm, iters in cases:
        g = rank_generator(torch, SEED, rank)
        x = (torch.randn(count, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to("cuda:0")
        t = x.clone()
        dist.all_reduce(t)
        # bit for bit against an fp32 chain over all ranks' inputs in ascending rank order
        acc = None
        for r in range(world):
            gr = rank_generator(torch, SEED, r)
            xr = (torch.randn(count, generator=gr, dtype=torch.float32) * 0.02).to(torch.bfloat16).to("cuda:0").float()
            acc = xr if acc is None else acc.add_(xr)
        exact = bool(torch.equal(t.view(torch.int16), acc.to(torch.bfloat16).view(torch.int16)))
        del acc, xr
        for _ in range(warm):
            dist.all_reduce(t)
        torch.cuda.synchronize()
        ts = []
        for _ in range(iters):
            t.copy_(x)
            torch.cuda.synchronize()
            dist.barrier()
            t0 = time.perf_counter()
            dist.all_reduce(t)
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        res[name] = {"p50_us": ts[len(ts) // 2] * 1e6, "p99_us": percentile(ts, 0.99) * 1e6, "iters": iters,
                     "first_call_bit_exact_vs_fp32_chain": exact}
        # the same call back to back (20 calls, one synchronize): what a loop of collectives pays per call
        torch.cuda.synchronize()
        dist.barrier()
        t0 = time.perf_counter()
        for _ in range(20):
            dist.all_reduce(t)
        torch.cuda.synchronize()
        res[name]["back_to_back_us"] = (time.perf_counter() - t0) / 20 * 1e6
        del x, t
    # What the call itself costs the host, and whether anybody's host thread waits for anybody: 20 calls of
    # the 64 MiB allreduce (enqueue time per call, rendezvous of the host threads among them), then one
    # 4 MiB allreduce that rank 1 enters 50 ms late (how long the OTHER ranks' calls take)
    try:
        be = dist.distributed_c10d._get_default_group()._get_backend(torch.device("cuda"))
        t = torch.ones(4096 * 8192, dtype=torch.bfloat16, device="cuda:0")
        for _ in range(3):
            dist.all_reduce(t)
            torch.cuda.synchronize()
        dist.barrier()
        before = be._rendezvous_counts()
        enq = []
        for _ in range(20):
            t0 = time.perf_counter()
            dist.all_reduce(t)
            enq.append(time.perf_counter() - t0)
        torch.cuda.synchronize()
        after = be._rendezvous_counts()
        enq.sort()
        z = torch.ones(1 << 21, dtype=torch.bfloat16, device="cuda:0")
        for _ in range(3):
            dist.all_reduce(z)
            torch.cuda.synchronize()
        dist.barrier()
        if rank == 1:
            time.sleep(0.05)
        t0 = time.perf_counter()
        w = dist.all_reduce(z, async_op=True)
        call_us = (time.perf_counter() - t0) * 1e6
        w.wait()
        torch.cuda.synchronize()
        done_us = (time.perf_counter() - t0) * 1e6
        res["host_side_of_all_reduce"] = {"c3_enqueue_us_p50": enq[10] * 1e6, "c3_calls": 20,
                                          "host_rendezvous_among_them": int(after[0] - before[0]),
                                          "path": be._last_path(),
                                          "4MiB_call_us_on_rank_0_while_rank_1_is_50_ms_late": call_us,
                                          "4MiB_call_plus_synchronize_us_on_rank_0": done_us}
        del t, z
    except Exception as e:
        res["host_side_of_all_reduce"] = {"error": repr(e)[:200]}

    # C2 as a decode loop runs it: 32 allreduces recorded into one HIP graph per rank process (one launch
    # per process for all 32), replayed; once bare and once with a small kernel of the caller's between them
    try:
        xs = torch.zeros(32, 16 * 8192, dtype=torch.bfloat16, device="cuda:0")
        one = torch.zeros(64, device="cuda:0")
        side = torch.cuda.Stream()  # ONE stream beside the default one for warm-up and capture: every further
        # stream is another hardware queue of this process, and with more queues than the GPU maps at
        # once the scheduler time-slices the rank processes, which a collective cannot stand
        for between in (False, True):
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for k in range(32):
                    dist.all_reduce(xs[k])
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for k in range(32):
                    dist.all_reduce(xs[k])
                    if between:
                        one.add_(1.0)
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
            ts = []
            for _ in range(30):
                xs.fill_(2.0 ** -10)
                torch.cuda.synchronize()
                dist.barrier()
                t0 = time.perf_counter()
                graph.replay()
                torch.cuda.synchronize()
                ts.append(time.perf_counter() - t0)
            ts.sort()
            ok = bool((xs == 2.0 ** -10 * world).all())
            key = "c2_per_allreduce_in_replayed_graph_with_a_small_kernel_between_us" if between else "c2_per_allreduce_in_replayed_graph_us"
            res[key] = {"p50_us": ts[len(ts) // 2] / 32 * 1e6, "p99_us": percentile(ts, 0.99) / 32 * 1e6, "replays": 30,
                        "allreduces_per_graph": 32, "results_exact": ok}
            del graph
        del xs
    except Exception as e:  # bisecting switches: waits or data are missing, results are not checked
        res["c2_per_allreduce_in_replayed_graph_us"] = {"error": repr(e)[:200]}

    # the floor of this way of timing: one trivial kernel of this process + synchronize, with all rank
    # processes doing the same at the same moment (every launch waits for its process's turn)
    one = torch.zeros(64, device="cuda:0")
    ts = []
    for _ in range(200):
        torch.cuda.synchronize()
        dist.barrier()
        t0 = time.perf_counter()
        one.add_(1.0)
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    res["one_trivial_kernel_plus_synchronize"] = {"p50_us": ts[len(ts) // 2] * 1e6, "p99_us": percentile(ts, 0.99) * 1e6, "iters": 200}

    if not large:
        if rank == 0:
            with open(out_path, "w") as f:
                json.dump(res, f)
        dist.destroy_process_group()
        return

    def timed(fn, iters=8, warm=2):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(iters):
            dist.barrier()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return {"p50_us": ts[len(ts) // 2] * 1e6, "iters": iters}

    # C4 through the backend: reduce_scatter_tensor of a 1 GiB bf16 gradient per rank (one staging window)
    grad = torch.empty(536_870_912, dtype=torch.bfloat16, device="cuda:0").normal_(0, 1e-3)
    shard = torch.empty(536_870_912 // world, dtype=torch.bfloat16, device="cuda:0")
    res["c4_reduce_scatter_tensor_1GiB_bf16"] = timed(lambda: dist.reduce_scatter_tensor(shard, grad), iters=5, warm=1)
    del grad, shard
    # C5 through the backend: all_to_all_single with the routing counts of the 256-expert reading
    tokens, hidden, topk = 4096, 7168, 8
    S = c5_split_matrix(torch, world, tokens, topk)
    a_in = torch.empty(tokens * topk, hidden, dtype=torch.bfloat16, device="cuda:0").normal_()
    a_out = torch.empty(int(S[:, rank].sum()), hidden, dtype=torch.bfloat16, device="cuda:0")
    in_split, out_split = S[rank].tolist(), S[:, rank].tolist()
    res["c5_all_to_all_single_448MiB_bf16"] = timed(
        lambda: dist.all_to_all_single(a_out, a_in, out_split, in_split), iters=5, warm=2)
    # ... back to back, what the call costs the host, whether anybody's host thread waits for anybody, and
    # how long the other ranks' calls take when rank 1 enters 50 ms late
    try:
        be = dist.distributed_c10d._get_default_group()._get_backend(torch.device("cuda"))
        dist.barrier()
        before = be._rendezvous_counts()
        enq = []
        t00 = time.perf_counter()
        for _ in range(10):
            t0 = time.perf_counter()
            dist.all_to_all_single(a_out, a_in, out_split, in_split)
            enq.append(time.perf_counter() - t0)
        torch.cuda.synchronize()
        b2b_us = (time.perf_counter() - t00) / 10 * 1e6
        after = be._rendezvous_counts()
        enq.sort()
        dist.barrier()
        if rank == 1:
            time.sleep(0.05)
        t0 = time.perf_counter()
        w = dist.all_to_all_single(a_out, a_in, out_split, in_split, async_op=True)
        call_us = (time.perf_counter() - t0) * 1e6
        w.wait()
        torch.cuda.synchronize()
        res["host_side_of_all_to_all_single"] = {"c5_back_to_back_us": b2b_us, "c5_enqueue_us_p50": enq[5] * 1e6, "c5_calls": 10,
                                                 "host_rendezvous_among_them": int(after[0] - before[0]),
                                                 "waits_for_single_peers_among_them": int(after[2] - before[2]),
                                                 "path": be._last_path(),
                                                 "c5_call_us_on_rank_0_while_rank_1_is_50_ms_late": call_us}
    except Exception as e:
        res["host_side_of_all_to_all_single"] = {"error": repr(e)[:200]}
    del a_in, a_out
    # all_gather_into_tensor of 64 MiB per rank (an FSDP parameter gather): every rank writes its shard
    # into all eight outputs
    part = torch.empty(33_554_432, dtype=torch.bfloat16, device="cuda:0").normal_()
    full = torch.empty(33_554_432 * world, dtype=torch.bfloat16, device="cuda:0")
    res["all_gather_into_tensor_64MiB_bf16"] = timed(lambda: dist.all_gather_into_tensor(full, part), iters=5, warm=1)
    del part, full
    if rank == 0:
        with open(out_path, "w") as f:
            json.dump(res, f)
    dist.destroy_process_group()


def backend_path(world=8, env=None):
    """The drop-in c10d path end to end: `world` rank processes share cuda:0 and call dist.* on GPU
    tensors, timed on the host around the call plus a synchronize.  env: environment of the rank
    processes beyond this process's (None = the backend's defaults); with one only C2 and C3 are timed."""
    import tempfile
    import torch.multiprocessing as mp
    cases = [("c2_256KiB_bf16", 16 * 8192, 20, 200), ("c3_64MiB_bf16", 4096 * 8192, 3, 20)]
    env_all = {"GPU_MAX_HW_QUEUES": "2"}  # what rank processes that share a GPU should run with: no more hardware queues than the GPU maps at once
    env_all.update(env or {})
    before = {k: os.environ.get(k) for k in env_all}
    os.environ.update(env_all)  # the spawned rank processes inherit it
    try:
        with tempfile.TemporaryDirectory() as d:
            out_path = os.path.join(d, "res.json")
            mp.spawn(_backend_rank, args=(world, os.path.join(d, "store"), cases, out_path, env is None), nprocs=world, join=True)
            with open(out_path) as f:
                res = json.load(f)
    finally:
        for k, v in before.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v
    def rounded(d):
        return {k: (round(v, 1) if isinstance(v, float) else rounded(v) if isinstance(v, dict) else v) for k, v in d.items()}
    if env is not None:
        return rounded(res)
    out = {"processes": world, "note": "host-timed dist.* call + synchronize per rank process; all ranks share the one "
                                       "GPU (GPU_MAX_HW_QUEUES=2 per process).  The ranks wait for each other on the device: large collectives (C3, C4, C5) in "
                                       "a one-wavefront barrier kernel in front of the data kernel, whose last workgroup "
                                       "waits for the closing epoch (two launches); small and medium ones (C2) in the "
                                       "data kernel itself, limited to workgroups that hold at most half of the compute "
                                       "units over all ranks; tensors from 1 MiB on are read by the peers in place.  "
                                       "Every launch of a process waits for its turn at the dispatcher, "
                                       "which is what one_trivial_kernel_plus_synchronize measures.  "
                                       "waits_inside_the_data_kernel: the same with MCCL_PG_SYNC=kernel (one launch per "
                                       "collective; not the default because the waiting grids of 7 ranks can keep a "
                                       "register-heavy kernel of the 8th from starting)"}
    out.update(rounded(res))
    return out


def gloo_baseline(world=8, c1_gpu_output=None):
    """N host processes running the same collectives through a CPU c10d backend: the reference's
    "ccl" backend (src/cpu/cpu_ccl.cpp:306-337 allreduce, 819-868 reduce_scatter, 870-961 alltoall)
    when its wheel is installed, else gloo (the stand-in the reference's own CPU harness uses,
    tests/DeepSpeed_test/testccl_cpu.py:20).  C1 runs with 2 processes and its output is compared bit
    for bit with the GPU's (c1_gpu_output: CPU tensor, or None); C2-C5 with `world`.  Reported
    baseline only; the iteration counts of the large cases are cut to keep the whole leg near a
    minute, and say so."""
    import importlib.util
    import tempfile
    import torch
    import torch.multiprocessing as mp
    # the reference's wheel, not the import-name shim this repository carries beside its own package
    spec = importlib.util.find_spec("oneccl_bindings_for_pytorch")
    reference_wheel = spec is not None and spec.origin and not os.path.abspath(spec.origin).startswith(ROOT + os.sep)
    backend = "ccl" if reference_wheel else "gloo"
    try:
        import psutil
        ram_gib = psutil.virtual_memory().available / 2**30
    except Exception:
        ram_gib = 0.0
    c4_factor = 1 if ram_gib >= 24 else 8
    c4_count = 536_870_912 // c4_factor
    tokens, hidden, topk = 4096, 7168, 8
    c1 = [dict(name="c1_16MiB_fp32_2proc", op="all_reduce", count=4_194_304, dtype="float32", dist="uniform", warm=5, iters=20, keep=True)]
    cases = [dict(name="c2_256KiB_bf16", op="all_reduce", count=16 * 8192, dtype="bfloat16", std=0.02, warm=20, iters=300),
             dict(name="c3_64MiB_bf16", op="all_reduce", count=4096 * 8192, dtype="bfloat16", std=0.02, warm=3, iters=12),
             dict(name="c4_reduce_scatter_tensor_bf16", op="reduce_scatter_tensor", count=c4_count, dtype="bfloat16", std=1e-3, warm=1, iters=3),
             dict(name="c5_all_to_all_single_bf16", op="all_to_all_single", count=tokens * topk * hidden, dtype="bfloat16", std=1.0,
                  hidden=hidden, warm=1, iters=5)]
    out = {"backend": backend, "processes": world, "host_cores": len(os.sched_getaffinity(0)),
           "os_cpu_count": os.cpu_count(), "torch": torch.__version__,
           "threads_per_process": max(1, len(os.sched_getaffinity(0)) // world), "pinning": "none",
           "note": "median of host-timed calls between barriers; effective GB/s = algorithmic bytes of the collective "
                   "((N+1) x S for the reductions, 2 x rows moved for the alltoall) / p50; C1 with 2 processes, the rest with %d; "
                   "C4 and C5 with 1 warm-up and 3 / 5 timed calls (a call takes seconds)" % world}
    with tempfile.TemporaryDirectory() as d:
        for w, group in ((2, c1), (world, cases)):
            out_path, keep_path = os.path.join(d, "res%d.json" % w), os.path.join(d, "keep%d.pt" % w)
            mp.spawn(_gloo_rank, args=(w, os.path.join(d, "store%d" % w), backend, group, out_path, keep_path), nprocs=w, join=True)
            with open(out_path) as f:
                res = json.load(f)
            for case in group:
                r = res[case["name"]]
                if "error" in r:
                    out[case["name"]] = r
                    continue
                es = 4 if case["dtype"] == "float32" else 2
                if case["op"] == "all_reduce":
                    alg = (w + 1) * case["count"] * es
                elif case["op"] == "reduce_scatter_tensor":
                    alg = (w + 1) * case["count"] * es  # all ranks' shards together: N inputs read, one gradient's worth written
                else:
                    alg = 2 * w * case["count"] * es
                out[case["name"]] = {"p50_us": round(r["p50_us"], 1), "p99_us": round(r["p99_us"], 1), "iters": r["iters"],
                                     "GBps_effective": round(alg / r["p50_us"] / 1e3, 3)}
            if w == 2 and os.path.exists(keep_path) and c1_gpu_output is not None:
                cpu_out = torch.load(keep_path, weights_only=True)
                out["c1_gpu_equals_cpu_bit_exact"] = bool(torch.equal(cpu_out.view(torch.int32), c1_gpu_output.view(torch.int32)))
    if c4_factor != 1:
        out["c4_reduce_scatter_tensor_bf16"]["scaled_down_by"] = c4_factor
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--extras", default="all",
                    help="comma list of c1,c2,c4,c5,moe,variants,ceilings,placement,lists,xrank,gloo,backend,copycal or all/none "
                         "(copycal: a 512 MiB single-segment copy, the known-size kernel that "
                         "calibrates the FETCH_SIZE / WRITE_SIZE counters; not part of 'all')")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build measures the single-GPU local-reduce path only; "
            "--gpus %d is not supported (run with --gpus 1)." % args.gpus)
        sys.exit(2)

    extras = set("c1,c2,c4,c5,moe,variants,ceilings,placement,lists,xrank,gloo,backend".split(",")) if args.extras == "all" else \
        set() if args.extras == "none" else set(args.extras.split(","))

    import importlib.util
    spec = importlib.util.spec_from_file_location("mccl_build", os.path.join(ROOT, "torch-ccl_amd", "csrc", "build.py"))
    build_mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build_mod)
    build_mod.ensure_built()  # uses what is built; compiles only if nothing is

    # ---------------- the drop-in c10d path (8 rank processes on the one GPU) ----------------
    # Runs first, while this process has not touched the GPU yet: the GPU runs at most eight
    # processes concurrently, a ninth context makes the scheduler time-slice them (20 ms quanta).
    backend_result = None
    if "backend" in extras:
        try:
            backend_result = backend_path(8)
            backend_result["waits_inside_the_data_kernel"] = backend_path(8, env={"MCCL_PG_SYNC": "kernel"})
            # the reference's bisecting switches (src/gpu/dpcpp_ccl.cpp:56-85): what the same calls cost
            # without their cross-rank waits, and what the waits cost alone (neither produces results)
            backend_result["work_only"] = backend_path(8, env={"MCCL_PG_WORK_ONLY": "1"})
            backend_result["sync_only"] = backend_path(8, env={"MCCL_PG_SYNC_ONLY": "1"})
            log("c10d backend:", json.dumps(backend_result))
        except Exception as e:  # informational: never fails the benchmark
            backend_result = {"error": repr(e)[:300]}
            log("c10d backend path failed:", repr(e)[:300])

    import torch
    import torch_ccl_amd as mccl
    from torch_ccl_amd import capi
    import benchlib

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the HIP path cannot run here.")
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(0)
    log("device: %s, %d CUs, %.0f GiB" % (props.name, props.multi_processor_count, props.total_memory / 2**30))

    # ---------------- headline workload: C3 ----------------
    N, COUNT = 8, 4096 * 8192
    S = COUNT * 2
    host_inputs = []
    for r in range(N):
        g = rank_generator(torch, SEED, r)
        host_inputs.append((torch.randn(COUNT, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16))
    ins = [t.to(dev) for t in host_inputs]
    out = torch.empty(COUNT, dtype=torch.bfloat16, device=dev)
    alg_bytes = (N + 1) * S

    # warm-up steps (untimed), then EXACTLY K timed steps between two synchronisations
    for _ in range(args.warmup):
        mccl.reduce_n(ins, out=out, op=mccl.SUM)
    # everything that is not a launch happens before the clock starts: library handle, pointer
    # tables, the event pair
    loop = benchlib.ReduceLoop([ins], [out], variant=capi.VARIANT_AUTO)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loop.run(args.steps)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_us = loop.elapsed_us() / args.steps
    loop.close()
    ms_per_step = wall / args.steps * 1e3
    value = alg_bytes * args.steps / wall / 1e9
    achieved = alg_bytes / (ev_us * 1e-6) / 1e9
    blk, lds = ctypes.c_int(0), ctypes.c_int(0)
    grid = capi.lib().mccl_query_launch(COUNT, N, capi.BF16, capi.SUM, capi.VARIANT_AUTO,
                                        ctypes.byref(blk), ctypes.byref(lds))
    log("C3: %.1f us/launch (events), %.1f GB/s, %.1f%% of peak; wall %.1f us/step" % (
        ev_us, achieved, achieved / PEAK_HBM_GBS * 100, ms_per_step * 1e3))

    result = {
        "metric": "8-rank bf16 allreduce local-reduce HBM GB/s (% of peak); p50 us at 256 KB",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 storage, f32 accumulation",
        "data": "synthetic: N(0,0.02) per (seed=1234, rank), rounded to bf16",
        "config": {"workload": "C3 allreduce SUM, 8 rank buffers x bf16 [4096 x 8192] (64 MiB each) -> one bf16 "
                               "output, all resident in one GPU's HBM",
                   "ranks": N, "elements_per_rank": COUNT, "algorithmic_bytes_per_step": alg_bytes,
                   "kernel": "reduce_vec_kernel<bf16,SUM,8 ranks> shape=stream grid=%d block=%d lds=%d" % (
                       grid, blk.value, lds.value),
                   "buffer_offsets_MiB": [round((t.data_ptr() - ins[0].data_ptr()) / 2**20, 3) for t in ins + [out]]},
        "pct_of_peak": round(value / PEAK_HBM_GBS * 100, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "traffic": profiled_traffic_bytes(),
                     "kernel_us": round(ev_us, 2),
                     "note": "achieved = (N+1)*S algorithmic bytes / average launch duration from one HIP "
                             "event pair around the K timed launches on the launch stream; traffic = "
                             "calibrated rocprofv3 FETCH_SIZE+WRITE_SIZE bytes per launch, read from "
                             "profiles/reduce_bf16_8rank_64MiB_stream.md (offline run of this script)"},
    }

    # parity spot check of the timed output against an on-device fp32 chain
    acc = torch.zeros(COUNT, dtype=torch.float32, device=dev)
    for t in ins:
        acc += t.float()
    same = torch.equal(out.view(torch.int16), acc.to(torch.bfloat16).view(torch.int16))
    result["parity_check"] = "bit-exact vs on-device fp32 chain" if same else "MISMATCH"
    del acc

    c1_gpu_output = None  # kept for the bit-for-bit comparison with the 2-process CPU run

    # ---------------- the same workload with all nine buffers carved from one allocation ----------------
    if "placement" in extras:
        slab = mccl.staggered_copies(ins + [out], stagger_bytes=4096)
        us_slab = min(benchlib.reduce_throughput([slab[:N]], [slab[N]], warmup=5, iters=50) for _ in range(2))
        result["c3_one_allocation_4KiB_stagger"] = {
            "us": round(us_slab, 2), "GBps": round(alg_bytes / us_slab / 1e3, 1),
            "pct_of_peak": round(alg_bytes / us_slab / 1e3 / PEAK_HBM_GBS * 100, 1),
            "headline_buffer_offsets_MiB": [round((t.data_ptr() - ins[0].data_ptr()) / 2**20, 1) for t in ins + [out]],
            "note": "the headline keeps the nine separate allocations torch hands out; carving them from one "
                    "allocation is between 0 and 2.5 % faster, depending on where torch put them"}
        log("placement:", json.dumps(result["c3_one_allocation_4KiB_stagger"]))
        del slab

    # ---------------- what the part sustains: a bare streaming kernel on the same buffers ----------------
    if "ceilings" in extras:
        sink = torch.empty_like(out)
        wide = torch.empty(512 << 20, dtype=torch.uint8, device=dev)  # pure-write target beyond the caches
        cases = (("read_8_streams", ins, sink, 0, 64, 9), ("write_1_stream_512MiB", [], wide, 1, 256, 0),
                 ("copy_1_to_1", ins[:1], sink, 1, 64, 0), ("read_8_write_1", ins, sink, 1, 64, 8))
        ceil = {}
        for name, rd, wr, do_write, block, per_cu in cases:
            us = benchlib.probe_stream(rd, wr, do_write, block=block, workgroups_per_cu=per_cu)
            nbytes = len(rd) * S + (wr.numel() * wr.element_size() if do_write else 0)
            ceil[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                          "pct_of_peak": round(nbytes / us / 1e3 / PEAK_HBM_GBS * 100, 1)}
        ceil["note"] = ("bare xor kernel of the bench library (no conversions, no product code), one 16-byte vector "
                        "per lane per stream; read_8_write_1 is the traffic mix of C3")
        result["machine_ceilings"] = ceil
        result["roofline"]["frac_of_bare_kernel_same_mix"] = round(ceil["read_8_write_1"]["us"] / ev_us, 4)
        # boxes differ: the read-only probe has measured between 81 % and 91 % of the nominal peak
        result["roofline"]["this_box_read_only_frac"] = round(ceil["read_8_streams"]["GBps"] / PEAK_HBM_GBS, 4)
        log("ceilings:", json.dumps(ceil))
        del sink, wide

    # ---------------- C2: 256 KiB latency ----------------
    if "c2" in extras:
        c2 = 16 * 8192
        sets = 16  # 16 sets x 9 buffers x 256 KiB = 36 MiB rotate through the caches
        in_sets = [make_rank_buffers(torch, N, c2, torch.bfloat16, 0.02, dev) for _ in range(sets)]
        outs = [torch.empty(c2, dtype=torch.bfloat16, device=dev) for _ in range(sets)]
        lat = {}
        for name, nsets in (("resident", 1), ("rotating", sets)):
            for vname, v in (("small", capi.VARIANT_SMALL), ("persistent", capi.VARIANT_PERSISTENT)):
                us = sorted(benchlib.reduce_latency(in_sets[:nsets], outs[:nsets], variant=v, warmup=100, iters=1000))
                lat["%s_%s" % (vname, name)] = {"p50_us": round(percentile(us, 0.5), 2),
                                                "p99_us": round(percentile(us, 0.99), 2),
                                                "min_us": round(us[0], 2)}
        b2b = benchlib.reduce_throughput(in_sets[:1], outs[:1], variant=capi.VARIANT_SMALL, warmup=100, iters=1000)
        lat["small_back_to_back_us"] = round(b2b, 2)
        # launch-bound loops belong in a HIP graph: 100 calls captured once, replayed 10 times
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            mccl.reduce_n(in_sets[0], out=outs[0], variant=capi.VARIANT_SMALL)
        torch.cuda.synchronize()
        with torch.cuda.graph(g):
            for _ in range(100):
                mccl.reduce_n(in_sets[0], out=outs[0], variant=capi.VARIANT_SMALL)
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        lat["small_graph_replay_us"] = round(e0.elapsed_time(e1) * 1e3 / 1000, 2)
        lat["iters"] = 1000
        lat["workload"] = "C2 allreduce SUM, 8 x bf16 [16 x 8192] (256 KiB each), one HIP event pair per call"
        result["latency_256KB"] = lat
        result["p50_us_256KB"] = lat["small_resident"]["p50_us"]
        log("C2:", json.dumps(lat))
        del in_sets, outs

    # ---------------- evidence for the shape choice on C3 and C2 ----------------
    if "variants" in extras:
        ev = {}
        for vname, v in (("small", capi.VARIANT_SMALL), ("persistent", capi.VARIANT_PERSISTENT),
                         ("stream", capi.VARIANT_STREAM)):
            us = benchlib.reduce_throughput([ins], [out], variant=v, warmup=5, iters=30)
            ev[vname] = {"us": round(us, 1), "GBps": round(alg_bytes / us / 1e3, 1)}
        result["c3_shapes"] = ev
        log("C3 shapes:", json.dumps(ev))
        # the reference's allreduce is in place on each rank's own buffer: the same launch writing
        # into rank 0's input (same bytes moved; the written DRAM pages were read a moment before)
        fresh = [t.clone() for t in ins]
        us = benchlib.reduce_throughput([fresh], [fresh[0]], warmup=5, iters=30)
        result["c3_in_place_on_rank0"] = {"us": round(us, 1), "GBps": round(alg_bytes / us / 1e3, 1),
                                          "pct_of_peak": round(alg_bytes / us / 1e3 / PEAK_HBM_GBS * 100, 1)}
        log("C3 in place:", json.dumps(result["c3_in_place_on_rank0"]))
        del fresh
        # every op and every rank count up to 8 on 64 MiB messages: % of the HBM peak (AUTO shape)
        matrix = {}
        for opname, opcode in (("SUM", capi.SUM), ("AVG", capi.AVG), ("PROD", capi.PROD), ("MIN", capi.MIN), ("MAX", capi.MAX)):
            row = {}
            for nr in range(2, N + 1):
                us = min(benchlib.reduce_throughput([ins[:nr]], [out], op=opcode, warmup=3, iters=20) for _ in range(2))
                row[str(nr)] = round((nr + 1) * S / us / 1e3 / PEAK_HBM_GBS * 100, 1)
            matrix[opname] = row
        result["pct_of_peak_by_op_and_ranks_64MiB"] = matrix
        log("ops x ranks:", json.dumps(matrix))
        # what a bare kernel (xor, no conversions) sustains for the same read:write mix, best of the
        # residency caps the library chooses from: a 2:1 mix has a lower ceiling than 8:1
        sink = torch.empty_like(out)
        bare = {}
        for nr in range(2, N + 1):
            us = min(benchlib.probe_stream(ins[:nr], sink, 1, block=64, workgroups_per_cu=w) for w in (0, 8, 10, 12, 14))
            bare[str(nr)] = round((nr + 1) * S / us / 1e3 / PEAK_HBM_GBS * 100, 1)
        result["bare_kernel_pct_of_peak_by_ranks_64MiB"] = bare
        log("bare kernel by ranks:", json.dumps(bare))
        del sink
        mccl.reduce_n(ins, out=out, op=mccl.SUM)  # the headline output again, for the checks below

    # ---------------- the cross-rank kernels, all ranks played by this process ----------------
    # Between rank processes these kernels run behind a barrier kernel (the default): no wait at
    # their start, fresh workgroups for the shard reduction and the push, and the last-dispatched
    # workgroup does the closing wait on the ranks' flag words.  Here every rank's word is the same
    # word of this process, so the closing wait passes at once and the figure is the kernel's own
    # (closing count included), without the turn taking of 8 processes that the backend leg includes.
    # (The form that waits at its start, MCCL_PG_SYNC=kernel, is cut to a rank's share of half the
    # GPU's residency and only means something with eight ranks' launches side by side: backend leg.)
    if "xrank" in extras:
        L = capi.lib()
        word = torch.zeros(8, dtype=torch.int64, device=dev)
        counter = torch.zeros(1024, dtype=torch.int32, device=dev)  # MCCL_SYNC_COUNTER_BYTES
        status = torch.zeros(16, dtype=torch.int32).pin_memory()
        words = capi.ptr_table([word.data_ptr()] * N)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        calls = [0]

        def xsync(rank):
            calls[0] += 1
            return capi.XSync(ctypes.cast(words, ctypes.c_void_p), N, rank, 0, 4 * calls[0] + 3,
                              counter.data_ptr(), 5_000_000, status.data_ptr())

        def event_us(fn, reps=20):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / reps

        xr = {}
        in_tab = capi.ptr_table([t.data_ptr() for t in ins])
        xout = torch.zeros_like(out)

        def reduce_sync():
            sy = xsync(0)
            capi.check(L.mccl_reduce_sync(in_tab, xout.data_ptr(), COUNT, capi.BF16, capi.SUM, ctypes.byref(sy), stream))
        us = event_us(reduce_sync)
        xr["reduce_sync_8x64MiB_to_64MiB"] = {"us": round(us, 1), "GBps": round(alg_bytes / us / 1e3, 1),
                                              "pct_of_peak": round(alg_bytes / us / 1e3 / PEAK_HBM_GBS * 100, 1),
                                              "bit_identical_to_reduce_n": bool(torch.equal(xout.view(torch.int16), out.view(torch.int16)))}
        # the in-place allreduce: rank 0's launch alone (its shard of all eight tensors reduced and written
        # back into all eight), checked against the headline output; the whole collective is timed by the
        # backend leg, where the eight ranks' launches run side by side
        tens = [t.clone() for t in ins]
        ten_tab = capi.ptr_table([t.data_ptr() for t in tens])
        shard = L.mccl_allreduce_sync_shard(COUNT, N)

        def allreduce_rank0():
            sy = xsync(0)
            capi.check(L.mccl_allreduce_sync(ten_tab, COUNT, capi.BF16, capi.SUM, ctypes.byref(sy), stream))
        allreduce_rank0()
        torch.cuda.synchronize()
        same = all(torch.equal(t[:shard].view(torch.int16), out[:shard].view(torch.int16)) for t in tens)
        us = event_us(allreduce_rank0)  # (the repetitions reduce an already reduced shard: same traffic)
        moved = 2 * N * shard * 2
        xr["allreduce_sync_rank0_shard_of_8x64MiB"] = {"us": round(us, 1), "bytes_moved": moved, "GBps": round(moved / us / 1e3, 1),
                                                       "pct_of_peak": round(moved / us / 1e3 / PEAK_HBM_GBS * 100, 1),
                                                       "first_pass_bit_identical_to_reduce_n": bool(same)}
        # the pushed allgather: rank 0's launch (its 64 MiB written into slice 0 of eight outputs)
        gathered = [torch.zeros(N * COUNT, dtype=torch.bfloat16, device=dev) for _ in range(N)]
        dst_tab = capi.ptr_table([g.data_ptr() for g in gathered])

        def fanout_rank0():
            sy = xsync(0)
            capi.check(L.mccl_fanout_sync(ins[0].data_ptr(), dst_tab, N, COUNT * 2, ctypes.byref(sy), stream))
        us = event_us(fanout_rank0)
        moved = (N + 1) * COUNT * 2
        xr["fanout_sync_64MiB_into_8_outputs"] = {"us": round(us, 1), "bytes_moved": moved, "GBps": round(moved / us / 1e3, 1),
                                                  "pct_of_peak": round(moved / us / 1e3 / PEAK_HBM_GBS * 100, 1),
                                                  "byte_identical": all(bool(torch.equal(g[:COUNT].view(torch.int16), ins[0].view(torch.int16))) for g in gathered)}
        del gathered
        # the pulls of an all-to-all over resolved addresses: one rank's share of C5's shape (eight pieces of
        # 56 MiB from eight buffers into 448 MiB), beside the plain segment copy of the same segments
        piece = 56 << 20
        a2a_out = torch.zeros(N * piece, dtype=torch.uint8, device=dev)
        table = torch.tensor([t.data_ptr() for t in ins], dtype=torch.int64, device=dev)
        pull_segs = (capi.Segment * N)(*[capi.Segment(0, a2a_out.data_ptr() + r * piece, piece) for r in range(N)])
        plain_segs = (capi.Segment * N)(*[capi.Segment(ins[r].data_ptr(), a2a_out.data_ptr() + r * piece, piece) for r in range(N)])
        from_rank = (ctypes.c_int * N)(*range(N))

        def pulls_resolved():
            sy = xsync(0)
            capi.check(L.mccl_copy_segments_sync_resolved(pull_segs, from_rank, N, table.data_ptr(), 0, ctypes.byref(sy), stream))
        us = event_us(pulls_resolved)
        same = all(bool(torch.equal(a2a_out[r * piece:(r + 1) * piece], ins[r].view(torch.uint8)[:piece])) for r in range(N))
        us_plain = event_us(lambda: capi.check(L.mccl_copy_segments(plain_segs, N, stream)))
        moved = 2 * N * piece
        xr["alltoall_pulls_resolved_8x56MiB"] = {"us": round(us, 1), "bytes_moved": moved, "GBps": round(moved / us / 1e3, 1),
                                                 "pct_of_peak": round(moved / us / 1e3 / PEAK_HBM_GBS * 100, 1),
                                                 "plain_copy_of_the_same_segments_us": round(us_plain, 1), "byte_identical": same}
        del a2a_out
        assert status.tolist()[:2] == [0, 0], status.tolist()
        xr["note"] = ("single process, the form that runs behind a barrier kernel (no opening wait, closing count and "
                      "closing wait): every rank's flag word is the same word, so no launch waits")
        result["cross_rank_kernels_single_process"] = xr
        log("cross-rank kernels:", json.dumps(xr))
        del tens, xout

    # ---------------- coalesced and list forms: one fused launch against one launch per tensor ----------------
    if "lists" in extras:
        def timed_us(fn, reps=20):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / reps
        nb, cnt = 32, 256 * 1024  # 32 gradient tensors of 512 KiB (bf16) on each of 8 ranks
        buckets = [make_rank_buffers(torch, N, cnt, torch.bfloat16, 0.02, dev, on_device=True) for _ in range(nb)]
        bouts = [torch.empty(cnt, dtype=torch.bfloat16, device=dev) for _ in range(nb)]
        # argument tables built once: the timed loops are the C ABI calls alone
        L = capi.lib()
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        all_in = capi.ptr_table([t.data_ptr() for b in buckets for t in b])
        all_out = capi.ptr_table([o.data_ptr() for o in bouts])
        counts = capi.size_table([cnt] * nb)
        per_in = [capi.ptr_table([t.data_ptr() for t in b]) for b in buckets]
        per_out = [ctypes.c_void_p(o.data_ptr()) for o in bouts]
        us_fused = timed_us(lambda: L.mccl_reduce_multi(all_in, N, all_out, counts, nb, capi.BF16, capi.SUM, st))
        fused_copy = [t.clone() for t in bouts]
        us_each = timed_us(lambda: [L.mccl_reduce_n(per_in[b], N, per_out[b], cnt, capi.BF16, capi.SUM,
                                                    capi.VARIANT_AUTO, st) for b in range(nb)])
        same = all(torch.equal(x.view(torch.int16), y.view(torch.int16)) for x, y in zip(fused_copy, bouts))
        pieces = [torch.randn(cnt * (1 + k % 3), device=dev).to(torch.bfloat16) for k in range(16)]
        flat = torch.empty(sum(t.numel() for t in pieces), dtype=torch.bfloat16, device=dev)
        us_pack = timed_us(lambda: mccl.pack(pieces, flat))
        us_copy_ = timed_us(lambda: [flat[o:o + t.numel()].copy_(t) for o, t in
                                     zip([sum(p.numel() for p in pieces[:i]) for i in range(len(pieces))], pieces)])
        result["coalesced_and_list_forms"] = {
            "note": "HIP events bracketing 20 repetitions; reduce calls go straight to the C ABI with prebuilt argument tables, pack/copy through the Python front ends",
            "allreduce_coalesced_32x512KiB_8ranks": {"fused_launches_us": round(us_fused, 1),
                                                      "one_launch_per_tensor_us": round(us_each, 1),
                                                      "bit_identical": same},
            "pack_16_tensors_%dMiB" % (flat.numel() * 2 >> 20): {"fused_pack_us": round(us_pack, 1),
                                                                  "torch_copy_per_tensor_us": round(us_copy_, 1)}}
        log("lists:", json.dumps(result["coalesced_and_list_forms"]))
        del buckets, bouts, fused_copy, pieces, flat

    # ---------------- C1: fp32, 2 ranks, 16 MiB ----------------
    if "c1" in extras:
        c1 = 4_194_304
        a = []
        for r in range(2):
            g = rank_generator(torch, SEED, r)
            a.append((torch.rand(c1, generator=g, dtype=torch.float32) * 2 - 1).to(dev))
        o = torch.empty(c1, dtype=torch.float32, device=dev)
        us = benchlib.reduce_throughput([a], [o], warmup=20, iters=200)
        ok = torch.equal(o, a[0] + a[1])
        c1_gpu_output = o.cpu()
        shapes = {name: round(benchlib.reduce_throughput([a], [o], variant=v, warmup=20, iters=200), 2)
                  for name, v in (("small", capi.VARIANT_SMALL), ("persistent", capi.VARIANT_PERSISTENT),
                                  ("stream", capi.VARIANT_STREAM))}
        # the same with the three buffers 4 KiB off their power-of-two spacing
        st = mccl.staggered_copies(a + [o])
        us_st = benchlib.reduce_throughput([st[:2]], [st[2]], warmup=20, iters=200)
        result["c1_fp32_2ranks_16MiB"] = {"us": round(us, 2), "GBps": round(3 * c1 * 4 / us / 1e3, 1), "bit_exact": ok,
                                          "us_by_shape": shapes,
                                          "buffer_offsets_MiB": [round((t.data_ptr() - a[0].data_ptr()) / 2**20, 3) for t in a + [o]],
                                          "staggered_4KiB_us": round(us_st, 2),
                                          "staggered_4KiB_GBps": round(3 * c1 * 4 / us_st / 1e3, 1)}
        del st
        log("C1:", json.dumps(result["c1_fp32_2ranks_16MiB"]))
        del a, o

    # ---------------- C4: reduce_scatter, 8 x 1 GiB ----------------
    if "c4" in extras:
        c4 = 536_870_912
        m = c4 // N
        big = make_rank_buffers(torch, N, c4, torch.bfloat16, 1e-3, dev, on_device=True)
        shards = [torch.empty(m, dtype=torch.bfloat16, device=dev) for _ in range(N)]
        us_all = benchlib.reduce_scatter_throughput(big, shards, 0, warmup=2, iters=5)
        us_one = benchlib.reduce_scatter_throughput(big, shards[3:4], 3, warmup=2, iters=10)
        # each shard reduced by a launch of its own (what each rank of a group runs)
        us_each = [benchlib.reduce_scatter_throughput(big, shards[r:r + 1], r, warmup=1, iters=5) for r in range(N)]
        # parity on one shard against an on-device fp32 chain
        acc = torch.zeros(m, dtype=torch.float32, device=dev)
        for t in big:
            acc += t[5 * m:6 * m].float()
        ok = torch.equal(shards[5].view(torch.int16), acc.to(torch.bfloat16).view(torch.int16))
        # the same with the rank buffers 4 KiB off their power-of-two spacing (what a caller who
        # places the buffers itself would do)
        offs4 = [round((t.data_ptr() - big[0].data_ptr()) / 2**20, 3) for t in big]
        big_st = mccl.staggered_copies(big)
        us_all_st = benchlib.reduce_scatter_throughput(big_st, shards, 0, warmup=2, iters=5)
        del big_st
        result["c4_reduce_scatter_8x1GiB"] = {
            "rank_buffer_offsets_MiB": offs4,
            "all_shards_staggered_4KiB_us": round(us_all_st, 1),
            "all_shards_staggered_4KiB_GBps": round((N + 1) * c4 * 2 / us_all_st / 1e3, 1),
            "all_shards_us": round(us_all, 1), "all_shards_GBps": round((N + 1) * c4 * 2 / us_all / 1e3, 1),
            "one_shard_us": round(us_one, 1), "one_shard_GBps": round((N + 1) * m * 2 / us_one / 1e3, 1),
            "each_shard_own_launch_us": [round(u, 1) for u in us_each],
            "each_shard_own_launch_GBps": round((N + 1) * c4 * 2 / sum(us_each) / 1e3, 1),
            "shard5_bit_exact_vs_fp32_chain": ok}
        log("C4:", json.dumps(result["c4_reduce_scatter_8x1GiB"]))
        del big, shards, acc

    # ---------------- C5: MoE dispatch all_to_all_single, uneven splits ----------------
    if "c5" in extras:
        # The config names 256 experts and 8 experts per rank, which disagree for 8 ranks: the default is
        # 256 experts (32 per rank); the 64-expert reading (8 per rank) runs as well.  Only the split
        # matrix differs; the bytes moved are the same.
        tokens, hidden, topk = 4096, 7168, 8
        a2a_in = []
        for r in range(N):
            gd = rank_generator(torch, SEED, r, dev)
            a2a_in.append(torch.randn(tokens * topk, hidden, generator=gd, device=dev, dtype=torch.float32).to(torch.bfloat16))
        for n_exp, key in ((256, "c5_alltoallv_moe"), (64, "c5_alltoallv_moe_64_experts")):
            per_rank = n_exp // N
            S5 = torch.zeros(N, N, dtype=torch.int64)
            for r in range(N):
                g = rank_generator(torch, SEED, r)
                logits = torch.randn(tokens, n_exp, generator=g)
                experts = torch.topk(logits, topk, dim=1).indices
                dest = (experts.reshape(-1) // per_rank)
                S5[r] = torch.bincount(dest, minlength=N)
            a2a_out = [torch.empty(int(S5[:, d].sum()), hidden, dtype=torch.bfloat16, device=dev) for d in range(N)]
            us = benchlib.alltoallv_throughput(a2a_in, a2a_out, S5, hidden * 2, warmup=2, iters=5)
            moved = int(S5.sum()) * hidden * 2
            # byte-exact spot check of one (source, destination) segment
            r, d = 2, 6
            so = int(S5[r, :d].sum()); ro = int(S5[:r, d].sum()); rows = int(S5[r, d])
            ok = torch.equal(a2a_out[d][ro:ro + rows], a2a_in[r][so:so + rows])
            result[key] = {"us": round(us, 1), "GBps": round(2 * moved / us / 1e3, 1),
                           "bytes_moved": moved, "n_experts": n_exp, "experts_per_rank": per_rank,
                           "segment_2_to_6_byte_exact": ok,
                           "split_rows_rank0": S5[0].tolist()}
            log("C5:", json.dumps(result[key]))
            del a2a_out
        # the same exchange at decode size: 16 tokens per rank (128 routed rows, 1.75 MiB per rank),
        # all 64 segments in one launch
        S5s = torch.zeros(N, N, dtype=torch.int64)
        for r in range(N):
            g = rank_generator(torch, SEED, r)
            experts = torch.topk(torch.randn(tokens, 256, generator=g)[:16], topk, dim=1).indices
            S5s[r] = torch.bincount(experts.reshape(-1) // 32, minlength=N)
        small_in = [t[:16 * topk] for t in a2a_in]
        small_out = [torch.empty(int(S5s[:, d].sum()), hidden, dtype=torch.bfloat16, device=dev) for d in range(N)]
        us = benchlib.alltoallv_throughput(small_in, small_out, S5s, hidden * 2, warmup=20, iters=200)
        result["c5_alltoallv_decode_16_tokens"] = {"us": round(us, 2), "bytes_moved": int(S5s.sum()) * hidden * 2,
                                                   "launches": 1}
        log("C5 decode size:", json.dumps(result["c5_alltoallv_decode_16_tokens"]))
        del a2a_in, small_in, small_out

    # ---------------- the steps either side of C5: token permute fused into the dispatch, weighted combine ----------------
    if "moe" in extras:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from moe_helpers import combine_tables, route
        tokens, hidden, topk, n_exp = 4096, 7168, 8, 256
        S6, send_tok, _ = route(N, tokens, n_exp, topk, seed=SEED)
        src_rank, src_row = combine_tables(N, tokens, topk, S6, send_tok)
        hid = []
        for r in range(N):
            gd = rank_generator(torch, SEED, r, dev)
            hid.append(torch.randn(tokens, hidden, generator=gd, device=dev, dtype=torch.float32).to(torch.bfloat16))
        idx = [t.to(dev) for t in send_tok]
        recv = [torch.empty(int(S6[:, d].sum()), hidden, dtype=torch.bfloat16, device=dev) for d in range(N)]
        recv2 = [torch.empty_like(t) for t in recv]
        sends = [torch.empty(tokens * topk, hidden, dtype=torch.bfloat16, device=dev) for _ in range(N)]
        sr = [t.to(dev) for t in src_rank]
        so = [t.to(dev) for t in src_row]
        wts = torch.softmax(torch.randn(tokens, topk, generator=rank_generator(torch, SEED, 99)), dim=1).to(dev)
        ys = [torch.empty(tokens, hidden, dtype=torch.bfloat16, device=dev) for _ in range(N)]

        def timed(fn, iters=5):
            fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / iters

        def unfused():
            for r in range(N):
                mccl.gather_rows(hid[r], idx[r], out=sends[r])
            mccl.alltoallv_n(sends, recv2, S6.tolist())

        us_unfused = timed(unfused)
        us_fused = timed(lambda: mccl.moe_dispatch_n(hid, idx, recv, S6.tolist()))
        same = all(torch.equal(a, b) for a, b in zip(recv, recv2))
        us_comb = timed(lambda: [mccl.moe_combine(recv, sr[r], so[r], wts, out=ys[r]) for r in range(N)])
        moved = N * tokens * topk * hidden * 2
        comb_bytes = moved + N * tokens * hidden * 2
        result["moe_dispatch_combine"] = {
            "unfused_gather_plus_alltoallv_us": round(us_unfused, 1), "fused_dispatch_us": round(us_fused, 1),
            "fused_dispatch_GBps": round(2 * moved / us_fused / 1e3, 1), "fused_equals_unfused": same,
            "combine_all_ranks_us": round(us_comb, 1), "combine_GBps": round(comb_bytes / us_comb / 1e3, 1),
            "rows_routed": N * tokens * topk, "row_bytes": hidden * 2}
        log("MoE:", json.dumps(result["moe_dispatch_combine"]))
        del hid, idx, recv, recv2, sends, ys

    # ---------------- counter calibration: a copy of known size ----------------
    if "copycal" in extras:
        cal = 512 << 20
        src = torch.randint(0, 255, (cal,), dtype=torch.uint8, device=dev)
        dst = torch.empty(cal, dtype=torch.uint8, device=dev)
        us = benchlib.copy_throughput([(src.data_ptr(), dst.data_ptr(), cal)], warmup=2, iters=10)
        result["copy_calibration_512MiB"] = {"us": round(us, 1), "GBps": round(2 * cal / us / 1e3, 1),
                                             "bytes_read": cal, "bytes_written": cal,
                                             "bit_exact": bool(torch.equal(src, dst))}
        log("copycal:", json.dumps(result["copy_calibration_512MiB"]))
        del src, dst

    # ---------------- CPU baseline (the oracle port) ----------------
    if not args.no_cpu:
        cb, cpu_out = cpu_baseline(torch, host_inputs, N, COUNT)
        result["cpu_baseline"] = cb
        import numpy as np
        gpu_bits = out.cpu().view(torch.int16).numpy().view(np.uint16)
        result["cpu_baseline"]["gpu_matches_cpu_bit_exact"] = bool(np.array_equal(gpu_bits, cpu_out))
        log("CPU:", json.dumps(cb))
    else:
        result["cpu_baseline"] = None

    # ---------------- N-process CPU c10d baseline (gloo unless the reference's wheel exists) ----------------
    if "gloo" in extras and not args.no_cpu:
        try:
            if c1_gpu_output is None:  # C1 on the GPU for the cross-check, when its own leg did not run
                c1_in = [(torch.rand(4_194_304, generator=rank_generator(torch, SEED, r), dtype=torch.float32) * 2 - 1).to(dev) for r in range(2)]
                c1_gpu_output = mccl.reduce_n(c1_in, op=mccl.SUM).cpu()
                del c1_in
            result["cpu_c10d_baseline"] = gloo_baseline(N, c1_gpu_output)
            log("CPU c10d:", json.dumps(result["cpu_c10d_baseline"]))
        except Exception as e:  # reported baseline only: never fails the benchmark
            result["cpu_c10d_baseline"] = {"error": repr(e)[:300]}
            log("CPU c10d baseline failed:", repr(e)[:300])

    if backend_result is not None:
        result["c10d_backend_path"] = backend_result

    print(json.dumps(result), flush=True)
    # a throughput figure for wrong results is no figure: the line above says what mismatched
    bad = [k for k in ("parity_check",) if result.get(k) == "MISMATCH"]
    if result.get("cpu_baseline") and result["cpu_baseline"].get("gpu_matches_cpu_bit_exact") is False:
        bad.append("cpu_baseline.gpu_matches_cpu_bit_exact")
    if bad:
        log("bench.py: PARITY MISMATCH in", ", ".join(bad))
        sys.exit(4)


if __name__ == "__main__":
    main()
