"""The c10d backend "ccl" end to end on one GPU: N rank processes share cuda:0, rendezvous through
a FileStore and construct ProcessGroupCCL(store, rank, size) directly, the way the reference's
MultiProcessTestCase does (tests/test_c10d_ccl.py:97-103)."""
import os
import tempfile

import pytest
import torch
import torch.multiprocessing as mp

import pg_worker

pytestmark = pytest.mark.gpu


def _spawn(world, mode):
    with tempfile.TemporaryDirectory() as d:
        mp.spawn(pg_worker.run_rank, args=(world, os.path.join(d, "store"), mode), nprocs=world, join=True)


@pytest.mark.parametrize("world", [2, 4, 8])
def test_reference_cases(world):
    _spawn(world, "reference")


@pytest.mark.parametrize("world", [2, 5, 8, 10])
def test_random_cases_against_oracle(world):
    """10 ranks: more than the one-launch kernels take (8), so every collective runs as barrier
    kernels around the tuned kernels, and more processes than the GPU runs side by side."""
    _spawn(world, "oracle")


@pytest.mark.parametrize("world", [2, 4])
def test_torch_distributed_api(world):
    _spawn(world, "dist")


@pytest.mark.parametrize("world", [2, 3, 8])
def test_send_recv(world):
    _spawn(world, "p2p")


@pytest.mark.parametrize("world", [2, 8])
def test_identity_replay_interleaved_with_compute(world):
    _spawn(world, "replay")


@pytest.mark.parametrize("world", [2, 8])
def test_all_reduce_recorded_into_a_hip_graph_and_replayed(world):
    """32 dist.all_reduce of the 256 KiB decode message per graph, 50 replays with fresh inputs,
    every result against the oracle; larger tensors and other collectives are refused under capture."""
    _spawn(world, "graph")


def test_a_rank_that_does_not_replay_is_found_by_the_recorded_launches(monkeypatch):
    monkeypatch.setenv("MCCL_BARRIER_TIMEOUT_MS", "1500")
    _spawn(3, "graph_late")


def test_subgroups():
    _spawn(4, "subgroup")


def test_reference_send_recv_cases():
    _spawn(6, "reference_p2p")


@pytest.mark.parametrize("window,world,mode,standing", [("65536", 2, "oracle", "0"), ("65536", 4, "oracle", "1"), ("4096", 3, "p2p", "1"),
                                                        ("65536", 2, "reference", "0"), ("65536", 4, "dist", "0"),
                                                        ("65536", 4, "coalesced_windows", "1"), ("6291456", 8, "oracle", "1"),
                                                        ("8192", 2, "ddp", "1"), ("4096", 6, "reference_p2p", "1"), ("65536", 4, "subgroup", "1"),
                                                        ("65536", 2, "replay", "1"), ("4096", 8, "p2p", "1"),
                                                        ("4096", 3, "list_windows", "0"), ("4096", 8, "list_windows", "0"),
                                                        ("1073741824", 4, "list_windows", "1")])
def test_every_windowed_path_with_a_shrunk_window(monkeypatch, window, world, mode, standing):
    """MCCL_STAGE_WINDOW_BYTES shrinks the staging window, so that messages of a few hundred KiB travel
    in many windows: the same case sets as above must give the same bits.  The 6 MiB window with 8
    ranks puts the two-shot allreduce and a second, shorter window into one message.  (The all-to-alls
    have windows only where the ranks meet on the host: MCCL_PG_STANDING_OFFERS=0 in those runs.)"""
    monkeypatch.setenv("MCCL_STAGE_WINDOW_BYTES", window)
    monkeypatch.setenv("MCCL_PG_STANDING_OFFERS", standing)
    _spawn(world, mode)


def test_coalesced_forms_between_rank_processes_in_one_window():
    """(the same cases without the shrunk window: packed into the staging buffers, which the peers keep mapped)"""
    _spawn(4, "coalesced_windows")


@pytest.mark.parametrize("standing", ["1", "0"])
def test_message_larger_than_one_staging_window(monkeypatch, standing):
    """(with standing offers the all-to-all's pieces of 900 and 1100 MiB are read in place, whatever the
    peers have mapped before; without, the images travel in windows)"""
    monkeypatch.setenv("MCCL_PG_STANDING_OFFERS", standing)
    _spawn(2, "large")


def test_world_size_one_is_a_no_op():
    """world == 1: allreduce leaves the tensor alone (src/gpu/dpcpp_ccl.cpp:752-756), -0.0 included."""
    import torch.distributed as dist
    import torch_ccl_amd  # noqa: F401
    with tempfile.TemporaryDirectory() as d:
        pg = dist.ProcessGroupCCL(dist.FileStore(os.path.join(d, "s"), 1), 0, 1)
        t = torch.tensor([-0.0, 1.5], device="cuda:0")
        pg.allreduce([t]).wait()
        assert t.cpu().view(torch.int32).tolist() == torch.tensor([-0.0, 1.5]).view(torch.int32).tolist()
        out = torch.empty(2, device="cuda:0")
        pg._allgather_base(out, t).wait()
        assert torch.equal(out.cpu(), t.cpu())


@pytest.mark.parametrize("sync", ["host", "barrier"])
def test_missing_rank_raises_instead_of_hanging(monkeypatch, sync):
    """Failure handling forced from the host: a rank skips a collective; the others give up after
    the (shortened) limit and raise -- at the rendezvous of the host threads, which small collectives
    have in both modes, before any kernel waits on the GPU."""
    monkeypatch.setenv("MCCL_BARRIER_TIMEOUT_MS", "1500")
    monkeypatch.setenv("MCCL_PG_SYNC", sync)
    _spawn(3, "missing")


@pytest.mark.parametrize("sync", ["", "kernel"])
def test_wait_honours_its_timeout(monkeypatch, sync):
    """(a 1 MiB allreduce has no rendezvous of the host threads in either device-side mode, so the
    call returns while a peer is still missing and the Work has to wait)"""
    if sync:
        monkeypatch.setenv("MCCL_PG_SYNC", sync)
    monkeypatch.setenv("CCL_BLOCKING_WAIT", "1")
    _spawn(3, "late_peer")


@pytest.mark.parametrize("world", [2, 7, 8, 10])
def test_zero_copy_collectives(world):
    _spawn(world, "zero_copy")


@pytest.mark.parametrize("world", [2, 5, 8])
def test_allreduce_with_offers_exchanged_on_the_device(world):
    """No rendezvous of the host threads in steady state; a late rank does not hold up the others' calls."""
    _spawn(world, "standing")


@pytest.mark.parametrize("world", [2, 5, 8])
def test_all_to_all_with_offers_exchanged_on_the_device(world):
    """all_to_all_single and all_to_all: no rendezvous of the host threads; two ranks meet (nobody else)
    when a piece between them outgrows the buffer kept for it."""
    _spawn(world, "standing_alltoall")


@pytest.mark.parametrize("world,limit", [(8, ""), (5, ""), (4, str(1 << 20))])
def test_a_mixture_of_the_collectives_that_only_enqueue(monkeypatch, world, limit):
    """(limit: MCCL_PG_STANDING_MAX_BYTES shrunk to 1 MiB, so that the all-to-alls' pieces also go the
    way of those larger than any outbox and the other collectives fall back to the rendezvous in between)"""
    if limit:
        monkeypatch.setenv("MCCL_PG_STANDING_MAX_BYTES", limit)
    _spawn(world, "standing_mix")


def test_all_to_all_with_split_sizes_that_do_not_match_is_reported():
    _spawn(3, "alltoall_mismatch")


def test_all_to_all_pieces_larger_than_any_outbox_are_read_in_place(monkeypatch):
    monkeypatch.setenv("MCCL_PG_STANDING_MAX_BYTES", str(2 << 20))
    _spawn(4, "standing_big")


def test_allreduce_with_the_host_rendezvous_instead(monkeypatch):
    """MCCL_PG_STANDING_OFFERS=0: the allreduce above the one-launch size meets at the host rendezvous as
    the other collectives do (tables and offers published per call): same bits."""
    monkeypatch.setenv("MCCL_PG_STANDING_OFFERS", "0")
    _spawn(4, "zero_copy")


def test_a_late_rank_with_gemms_of_its_own_still_gets_in():
    _spawn(8, "heavy_predecessor")


def test_baseline_configs_at_full_size_through_the_backend():
    _spawn(8, "baseline_configs")


@pytest.mark.parametrize("world,mode", [(2, "reference"), (4, "oracle"), (3, "p2p"), (4, "dist"), (2, "zero_copy"), (8, "baseline_configs")])
def test_host_synchronised_fallback(monkeypatch, world, mode):
    """MCCL_PG_SYNC=host: the same cases with hipStreamSynchronize + the host barrier instead of
    device-side waits (what ranks that share a process always use)."""
    monkeypatch.setenv("MCCL_PG_SYNC", "host")
    _spawn(world, mode)


@pytest.mark.parametrize("world,mode", [(4, "oracle"), (8, "oracle"), (8, "zero_copy"), (8, "baseline_configs"), (2, "reference"),
                                        (4, "dist"), (8, "replay")])
def test_waits_inside_the_data_kernels(monkeypatch, world, mode):
    """MCCL_PG_SYNC=kernel: one launch per collective, whose workgroups wait for the other ranks
    themselves (the small fused allreduce, the in-place allreduce, the one-launch pulls and shard
    reductions) instead of a barrier kernel in front of the data kernel: same bits."""
    monkeypatch.setenv("MCCL_PG_SYNC", "kernel")
    _spawn(world, mode)


@pytest.mark.parametrize("sync,elems", [("", 16), ("", 1 << 18), ("kernel", 1 << 18)])
@pytest.mark.parametrize("blocking", ["0", "1"])
def test_missing_rank_found_by_the_wait_on_the_device(monkeypatch, blocking, sync, elems):
    """The same failure with the cross-rank wait on the device (an allreduce of up to 1 MiB is one
    kernel and has no rendezvous of the host threads): the kernel's own bounded wait ends it (a
    1.5 s limit forced from the host), the Work reports failure, the group refuses to go on."""
    if sync:
        monkeypatch.setenv("MCCL_PG_SYNC", sync)
    monkeypatch.setenv("MCCL_TEST_ELEMS", str(elems))
    monkeypatch.setenv("MCCL_BARRIER_TIMEOUT_MS", "1500")
    monkeypatch.setenv("CCL_BLOCKING_WAIT", blocking)
    _spawn(3, "missing_device")


def test_zero_copy_with_barrier_kernels_instead_of_one_launch(monkeypatch):
    """MCCL_PG_ONE_LAUNCH_MAX_BYTES=0: the peers' tensors are still read in place, but between
    barrier kernels by the bandwidth-tuned kernels (what groups of more than eight ranks and very
    large tensors use): same bits."""
    monkeypatch.setenv("MCCL_PG_ONE_LAUNCH_MAX_BYTES", "0")
    _spawn(4, "zero_copy")


def test_all_gather_with_pulls_instead_of_pushes(monkeypatch):
    """MCCL_PG_ALLGATHER_PUSH=0: all_gather_into_tensor offers the inputs and every rank pulls (what
    outputs too large to be shared use) instead of writing into the peers' outputs: same bits."""
    monkeypatch.setenv("MCCL_PG_ALLGATHER_PUSH", "0")
    _spawn(4, "zero_copy")


def test_staged_when_zero_copy_is_switched_off(monkeypatch):
    monkeypatch.setenv("MCCL_PG_ZERO_COPY", "0")
    _spawn(4, "oracle")


def test_receive_without_a_sender_raises_instead_of_hanging(monkeypatch):
    monkeypatch.setenv("MCCL_BARRIER_TIMEOUT_MS", "1500")
    _spawn(2, "missing_sender")


def test_thread_ranks_in_one_process():
    """Ranks as threads of one process (same address space: staging buffers are shared by raw
    pointer instead of an IPC handle), rendezvous through a HashStore."""
    import threading
    import torch.distributed as dist
    import torch_ccl_amd  # noqa: F401
    world = 4
    store = dist.HashStore()
    errors = []

    def body(rank):
        try:
            pg = dist.ProcessGroupCCL(store, rank, world)
            t = torch.full((100000,), float(rank + 1), device="cuda:0")
            pg.allreduce([t]).wait()
            torch.cuda.synchronize()
            assert float(t[0]) == world * (world + 1) / 2 and float(t[-1]) == world * (world + 1) / 2
            out = torch.empty(world * 5, device="cuda:0")
            pg._allgather_base(out, torch.full((5,), float(rank), device="cuda:0")).wait()
            torch.cuda.synchronize()
            assert out.cpu().tolist() == [float(r) for r in range(world) for _ in range(5)]
            got = torch.zeros(1000, device="cuda:0")
            w = pg.recv([got], (rank - 1) % world, 0)
            pg.send([torch.full((1000,), float(rank), device="cuda:0")], (rank + 1) % world, 0).wait()
            w.wait()
            assert got.cpu().tolist() == [float((rank - 1) % world)] * 1000
            pg.barrier().wait()
            del w, pg
        except Exception as e:  # noqa: BLE001
            errors.append((rank, repr(e)))

    threads = [threading.Thread(target=body, args=(r,)) for r in range(world)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert not errors, errors
    assert not any(th.is_alive() for th in threads)


@pytest.mark.parametrize("same_stream,blocking", [("1", "0"), ("0", "1"), ("1", "1")])
def test_env_switches(monkeypatch, same_stream, blocking):
    monkeypatch.setenv("CCL_SAME_STREAM", same_stream)
    monkeypatch.setenv("CCL_BLOCKING_WAIT", blocking)
    _spawn(2, "env")


@pytest.mark.parametrize("world", [2, 4])
def test_ddp_and_fsdp_style_callers(world):
    _spawn(world, "ddp")


def test_verbose_logs_one_line_per_collective(monkeypatch, capfd):
    """ONECCL_BINDINGS_FOR_PYTORCH_ENV_VERBOSE=1: every collective says which way it took, the
    one-launch small allreduce included."""
    monkeypatch.setenv("ONECCL_BINDINGS_FOR_PYTORCH_ENV_VERBOSE", "1")
    _spawn(2, "env")
    out = capfd.readouterr().out
    assert "oneccl_bindings_for_pytorch::allreduce [0/2#" in out and "oneccl_bindings_for_pytorch::allreduce [1/2#" in out, out[-2000:]
    assert "standing offers" in out, out[-2000:]  # (the 4 MiB allreduce of the case: offers exchanged on the device)

