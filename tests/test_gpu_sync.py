"""The cross-rank entry points of the C ABI with ranks that are processes of their own on one GPU:
mccl_rank_barrier (device-flag barrier, stream-ordered, no host round trip) and
mccl_allreduce_fused (copy-in, rank synchronisation and N-peer reduction in one launch; the
structure of the reference's small allreduce, src/gpu/allreduce_small.h:166-361), checked bit for
bit against the CPU oracle."""
import pytest
import torch.multiprocessing as mp

import sync_worker

pytestmark = pytest.mark.gpu


def _spawn(world, mode):
    ctx = mp.get_context("spawn")
    queues = [ctx.Queue() for _ in range(world)]
    barrier = ctx.Barrier(world)
    mp.spawn(sync_worker.run_rank, args=(world, queues, barrier, mode), nprocs=world, join=True)


@pytest.mark.parametrize("world", [2, 8])
def test_rank_barrier_orders_kernels_across_processes(world):
    _spawn(world, "barrier")


@pytest.mark.parametrize("world", [2, 3, 8])
def test_allreduce_fused_matches_the_oracle(world):
    _spawn(world, "fused")


@pytest.mark.parametrize("world", [2, 8])
def test_allreduce_fused_with_its_epoch_on_the_device_eager_and_replayed_from_a_graph(world):
    _spawn(world, "fused_replay")


@pytest.mark.parametrize("world", [2, 5, 8])
def test_allreduce_over_offers_resolved_on_the_device(world):
    _spawn(world, "offers")


@pytest.mark.parametrize("world", [2, 5, 8])
def test_one_launch_collectives_match_the_oracle(world):
    _spawn(world, "xrank")


def test_waits_are_bounded_and_name_the_late_rank():
    """Failure forced from the host (a rank that never calls, a 0.2 s limit): every kernel exits by
    itself."""
    _spawn(3, "timeout")
