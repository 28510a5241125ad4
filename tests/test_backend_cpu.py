"""No-GPU checks of the c10d backend: registration contract, construction, argument errors that
are raised before any device work."""
import os
import tempfile

import pytest
import torch
import torch.distributed as dist


@pytest.fixture(scope="module")
def pkg(mccl):
    return mccl


def _pg(world=1, rank=0):
    d = tempfile.mkdtemp()
    return dist.ProcessGroupCCL(dist.FileStore(os.path.join(d, "s"), world), rank, world)


def test_registration_contract(pkg):
    """import registers backend "ccl" for ROCm ("cuda") tensors and attaches ProcessGroupCCL to
    torch.distributed (oneccl_bindings_for_pytorch/csrc/init.cpp:123-154)."""
    assert "ccl" in dist.Backend.backend_list and "mccl" in dist.Backend.backend_list
    assert dist.Backend.backend_capability["ccl"] == ["cuda"]
    assert dist.ProcessGroupCCL is pkg.ProcessGroupCCL
    assert issubclass(dist.ProcessGroupCCL, torch._C._distributed_c10d.Backend)


def test_construct_without_gpu(pkg):
    pg = _pg(world=4, rank=3)
    assert pg.name() == "ccl" and pg.rank() == 3 and pg.size() == 4
    with pytest.raises(ValueError, match="unexpected rank"):
        _pg(world=2, rank=2)


def test_unexpected_root_rank(pkg):
    """tests/test_c10d_ccl.py:109-113"""
    pg = _pg()
    opts = dist.BroadcastOptions()
    opts.rootRank = -1
    opts.rootTensor = 0
    with pytest.raises(ValueError, match="unexpected rank"):
        pg.broadcast([torch.zeros(1)], opts)


def test_cpu_tensors_are_rejected(pkg):
    pg = _pg()
    with pytest.raises(RuntimeError, match="Tensors are not in same device type"):
        pg.allreduce([torch.zeros(4)])
    with pytest.raises(RuntimeError, match="Tensors are not equal in data type"):
        pg._allgather_base(torch.zeros(2, dtype=torch.int64), torch.zeros(1))
    with pytest.raises(RuntimeError, match="does not support tensors count 2"):
        pg.allreduce([torch.zeros(1), torch.zeros(1)])


def test_collectives_outside_the_path_fail_like_the_reference(pkg):
    pg = _pg()
    with pytest.raises(RuntimeError, match="does not support recvAnysource"):
        pg.recv_anysource([torch.zeros(1)], 0)
    with pytest.raises(RuntimeError, match="Tensors are not in same device type"):
        pg.send([torch.zeros(1)], 0, 0)
    with pytest.raises(ValueError, match="unexpected rank"):
        pg.recv([torch.zeros(1)], 5, 0)
    with pytest.raises(RuntimeError, match="does not support allgather_coalesced"):
        pg.allgather_coalesced([[torch.zeros(1)]], [torch.zeros(1)])


def test_reference_import_name_registers_the_backend(pkg):
    """`import oneccl_bindings_for_pytorch` is what users of the reference write (README.md:176-190)."""
    import oneccl_bindings_for_pytorch as torch_ccl
    import torch.distributed as dist
    assert torch_ccl.ProcessGroupCCL is dist.ProcessGroupCCL
    assert "ccl" in dist.Backend.backend_list
    assert os.path.isdir(torch_ccl.cwd)
    a, b = torch.zeros(4), torch.zeros(4, 4).t()
    assert torch_ccl.is_available([a]) and not torch_ccl.is_available([b]) and not torch_ccl.is_available([a, a])


@pytest.mark.parametrize("env,mode", [({}, 0), ({"TORCH_CCL_WORK_ONLY": "1"}, 1), ({"MCCL_PG_WORK_ONLY": "1"}, 1),
                                      ({"TORCH_CCL_SYNC_ONLY": "1"}, 2), ({"MCCL_PG_SYNC_ONLY": "1"}, 2),
                                      ({"TORCH_CCL_DISABLE_ALLREDUCE": "1"}, 4),
                                      ({"TORCH_CCL_WORK_ONLY": "1", "TORCH_CCL_DISABLE_ALLREDUCE": "1"}, 5),
                                      ({"TORCH_CCL_WORK_ONLY": "0", "MCCL_PG_SYNC_ONLY": "0"}, 0)])
def test_bisecting_switches_parse(pkg, monkeypatch, env, mode):
    """TORCH_CCL_WORK_ONLY / TORCH_CCL_SYNC_ONLY / TORCH_CCL_DISABLE_ALLREDUCE of the reference
    (src/gpu/dpcpp_ccl.cpp:56-85), read when the group is constructed."""
    for k, v in env.items():
        monkeypatch.setenv(k, v)
    assert _pg()._bisect_mode() == mode


def test_work_only_and_sync_only_exclude_each_other(pkg, monkeypatch):
    monkeypatch.setenv("TORCH_CCL_WORK_ONLY", "1")
    monkeypatch.setenv("MCCL_PG_SYNC_ONLY", "1")
    with pytest.raises(RuntimeError, match="exclude each other"):
        _pg()
