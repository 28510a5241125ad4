"""The entry point that allocates nothing: mccl_route_counts_noalloc keeps its counters in an array
the library holds on the GPU instead of a caller-provided workspace.  Called through the C ABI and
compared, bit for bit, with mccl_route_counts on the same inputs: two calls in a row, the second
with a smaller input (the shared array keeps the last call's contents), and a refusal beyond the
array's size."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(L, ids_dev, n_experts):
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws = torch.empty(n_experts, dtype=torch.int32, device=DEV)
    want = torch.full((n_experts,), -1, dtype=torch.int64, device=DEV)
    got = torch.full((n_experts,), -2, dtype=torch.int64, device=DEV)
    assert L.mccl_route_counts(ids_dev.data_ptr(), ids_dev.numel(), n_experts, ws.data_ptr(), want.data_ptr(), stream) == 0
    assert L.mccl_route_counts_noalloc(ids_dev.data_ptr(), ids_dev.numel(), n_experts, got.data_ptr(), stream) == 0, \
        L.mccl_last_error().decode()
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_route_counts_without_allocation_equals_the_workspace_form(mccl):
    from torch_ccl_amd import capi
    L = capi.lib()
    g = torch.Generator().manual_seed(2024)
    n_experts = 256
    big = torch.randint(-1, n_experts + 1, (4096 * 8,), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
    small = big[:1000].contiguous()  # second call: smaller input, fewer experts hit
    for ids, n in ((big, n_experts), (small, n_experts), (small[:7].contiguous(), 8), (big, 4096)):
        got, want = _both(L, ids, n)
        assert np.array_equal(got, want), (ids.numel(), n)
        keep = ids.cpu().numpy()
        keep = keep[(keep >= 0) & (keep < n)]
        assert np.array_equal(got, np.bincount(keep, minlength=n))
    # empty input: all zero
    got, want = _both(L, big[:0].contiguous(), 16)
    assert np.array_equal(got, want) and not got.any()
    # beyond the array the library holds: refused, nothing launched
    out = torch.zeros(8192, dtype=torch.int64, device=DEV)
    rc = L.mccl_route_counts_noalloc(big.data_ptr(), big.numel(), 8192, out.data_ptr(), None)
    assert rc == -1 and b"exceed" in L.mccl_last_error()
