"""Every tuning knob of mccl_set_tuning changes launch geometry only: results must stay the
oracle's bits at unusual values of each knob (the values a sweep would visit)."""
import numpy as np
import pytest
import torch

from helpers import TORCH_TO_CODE, assert_bits_equal, bits, oracle_reduce_bits, rank_buffer, to_carrier
from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture
def knobs(mccl):
    from torch_ccl_amd import capi
    L = capi.lib()
    yield lambda knob, value: L.mccl_set_tuning(knob, value)
    for k in range(7):  # MCCL_TUNE_COUNT_
        assert L.mccl_set_tuning(k, 0) == 0  # back to the default


@pytest.mark.parametrize("waves", [1, 5, 13, 40])
def test_stream_residency(mccl, knobs, waves):
    from torch_ccl_amd import capi
    knobs(capi.TUNE_STREAM_WAVES_PER_CU, waves)
    for n, dtype in ((8, torch.bfloat16), (3, torch.float32)):
        ins = [rank_buffer((1 << 20) + 3, dtype, r) for r in range(n)]
        got = mccl.reduce_n([t.to(DEV) for t in ins], variant=capi.VARIANT_STREAM)
        torch.cuda.synchronize()
        assert_bits_equal(bits(got), oracle_reduce_bits(ins), "stream waves %d n %d" % (waves, n))


@pytest.mark.parametrize("blocks", [1, 3, 32])
def test_persistent_grid(mccl, knobs, blocks):
    from torch_ccl_amd import capi
    knobs(capi.TUNE_PERSISTENT_BLOCKS_PER_CU, blocks)
    ins = [rank_buffer((1 << 21) + 77, torch.float16, r) for r in range(4)]
    got = mccl.reduce_n([t.to(DEV) for t in ins], variant=capi.VARIANT_PERSISTENT)
    torch.cuda.synchronize()
    assert_bits_equal(bits(got), oracle_reduce_bits(ins), "persistent blocks %d" % blocks)


@pytest.mark.parametrize("small_max,stream_min", [(1, 1), (1 << 40, 1 << 40), (1, 1 << 40)])
def test_auto_thresholds(mccl, knobs, small_max, stream_min):
    """AUTO pushed to each of its three shapes for the same message."""
    from torch_ccl_amd import capi
    knobs(capi.TUNE_SMALL_MAX_BYTES, small_max)
    knobs(capi.TUNE_STREAM_MIN_TOTAL_BYTES, stream_min)
    for n in (2, 8):
        ins = [rank_buffer(300001, torch.bfloat16, r) for r in range(n)]
        got = mccl.reduce_n([t.to(DEV) for t in ins])
        torch.cuda.synchronize()
        assert_bits_equal(bits(got), oracle_reduce_bits(ins), "auto n %d" % n)


@pytest.mark.parametrize("waves", [1, 7, 64])
def test_copy_residency(mccl, knobs, waves):
    from torch_ccl_amd import capi
    knobs(capi.TUNE_COPY_WAVES_PER_CU, waves)
    g = torch.Generator().manual_seed(waves)
    src = torch.randint(0, 255, ((8 << 20) + 5,), generator=g, dtype=torch.uint8)
    d_src = src.to(DEV)
    dst = torch.zeros_like(d_src)
    mccl.copy_segments([(d_src.data_ptr(), dst.data_ptr(), src.numel())])
    rows = torch.randint(0, 255, (3000, 4096), generator=g, dtype=torch.uint8)
    idx = torch.randint(0, 3000, (9000,), generator=g, dtype=torch.int64)
    out = mccl.gather_rows(rows.to(DEV), idx.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), src)
    assert torch.equal(out.cpu(), rows[idx])


@pytest.mark.parametrize("pieces,waves", [(1, 0), (3, 0), (16, 0), (2, 1), (2, 4), (5, 32)])
@pytest.mark.parametrize("topk", [2, 8])
def test_combine_geometry(mccl, knobs, pieces, waves, topk):
    """Pieces per wavefront and the persistent grid of the combine (the latter walks several chunks
    per wavefront and looks the next chunk's routing up early)."""
    from torch_ccl_amd import capi
    knobs(capi.TUNE_COMBINE_PIECES_PER_WAVE, pieces)
    if waves:
        knobs(capi.TUNE_COMBINE_WAVES_PER_CU, waves)
    n, tokens, hidden, dtype = 4, 700, 7168, torch.bfloat16
    g = torch.Generator().manual_seed(pieces * 100 + waves + topk)
    x = [torch.randn(90 + r, hidden, generator=g).to(dtype) for r in range(n)]
    src_rank = torch.randint(0, n, (tokens, topk), generator=g, dtype=torch.int32)
    src_row = torch.randint(0, 90, (tokens, topk), generator=g, dtype=torch.int64)
    src_rank[5, 0] = -1          # skipped entries
    src_row[6, topk - 1] = 10_000
    w = torch.randn(tokens, topk, generator=g).contiguous()
    y = mccl.moe_combine([t.to(DEV) for t in x], src_rank.to(DEV), src_row.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    want = O.moe_combine([to_carrier(t) for t in x], src_rank.numpy(), src_row.numpy(), w.numpy(),
                         tokens, topk, hidden, TORCH_TO_CODE[dtype])
    assert_bits_equal(bits(y), want.view(np.uint16), "combine pieces %d waves %d topk %d" % (pieces, waves, topk))
