"""The two largest configurations of the headline benchmark at their full sizes, through the C ABI.

The CPU oracle would need minutes for these, so each result is checked three ways instead:
against an IEEE-defined chain of torch ops on the device (no kernel of the library involved),
through size-independent properties (shards equal slices of the full reduction; an alltoallv
followed by its transpose returns the input; per-segment checksums), and against the oracle on
windows downloaded from the full-size buffers."""
import numpy as np
import pytest
import torch

from helpers import SEED, assert_bits_equal, bits, oracle_reduce_bits
from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
N = 8


def _device_rank_buffer(rank, count, std, chunk):
    g = torch.Generator(device=DEV).manual_seed(SEED * 1_000_003 + rank)
    x = torch.empty(count, dtype=torch.bfloat16, device=DEV)
    for lo in range(0, count, chunk):
        hi = min(count, lo + chunk)
        x[lo:hi] = (torch.randn(hi - lo, generator=g, device=DEV) * std).to(torch.bfloat16)
    return x


def test_config4_reduce_scatter_8x1gib_full_size(mccl):
    """FSDP gradient reduce_scatter: 8 rank buffers of 536,870,912 bf16 (1 GiB each), N(0, 1e-3),
    8 shards of 67,108,864 elements."""
    count = 536_870_912
    m = count // N
    ins = [_device_rank_buffer(r, count, 1e-3, m) for r in range(N)]
    shards = [torch.empty(m, dtype=torch.bfloat16, device=DEV) for _ in range(N)]
    mccl.reduce_scatter_n(ins, shards, op=O.SUM)  # all shards, one launch
    torch.cuda.synchronize()

    # (1) every shard against the fp32 chain of torch ops
    for s in range(N):
        acc = torch.zeros(m, dtype=torch.float32, device=DEV)
        for t in ins:
            acc += t[s * m:(s + 1) * m].float()
        assert torch.equal(shards[s].view(torch.int16), acc.to(torch.bfloat16).view(torch.int16)), "shard %d" % s
    del acc

    # (2) a shard reduced by a launch of its own equals the same shard of the joint launch
    one = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    for s in (0, 3, 7):
        mccl.reduce_scatter_n(ins, [one], op=O.SUM, shard_first=s)
        torch.cuda.synchronize()
        assert torch.equal(one.view(torch.int16), shards[s].view(torch.int16)), "own launch of shard %d" % s
    del one

    # (3) the shards are the slices of the full allreduce result
    full = mccl.reduce_n(ins, op=O.SUM)
    torch.cuda.synchronize()
    for s in range(N):
        assert torch.equal(full[s * m:(s + 1) * m].view(torch.int16), shards[s].view(torch.int16)), "slice %d" % s

    # (4) the oracle on windows of the full-size buffers (also across a shard boundary)
    win = 1 << 18
    for lo in (0, m - win // 2, 5 * m + 12345, count - win):
        want = oracle_reduce_bits([t[lo:lo + win].cpu() for t in ins])
        assert_bits_equal(bits(full[lo:lo + win]), want, "oracle window at %d" % lo)


def _routing_splits(tokens, topk, n_experts):
    per_rank = n_experts // N
    S = torch.zeros(N, N, dtype=torch.int64)
    for r in range(N):
        g = torch.Generator(device="cpu").manual_seed(SEED * 1_000_003 + r)
        experts = torch.topk(torch.randn(tokens, n_experts, generator=g), topk, dim=1).indices
        S[r] = torch.bincount(experts.reshape(-1) // per_rank, minlength=N)
    return S


@pytest.mark.parametrize("n_experts", [256, 64])
def test_config5_moe_alltoallv_full_size(mccl, n_experts):
    """MoE token dispatch: 8 ranks x (4096 tokens x top-8) rows of 7168 bf16 (448 MiB per rank),
    uneven splits from the routing counts."""
    tokens, topk, hidden = 4096, 8, 7168
    S = _routing_splits(tokens, topk, n_experts)
    assert int(S.sum()) == N * tokens * topk and len(set(S.reshape(-1).tolist())) > 8  # uneven
    ins = []
    for r in range(N):
        g = torch.Generator(device=DEV).manual_seed(SEED * 1_000_003 + r)
        ins.append(torch.randn(tokens * topk, hidden, generator=g, device=DEV).to(torch.bfloat16))
    outs = [torch.full((int(S[:, d].sum()), hidden), float("nan"), dtype=torch.bfloat16, device=DEV) for d in range(N)]
    mccl.alltoallv_n(ins, outs, S)
    torch.cuda.synchronize()

    # (1) the index map, segment by segment, with torch slicing; (2) per-segment checksums
    for r in range(N):
        for d in range(N):
            so, ro, rows = int(S[r, :d].sum()), int(S[:r, d].sum()), int(S[r, d])
            src, dst = ins[r][so:so + rows], outs[d][ro:ro + rows]
            assert torch.equal(src.view(torch.int16), dst.view(torch.int16)), "segment %d -> %d" % (r, d)
            assert int(src.view(torch.int16).sum(dtype=torch.int64)) == int(dst.view(torch.int16).sum(dtype=torch.int64))

    # (3) the transpose alltoallv brings every row home
    back = [torch.empty_like(t) for t in ins]
    mccl.alltoallv_n(outs, back, S.t().contiguous())
    torch.cuda.synchronize()
    for r in range(N):
        assert torch.equal(back[r].view(torch.int16), ins[r].view(torch.int16)), "round trip of rank %d" % r

    # (4) the oracle on one destination rank (its 8 source segments downloaded)
    d = 5
    cpu_in = [t.cpu().view(torch.int16).numpy().view(np.uint16) for t in ins]
    want = O.alltoallv(cpu_in, S.numpy(), hidden * 2)[d]
    assert_bits_equal(bits(outs[d]).view(np.uint8), want, "oracle, destination %d" % d)


def test_more_than_four_gi_elements(mccl):
    """Element and byte offsets beyond 2^32: two u8 buffers of 4 GiB + 1000 bytes summed (u8 wraps),
    and the same span moved as one copy segment; checked against torch's own elementwise add and
    compare on the device."""
    count = (1 << 32) + 1000
    g = torch.Generator(device=DEV).manual_seed(5)
    a = torch.randint(0, 256, (count,), dtype=torch.uint8, device=DEV, generator=g)
    b = torch.randint(0, 256, (count,), dtype=torch.uint8, device=DEV, generator=g)
    out = mccl.reduce_n([a, b])
    torch.cuda.synchronize()
    assert torch.equal(out, a + b)
    assert int(out[-1]) == (int(a[-1]) + int(b[-1])) % 256
    dst = torch.zeros(count + 3, dtype=torch.uint8, device=DEV)
    mccl.copy_segments([(a.data_ptr() + 1, dst.data_ptr() + 3, count - 1)])  # both ends off any boundary
    torch.cuda.synchronize()
    assert torch.equal(dst[3:3 + count - 1], a[1:])
    assert int(dst[:3].sum()) == 0 and int(dst[-1]) == 0


def test_grids_that_wrap(mccl):
    """33 GiB in one buffer: more tiles (reduction) and more chunks (copy) than the largest grid the
    launches use, so every workgroup walks several of them."""
    count = 33 * (1 << 30) + 5
    a = torch.empty(count, dtype=torch.uint8, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(9)
    step = 1 << 32
    for lo in range(0, count, step):
        a[lo:lo + step].random_(0, 256, generator=g)
    out = mccl.reduce_n([a])  # one rank: the chain from +0 returns the input
    torch.cuda.synchronize()
    assert torch.equal(out, a)
    out.zero_()
    mccl.copy_segments([(a.data_ptr(), out.data_ptr(), count)])
    torch.cuda.synchronize()
    assert torch.equal(out, a)
