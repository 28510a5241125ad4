"""GPU parity of the steps either side of the MoE all_to_all: row gather, fused dispatch, weighted
combine.  Copies are byte-exact; the combine is bit-exact against the oracle's fp32 chain."""
import numpy as np
import pytest
import torch

from helpers import assert_bits_equal, bits, to_carrier, TORCH_TO_CODE
from moe_helpers import combine_tables, route
from oracle import oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _u8(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().reshape(-1)


@pytest.mark.parametrize("row_elems,dtype", [(7168, torch.bfloat16), (128, torch.bfloat16), (1025, torch.float32),
                                             (3, torch.uint8), (1000, torch.int16)])
def test_gather_rows_matches_oracle(mccl, row_elems, dtype):
    g = torch.Generator().manual_seed(row_elems)
    rows = 300
    src = torch.randint(0, 127, (rows, row_elems), generator=g).to(dtype)
    idx = torch.randint(0, rows, (1000,), generator=g, dtype=torch.int64)
    out = mccl.gather_rows(src.to(DEV), idx.to(DEV))
    torch.cuda.synchronize()
    want = O.gather_rows(_u8(src), idx.numpy(), row_elems * src.element_size())
    assert_bits_equal(_u8(out), want, "gather_rows")
    assert torch.equal(out.cpu(), src[idx])


def test_gather_rows_skips_out_of_range_indices(mccl):
    src = torch.arange(40, dtype=torch.float32).view(10, 4).to(DEV)
    idx = torch.tensor([3, -1, 10, 0, 99], dtype=torch.int64, device=DEV)
    out = torch.full((5, 4), -7.0, device=DEV)
    mccl.gather_rows(src, idx, out=out)
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [[12, 13, 14, 15], [-7] * 4, [-7] * 4, [0, 1, 2, 3], [-7] * 4]


@pytest.mark.parametrize("n,tokens,hidden,topk,n_exp", [(8, 64, 128, 8, 256), (4, 100, 96, 2, 16), (2, 33, 7168, 4, 8),
                                                        (17, 30, 64, 3, 34)])
def test_fused_dispatch_equals_gather_then_alltoallv(mccl, n, tokens, hidden, topk, n_exp):
    S, send_tok, _ = route(n, tokens, n_exp, topk)
    hid = []
    for r in range(n):
        g = torch.Generator().manual_seed(77 + r)
        hid.append(torch.randn(tokens, hidden, generator=g).to(torch.bfloat16))
    dev_h = [h.to(DEV) for h in hid]
    dev_i = [t.to(DEV) for t in send_tok]
    fused = [torch.zeros(int(S[:, d].sum()), hidden, dtype=torch.bfloat16, device=DEV) for d in range(n)]
    mccl.moe_dispatch_n(dev_h, dev_i, fused, S.tolist())
    # unfused: materialise the permuted send buffers, then the uneven alltoall copy
    sends = [mccl.gather_rows(dev_h[r], dev_i[r]) for r in range(n)]
    unfused = [torch.zeros_like(f) for f in fused]
    mccl.alltoallv_n(sends, unfused, S.tolist())
    torch.cuda.synchronize()
    want = O.moe_dispatch([_u8(h) for h in hid], [t.numpy() for t in send_tok], S, hidden * 2)
    for d in range(n):
        assert_bits_equal(_u8(fused[d]), want[d], "fused dispatch dest %d" % d)
        assert_bits_equal(_u8(unfused[d]), want[d], "unfused dispatch dest %d" % d)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("n,tokens,hidden,topk,n_exp", [(8, 64, 128, 8, 256), (4, 50, 200, 3, 16)])
def test_combine_matches_oracle(mccl, dtype, n, tokens, hidden, topk, n_exp):
    """Rank 0's tokens: dispatch, pretend the experts scaled their rows, combine with random
    weights; compare with the oracle's fp32 chain bit for bit."""
    S, send_tok, _ = route(n, tokens, n_exp, topk)
    src_rank, src_row = combine_tables(n, tokens, topk, S, send_tok)
    x = []
    for d in range(n):
        g = torch.Generator().manual_seed(500 + d)
        x.append(torch.randn(int(S[:, d].sum()), hidden, generator=g).to(dtype))
    g = torch.Generator().manual_seed(9)
    w = torch.softmax(torch.randn(tokens, topk, generator=g), dim=1).contiguous()
    for r in (0, n - 1):
        y = mccl.moe_combine([t.to(DEV) for t in x], src_rank[r].to(DEV), src_row[r].to(DEV), w.to(DEV))
        torch.cuda.synchronize()
        want = O.moe_combine([to_carrier(t) for t in x], src_rank[r].numpy(), src_row[r].numpy(), w.numpy(),
                             tokens, topk, hidden, TORCH_TO_CODE[dtype])
        width = {2: np.uint16, 4: np.uint32}[y.element_size()]
        assert_bits_equal(bits(y), want.view(width), "combine rank %d %s" % (r, dtype))


def test_dispatch_then_one_hot_combine_returns_the_tokens(mccl):
    """Round trip at the real row length: with weight 1 on a token's first copy and 0 elsewhere,
    combine(dispatch(h)) == h exactly (0 + 1*x + 0*y... adds exact zeros)."""
    n, tokens, hidden, topk, n_exp = 8, 256, 7168, 8, 256
    S, send_tok, _ = route(n, tokens, n_exp, topk)
    src_rank, src_row = combine_tables(n, tokens, topk, S, send_tok)
    hid = []
    for r in range(n):
        g = torch.Generator().manual_seed(31 + r)
        hid.append((torch.randn(tokens, hidden, generator=g).abs() + 0.5).to(torch.bfloat16).to(DEV))  # no -0, no NaN
    recv = [torch.zeros(int(S[:, d].sum()), hidden, dtype=torch.bfloat16, device=DEV) for d in range(n)]
    mccl.moe_dispatch_n(hid, [t.to(DEV) for t in send_tok], recv, S.tolist())
    w = torch.zeros(tokens, topk)
    w[:, 0] = 1.0
    for r in range(n):
        y = mccl.moe_combine(recv, src_rank[r].to(DEV), src_row[r].to(DEV), w.to(DEV))
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), hid[r].view(torch.int16)), "rank %d" % r
    # and with uniform weights 1/8 (a power of two: exact products) every copy is the token itself
    w = torch.full((tokens, topk), 0.125)
    y = mccl.moe_combine(recv, src_rank[3].to(DEV), src_row[3].to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), hid[3].view(torch.int16))


@pytest.mark.parametrize("topk", [1, 2, 3, 4, 5, 8, 9, 12, 17])
@pytest.mark.parametrize("hidden", [8, 520, 7168])
def test_combine_any_topk_with_skipped_entries(mccl, topk, hidden):
    """Random routing tables (any rank, any row) for top-k below, at and above the 8 entries one
    group of row loads covers; a tenth of the entries point outside their buffer (negative rank,
    rank >= n, negative row, row past the end) and must be skipped, as the oracle skips them."""
    n, tokens, dtype = 4, 77, torch.bfloat16
    g = torch.Generator().manual_seed(1000 * topk + hidden)
    rows = [60 + 11 * r for r in range(n)]
    x = [torch.randn(rows[r], hidden, generator=g).to(dtype) for r in range(n)]
    src_rank = torch.randint(0, n, (tokens, topk), generator=g, dtype=torch.int32)
    src_row = torch.stack([torch.randint(0, rows[int(r)], (1,), generator=g)[0] for r in src_rank.reshape(-1)]).reshape(tokens, topk).to(torch.int64)
    bad = torch.rand(tokens, topk, generator=g) < 0.1
    kind = torch.randint(0, 4, (tokens, topk), generator=g)
    src_rank = torch.where(bad & (kind == 0), torch.full_like(src_rank, -1), src_rank)
    src_rank = torch.where(bad & (kind == 1), torch.full_like(src_rank, n), src_rank)
    src_row = torch.where(bad & (kind == 2), torch.full_like(src_row, -3), src_row)
    src_row = torch.where(bad & (kind == 3), torch.full_like(src_row, 10_000), src_row)
    w = torch.randn(tokens, topk, generator=g).contiguous()
    y = mccl.moe_combine([t.to(DEV) for t in x], src_rank.to(DEV), src_row.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    want = O.moe_combine([to_carrier(t) for t in x], src_rank.numpy(), src_row.numpy(), w.numpy(),
                         tokens, topk, hidden, TORCH_TO_CODE[dtype])
    assert_bits_equal(bits(y), want.view(np.uint16), "combine topk %d hidden %d" % (topk, hidden))


@pytest.mark.parametrize("row_bytes", [1, 15, 16, 17, 32, 48, 256, 1008, 1024, 1040, 2047, 2048, 2049, 2560, 4099, 6160, 14338])
@pytest.mark.parametrize("src_off,dst_off", [(0, 0), (1, 0), (0, 3), (5, 9)])
def test_gather_rows_any_row_size_and_alignment(mccl, row_bytes, src_off, dst_off):
    """Byte rows of every size class (below a vector, around one 2 KiB piece, several pieces with a
    ragged end) gathered between buffers that start off any boundary; the bytes around the
    destination must stay untouched."""
    g = torch.Generator().manual_seed(row_bytes * 31 + src_off * 7 + dst_off)
    rows, picks = 37, 90
    src_buf = torch.randint(0, 255, (src_off + rows * row_bytes + 8,), generator=g, dtype=torch.uint8).to(DEV)
    dst_buf = torch.full((dst_off + picks * row_bytes + 64,), 0xAB, dtype=torch.uint8, device=DEV)
    src = src_buf[src_off:src_off + rows * row_bytes].view(rows, row_bytes)
    dst = dst_buf[dst_off:dst_off + picks * row_bytes].view(picks, row_bytes)
    idx = torch.randint(0, rows, (picks,), generator=g, dtype=torch.int64)
    mccl.gather_rows(src, idx.to(DEV), out=dst)
    torch.cuda.synchronize()
    want = O.gather_rows(_u8(src), idx.numpy(), row_bytes)
    assert_bits_equal(_u8(dst), want, "gather_rows %d bytes" % row_bytes)
    assert int((dst_buf[:dst_off] != 0xAB).sum()) == 0 and int((dst_buf[dst_off + picks * row_bytes:] != 0xAB).sum()) == 0


@pytest.mark.parametrize("row_bytes", [16, 80, 512, 1024, 1536, 2560, 10256])
def test_gather_small_rows_skip_out_of_range_and_ragged_ends(mccl, row_bytes):
    """Rows that are not a whole number of 2 KiB pieces travel as 2 KiB windows of the destination
    (several rows, or parts of two, per wavefront): a byte count that does not fill the last window,
    indices outside the source (skipped: the destination row keeps its bytes) and the fused dispatch
    over several segments."""
    g = torch.Generator().manual_seed(row_bytes)
    rows, picks = 53, 1001
    src = torch.randint(0, 255, (rows, row_bytes), generator=g, dtype=torch.uint8)
    idx = torch.randint(0, rows, (picks,), generator=g, dtype=torch.int64)
    bad = torch.rand(picks, generator=g) < 0.15
    idx = torch.where(bad, torch.where(torch.rand(picks, generator=g) < 0.5, torch.full_like(idx, -2), torch.full_like(idx, rows + 7)), idx)
    out = torch.full((picks, row_bytes), 0xCD, dtype=torch.uint8, device=DEV)
    mccl.gather_rows(src.to(DEV), idx.to(DEV), out=out)
    torch.cuda.synchronize()
    want = torch.full((picks, row_bytes), 0xCD, dtype=torch.uint8)
    good = ~bad
    want[good] = src[idx[good]]
    assert torch.equal(out.cpu(), want)
    # fused dispatch with small rows: 3 ranks, uneven splits, against gather + alltoallv
    n = 3
    S = np.array([[5, 0, 300], [17, 40, 1], [0, 129, 64]])
    hid = [torch.randint(0, 255, (200, row_bytes), generator=g, dtype=torch.uint8).to(DEV) for _ in range(n)]
    ix = [torch.randint(0, 200, (int(S[r].sum()),), generator=g, dtype=torch.int64).to(DEV) for r in range(n)]
    fused = [torch.zeros(int(S[:, d].sum()), row_bytes, dtype=torch.uint8, device=DEV) for d in range(n)]
    mccl.moe_dispatch_n(hid, ix, fused, S.tolist())
    torch.cuda.synchronize()
    want = O.moe_dispatch([_u8(h) for h in hid], [t.cpu().numpy() for t in ix], S, row_bytes)
    for d in range(n):
        assert_bits_equal(_u8(fused[d]), want[d], "small-row dispatch dest %d" % d)


@pytest.mark.parametrize("n_experts,npairs", [(1, 5), (8, 0), (64, 4096 * 8), (256, 4096 * 8), (4096, 1_000_003), (257, 77)])
def test_route_counts_match_the_oracle(mccl, n_experts, npairs):
    """Per-expert pair counts on the device against the oracle; ids out of range are ignored; the
    workspace comes back zero, so that a second, smaller call through the same workspace is right too."""
    from oracle import oracle as O
    g = torch.Generator().manual_seed(11 + n_experts)
    ids = torch.randint(-2, n_experts + 2, (npairs,), generator=g, dtype=torch.int64).to(torch.int32)
    ws = torch.full((n_experts,), 12345, dtype=torch.int32, device=DEV)  # dirty on purpose: the call clears it
    got = mccl.route_counts(ids.to(DEV), n_experts, workspace=ws)
    assert np.array_equal(got.cpu().numpy(), O.route_counts(ids.numpy(), n_experts))
    assert int(ws.abs().sum()) == 0
    half = ids[: npairs // 3].contiguous()
    got = mccl.route_counts(half.to(DEV), n_experts, workspace=ws)
    assert np.array_equal(got.cpu().numpy(), O.route_counts(half.numpy(), n_experts))


def test_route_counts_of_the_c5_routing_give_the_split_matrix(mccl):
    """The top-8-of-256 routing of the dispatch workload: counts summed per destination rank equal
    torch.bincount of the destination ranks, i.e. the row of the all_to_all_single split matrix."""
    g = torch.Generator().manual_seed(1234 * 1_000_003)
    experts = torch.topk(torch.randn(4096, 256, generator=g), 8, dim=1).indices.to(torch.int32)
    counts = mccl.route_counts(experts.reshape(-1).contiguous().to(DEV), 256).cpu()
    per_rank = counts.view(8, 32).sum(dim=1)
    assert torch.equal(per_rank, torch.bincount(experts.reshape(-1).long() // 32, minlength=8))
    assert int(per_rank.sum()) == 4096 * 8
