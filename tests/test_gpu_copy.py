"""GPU parity of the copy collectives (allgather, alltoall(v), pack/unpack, raw segments)
against the CPU oracle's index maps.  Bar: byte-exact."""
import numpy as np
import pytest
import torch

from helpers import assert_bits_equal
from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _bytes(rng, n):
    return torch.from_numpy(rng.integers(0, 256, size=n, dtype=np.uint8))


def _np(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().reshape(-1)


@pytest.mark.parametrize("n", [1, 2, 8, 13])
@pytest.mark.parametrize("nbytes", [1, 2, 15, 16, 17, 4096, 16384, 16385, 1_000_001])
def test_allgather_bytes(mccl, n, nbytes):
    rng = np.random.default_rng(n * 1000 + nbytes)
    ins = [_bytes(rng, nbytes) for _ in range(n)]
    dev = [t.to(DEV) for t in ins]
    out = torch.zeros(n * nbytes + 32, dtype=torch.uint8, device=DEV)
    mccl.allgather_n(dev, out[:n * nbytes])
    torch.cuda.synchronize()
    assert_bits_equal(_np(out[:n * nbytes]), O.allgather([t.numpy() for t in ins]), "allgather")
    assert int(out[n * nbytes:].sum()) == 0


def test_allgather_kat_rank_values(mccl):
    """_allgather_base of [rank] gives arange(W) (reference tests/test_c10d_ccl.py:377-391)."""
    for W in (2, 4, 8):
        ins = [torch.tensor([r], device=DEV) for r in range(W)]
        out = torch.empty(W, dtype=torch.int64, device=DEV)
        mccl.allgather_n(ins, out)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), torch.arange(W))


def test_allgather_size_error(mccl):
    ins = [torch.tensor([r], device=DEV) for r in range(2)]
    out = torch.empty(3, dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="output tensor size must be equal to world_size times input tensor size"):
        mccl.allgather_n(ins, out)
    with pytest.raises(RuntimeError, match="Tensors are not equal in data type"):
        mccl.allgather_n([torch.tensor([1.0], device=DEV)] * 2, torch.empty(2, dtype=torch.int64, device=DEV))


def test_alltoall_equal_split_kat(mccl):
    """alltoall_base, equal split: in = ones[W,W]*rank -> every rank receives rows i
    (reference tests/test_c10d_ccl.py:443-456)."""
    for W in (2, 4, 8):
        ins = [(torch.ones(W, W) * r).to(DEV) for r in range(W)]
        outs = [(torch.ones(W, W) * -1).to(DEV) for _ in range(W)]
        mccl.alltoallv_n(ins, outs, [[1] * W for _ in range(W)])
        torch.cuda.synchronize()
        expected = torch.cat([torch.ones(1, W) * i for i in range(W)])
        for d in range(W):
            assert torch.equal(outs[d].cpu(), expected)


def test_alltoall_unequal_split_kat(mccl):
    """alltoall_base, uneven: in_splits=[i+1], out_splits=[rank+1]*W
    (reference tests/test_c10d_ccl.py:458-473): rank d sends d+1... precisely, rank r's
    split toward rank i is i+1 rows, so rank d receives d+1 rows from everybody."""
    for W in (2, 4, 8):
        S = [[d + 1 for d in range(W)] for _ in range(W)]
        ins = [(torch.ones(sum(S[r]), W) * r).to(DEV) for r in range(W)]
        outs = [torch.ones((d + 1) * W, W, device=DEV) for d in range(W)]
        mccl.alltoallv_n(ins, outs, S)
        torch.cuda.synchronize()
        for d in range(W):
            expected = torch.cat([torch.ones(d + 1, W) * i for i in range(W)])
            assert torch.equal(outs[d].cpu(), expected)


@pytest.mark.parametrize("n", [2, 5, 8, 17, 64])  # 17 and 64: more segments than one batch of launches holds
@pytest.mark.parametrize("row_bytes", [1, 2, 6, 16, 14336])
@pytest.mark.parametrize("seed", [0, 1])
def test_alltoallv_random_splits(mccl, n, row_bytes, seed):
    rng = np.random.default_rng(seed * 100 + n)
    hi = (40 if row_bytes > 1000 else 3000) if n <= 8 else (6 if row_bytes > 1000 else 300)
    S = rng.integers(0, hi, size=(n, n))
    S[rng.integers(0, n), rng.integers(0, n)] = 0  # at least one empty segment
    if seed == 1:
        S[1, :] = 0  # a rank that sends nothing
    ins = [_bytes(rng, int(S[r].sum()) * row_bytes) for r in range(n)]
    dev_in = [t.to(DEV).view(-1, row_bytes) if t.numel() else torch.empty(0, row_bytes, dtype=torch.uint8, device=DEV) for t in ins]
    dev_out = [torch.zeros(int(S[:, d].sum()), row_bytes, dtype=torch.uint8, device=DEV) for d in range(n)]
    mccl.alltoallv_n(dev_in, dev_out, S.tolist())
    torch.cuda.synchronize()
    want = O.alltoallv([t.numpy() for t in ins], S, row_bytes)
    for d in range(n):
        assert_bits_equal(_np(dev_out[d]), want[d], "dest %d" % d)


def test_alltoallv_pull_matches_all_ranks(mccl):
    """One rank's pull of its n segments equals that rank's output of the all-ranks form."""
    import ctypes
    from torch_ccl_amd import capi
    n, row = 8, 64
    rng = np.random.default_rng(5)
    S = rng.integers(0, 200, size=(n, n))
    ins = [_bytes(rng, int(S[r].sum()) * row).to(DEV) for r in range(n)]
    want = O.alltoallv([t.cpu().numpy() for t in ins], S, row)
    for d in range(n):
        out = torch.zeros(int(S[:, d].sum()) * row, dtype=torch.uint8, device=DEV)
        displ = [int(S[r, :d].sum()) * row for r in range(n)]
        recv = [int(S[r, d]) * row for r in range(n)]
        rc = capi.lib().mccl_alltoallv_pull(capi.ptr_table([t.data_ptr() for t in ins]), n, out.data_ptr(),
                                            capi.size_table(displ), capi.size_table(recv),
                                            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        capi.check(rc)
        torch.cuda.synchronize()
        assert_bits_equal(_np(out), want[d], "pull %d" % d)


@pytest.mark.parametrize("sizes", [[1], [3, 0, 5], [16, 16, 16], [1, 2, 3, 4, 5, 6, 7, 8, 9], [100000, 1, 65537],
                                   list(range(1, 130))])
def test_pack_unpack_roundtrip(mccl, sizes):
    rng = np.random.default_rng(len(sizes))
    srcs = [_bytes(rng, s) for s in sizes]
    dev = [t.to(DEV) for t in srcs]
    flat = torch.zeros(sum(sizes) + 16, dtype=torch.uint8, device=DEV)
    mccl.pack(dev, flat[:sum(sizes)])
    torch.cuda.synchronize()
    assert_bits_equal(_np(flat[:sum(sizes)]), O.pack([t.numpy() for t in srcs]), "pack")
    assert int(flat[sum(sizes):].sum()) == 0
    back = [torch.zeros(s, dtype=torch.uint8, device=DEV) for s in sizes]
    mccl.unpack(flat[:sum(sizes)], back)
    torch.cuda.synchronize()
    for a, b in zip(back, srcs):
        assert_bits_equal(_np(a), b.numpy(), "unpack")


@pytest.mark.parametrize("src_off", [0, 1, 4, 7])
@pytest.mark.parametrize("dst_off", [0, 2, 4, 9])
@pytest.mark.parametrize("nbytes", [1, 5, 31, 127, 129, 2048 + 130, 16384 * 3 + 11])
def test_copy_segments_alignments(mccl, src_off, dst_off, nbytes):
    """Every src/dst alignment class (congruent mod 16, mod 4, neither), sizes below one vector,
    below one cache line and several chunks; canaries around the destination stay untouched."""
    rng = np.random.default_rng(src_off * 100 + dst_off * 10 + nbytes % 7)
    src = _bytes(rng, nbytes + 64).to(DEV)
    dst = torch.full((nbytes + 64,), 0xAB, dtype=torch.uint8, device=DEV)
    mccl.copy_segments([(src.data_ptr() + src_off, dst.data_ptr() + dst_off, nbytes)])
    torch.cuda.synchronize()
    assert torch.equal(dst[dst_off:dst_off + nbytes].cpu(), src[src_off:src_off + nbytes].cpu())
    assert int((dst[:dst_off] != 0xAB).sum()) == 0
    assert int((dst[dst_off + nbytes:] != 0xAB).sum()) == 0


def test_moe_dispatch_small(mccl):
    """Scaled-down MoE token dispatch (uneven all_to_all_single): 8 ranks x 64 tokens x 128
    hidden bf16, top-8 of 256 experts, 32 experts per rank; rows sorted by destination."""
    n, tokens, hidden, topk, n_exp = 8, 64, 128, 8, 256
    per_rank = n_exp // n
    ins, S = [], np.zeros((n, n), dtype=np.int64)
    for r in range(n):
        g = torch.Generator().manual_seed(1234 * 1_000_003 + r)
        logits = torch.randn(tokens, n_exp, generator=g)
        hid = torch.randn(tokens, hidden, generator=g).to(torch.bfloat16)
        experts = torch.topk(logits, topk, dim=1).indices  # [tokens, topk]
        tok = torch.arange(tokens).repeat_interleave(topk)
        exp = experts.reshape(-1)
        order = torch.argsort(exp * tokens + tok, stable=True)  # by (expert, token) => by dest rank
        ins.append(hid[tok[order]].contiguous())
        dest = (exp[order] // per_rank).numpy()
        for d in range(n):
            S[r, d] = int((dest == d).sum())
    dev_in = [t.to(DEV) for t in ins]
    dev_out = [torch.zeros(int(S[:, d].sum()), hidden, dtype=torch.bfloat16, device=DEV) for d in range(n)]
    mccl.alltoallv_n(dev_in, dev_out, S.tolist())
    torch.cuda.synchronize()
    want = O.alltoallv([t.view(torch.int16).numpy() for t in ins], S, hidden * 2)
    for d in range(n):
        assert_bits_equal(_np(dev_out[d]), want[d], "moe dest %d" % d)


def test_copy_segment_larger_than_4gib(mccl):
    """One 4 GiB + 3 byte segment with a misaligned start: 64-bit offsets inside a segment."""
    nbytes = (1 << 32) + 3
    src = torch.arange(253, dtype=torch.uint8, device=DEV).repeat(nbytes // 253 + 2)[:nbytes + 16]
    dst = torch.zeros(nbytes + 32, dtype=torch.uint8, device=DEV)
    mccl.copy_segments([(src.data_ptr() + 5, dst.data_ptr() + 5, nbytes)])
    torch.cuda.synchronize()
    assert torch.equal(dst[5:5 + nbytes], src[5:5 + nbytes])
    assert int(dst[:5].sum()) == 0 and int(dst[5 + nbytes:].sum()) == 0


def test_staggered_copies_keep_the_data_and_leave_the_power_of_two_spacing(mccl):
    ts = [torch.full((1 << 20,), float(k), dtype=torch.float32, device=DEV) for k in range(5)]
    st = mccl.staggered_copies(ts)
    torch.cuda.synchronize()
    for k, (a, b) in enumerate(zip(ts, st)):
        assert torch.equal(a, b) and b.data_ptr() % 256 == 0
        if k:
            assert (b.data_ptr() - st[k - 1].data_ptr()) == (4 << 20) + 4096
    out = mccl.reduce_n(st[:4], op=O.SUM)
    torch.cuda.synchronize()
    assert torch.equal(out, torch.full_like(out, 6.0))


def test_empty_staggered_places_rank_buffers_off_the_regular_spacing(mccl):
    bufs = mccl.empty_staggered(8, (3, 1 << 18), torch.bfloat16, device=DEV)
    nbytes = 3 * (1 << 18) * 2
    assert all(b.shape == (3, 1 << 18) and b.dtype == torch.bfloat16 and b.data_ptr() % 256 == 0 for b in bufs)
    assert all(bufs[k].data_ptr() - bufs[k - 1].data_ptr() == nbytes + 4096 for k in range(1, 8))
    for k, b in enumerate(bufs):
        b.fill_(float(k))
    out = mccl.reduce_n([b.view(-1) for b in bufs])
    torch.cuda.synchronize()
    assert torch.equal(out, torch.full_like(out, 28.0))
    assert all(torch.equal(b, torch.full_like(b, float(k))) for k, b in enumerate(bufs))  # neighbours untouched


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_copy_many_random_segments_in_one_call(mccl, seed):
    """300 segments of random size (0 .. 10 KiB) at random byte offsets in one call: more than one
    kernel-argument table's worth, every alignment, empty segments in between.  The destination
    ranges are disjoint; everything outside them keeps its canary."""
    rng = np.random.default_rng(seed)
    sizes = rng.integers(0, 10240, size=300)
    sizes[rng.integers(0, 300, size=20)] = 0
    gaps = rng.integers(1, 40, size=300)
    src = _bytes(rng, int(sizes.sum()) + 4096).to(DEV)
    dst = torch.full((int((sizes + gaps).sum()) + 64,), 0xCD, dtype=torch.uint8, device=DEV)
    want = np.full(dst.numel(), 0xCD, dtype=np.uint8)
    src_np = src.cpu().numpy()
    segs, so, do = [], int(rng.integers(0, 16)), int(rng.integers(0, 16))
    for sz, gap in zip(sizes.tolist(), gaps.tolist()):
        segs.append((src.data_ptr() + so, dst.data_ptr() + do, sz))
        want[do:do + sz] = src_np[so:so + sz]
        so += sz
        do += sz + gap
    mccl.copy_segments(segs)
    torch.cuda.synchronize()
    assert_bits_equal(dst.cpu().numpy(), want, "random segments")
