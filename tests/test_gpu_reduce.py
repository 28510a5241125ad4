"""GPU parity of the N-buffer reduction (mccl_reduce_n / _reduce_scatter_n / _reduce_multi)
against the CPU oracle.  Bar: bit-exact for every dtype (the kernel runs the same
ascending-rank chain and the same single rounding as the oracle; the 1-ulp allowance for
f16/bf16 is not needed)."""
import numpy as np
import pytest
import torch

from helpers import (ALL_DTYPES, FLOAT_DTYPES, INT_DTYPES, assert_bits_equal, bits,
                     oracle_reduce_bits, rank_buffer, to_carrier, TORCH_TO_CODE)
from oracle import oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
OPS = {"sum": O.SUM, "prod": O.PROD, "min": O.MIN, "max": O.MAX}


def _run(mccl, cpu_inputs, op, variant=0, out=None):
    dev_in = [t.to(DEV) for t in cpu_inputs]
    res = mccl.reduce_n(dev_in, out=out, op=op, variant=variant)
    torch.cuda.synchronize()
    return res


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
@pytest.mark.parametrize("opname", list(OPS))
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_reduce_all_dtypes_ops(mccl, dtype, opname, n):
    count = 5000  # not a multiple of the vector width: head/tail paths run
    scale = 1.0 if opname == "prod" else 0.02
    ins = [rank_buffer(count, dtype, r, scale=scale) for r in range(n)]
    for variant in (1, 2, 3):
        got = _run(mccl, ins, OPS[opname], variant)
        assert_bits_equal(bits(got), oracle_reduce_bits(ins, OPS[opname]),
                          "%s %s n=%d variant=%d" % (dtype, opname, n, variant))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int32], ids=str)
@pytest.mark.parametrize("n", [2, 4, 5, 7, 8, 16, 64])
@pytest.mark.parametrize("count", [0, 1, 7, 8, 9, 63, 64, 511, 512, 513, 4096 + 3, 131072, 1_000_003])
def test_reduce_sum_counts_and_ranks(mccl, dtype, n, count):
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    got = _run(mccl, ins, O.SUM)
    if count == 0:
        assert got.numel() == 0
        return
    assert_bits_equal(bits(got), oracle_reduce_bits(ins), "%s n=%d count=%d" % (dtype, n, count))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.uint8, torch.float64], ids=str)
@pytest.mark.parametrize("shift", [1, 3, 5, 8])
def test_reduce_shifted_congruent(mccl, dtype, shift):
    """All buffers start `shift` elements past a 16-byte boundary: the head is peeled."""
    n, count = 4, 10007
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    dev = []
    for t in ins:
        base = torch.zeros(count + 64, dtype=dtype, device=DEV)
        view = base[shift:shift + count]
        view.copy_(t)
        dev.append(view)
    outbase = torch.zeros(count + 64, dtype=dtype, device=DEV)
    out = outbase[shift:shift + count]
    mccl.reduce_n(dev, out=out, op=O.SUM)
    torch.cuda.synchronize()
    assert_bits_equal(bits(out), oracle_reduce_bits(ins), "shift=%d" % shift)
    # canaries: nothing outside the view was written
    assert int(outbase[:shift].abs().sum()) == 0 and int(outbase[shift + count:].abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int8], ids=str)
def test_reduce_incongruent_alignment(mccl, dtype):
    """Each buffer has a different offset mod 16 bytes: the element-wise kernel runs."""
    n, count = 5, 9001
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    dev = []
    for r, t in enumerate(ins):
        base = torch.zeros(count + 64, dtype=dtype, device=DEV)
        view = base[r + 1:r + 1 + count]
        view.copy_(t)
        dev.append(view)
    out = torch.zeros(count + 64, dtype=dtype, device=DEV)
    mccl.reduce_n(dev, out=out[:count], op=O.SUM)
    torch.cuda.synchronize()
    assert_bits_equal(bits(out[:count]), oracle_reduce_bits(ins), "incongruent")
    assert int(out[count:].abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("which", [0, 3, 7])
def test_reduce_in_place(mccl, dtype, which):
    """The allreduce of the reference is in place: out aliases one of the inputs."""
    n, count = 8, 70001
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    want = oracle_reduce_bits(ins)
    for variant in (1, 2, 3):
        dev = [t.to(DEV) for t in ins]
        mccl.reduce_n(dev, out=dev[which], op=O.SUM, variant=variant)
        torch.cuda.synchronize()
        assert_bits_equal(bits(dev[which]), want, "in place on %d variant %d" % (which, variant))
        for r in range(n):
            if r != which:
                assert_bits_equal(bits(dev[r]), bits(ins[r]), "input %d untouched" % r)


def _special_values(dtype):
    """+-0, subnormals, +-inf, max-finite cancellation, rounding ties, and NaNs: quiet and
    signalling, both signs, with and without payload."""
    if dtype == torch.bfloat16:
        pats = [0x0000, 0x8000, 0x0001, 0x8001, 0x007f, 0x0080, 0x7f7f, 0xff7f, 0x7f80, 0xff80,
                0x3f80, 0xbf80, 0x3f81, 0x3c00, 0x3b80, 0x4000, 0x0100, 0x8100,
                0x7fc0, 0xffc0, 0x7f81, 0xff81, 0x7fc5]
        return torch.tensor(np.array(pats, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)
    if dtype == torch.float16:
        pats = [0x0000, 0x8000, 0x0001, 0x8001, 0x03ff, 0x0400, 0x7bff, 0xfbff, 0x7c00, 0xfc00,
                0x3c00, 0xbc00, 0x3c01, 0x1400, 0x1000, 0x4000, 0x0002, 0x8002,
                0x7e00, 0xfe00, 0x7c01, 0xfc01, 0x7e05]
        return torch.tensor(np.array(pats, dtype=np.uint16).view(np.int16)).view(torch.float16)
    pats = [0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007fffff, 0x00800000, 0x7f7fffff,
            0xff7fffff, 0x7f800000, 0xff800000, 0x3f800000, 0xbf800000, 0x3f800001, 0x33800000,
            0x33000000, 0x40000000, 0x00000002, 0x80000002,
            0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001, 0x7fc12345]
    return torch.tensor(np.array(pats, dtype=np.uint32).view(np.int32)).view(torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("opname", ["sum", "prod", "min", "max"])
def test_reduce_special_values(mccl, dtype, opname):
    """Every ordered triple of special values (signed zeros, subnormals, infinities, ties, NaNs of
    every kind in every rank position).  MIN / MAX select, so their fp32 results are compared bit
    for bit, NaN included (the highest rank's NaN, bits untouched); NaN results of fp32 arithmetic
    (SUM, PROD) are compared as "is NaN" (their payloads are not part of the contract); f16 / bf16
    NaNs are canonical in both implementations and compared bit for bit."""
    v = _special_values(dtype)
    k = v.numel()
    a = v.repeat_interleave(k * k)
    b = v.repeat_interleave(k).repeat(k)
    c = v.repeat(k * k)
    ins = [a.contiguous(), b.contiguous(), c.contiguous()]
    got = bits(_run(mccl, ins, OPS[opname]))
    want = oracle_reduce_bits(ins, OPS[opname])
    if dtype == torch.float32 and opname in ("sum", "prod"):
        gf, wf = got.view(np.float32), want.view(np.float32)
        nan_g, nan_w = np.isnan(gf), np.isnan(wf)
        assert np.array_equal(nan_g, nan_w)
        assert_bits_equal(got[~nan_w], want[~nan_w], "%s %s" % (dtype, opname))
    else:
        assert_bits_equal(got, want, "%s %s" % (dtype, opname))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
def test_reduce_nan_inputs(mccl, dtype):
    """NaN in any rank makes the SUM NaN; f16/bf16 produce the canonical quiet NaN."""
    n, count = 4, 1024
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    ins[2][5] = float("nan")
    ins[0][100] = float("inf")
    ins[3][100] = float("-inf")
    got = _run(mccl, ins, O.SUM)
    assert torch.isnan(got[5]) and torch.isnan(got[100])
    want = oracle_reduce_bits(ins)
    if dtype != torch.float32:
        assert_bits_equal(bits(got), want, "nan canonical")


@pytest.mark.parametrize("dtype", FLOAT_DTYPES, ids=str)
@pytest.mark.parametrize("n,count", [(2, 4099), (3, 4099), (4, 70_001), (8, 4099), (16, 1000), (8, 9 * (1 << 20) + 5)])
def test_reduce_avg(mccl, dtype, n, count):
    """AVG = SUM chain, then one division by n in the accumulation type; compile-time rank counts
    (2, 4, 8), the generic path, and a size whose output is written with streaming stores."""
    ins = [rank_buffer(count, dtype, r) for r in range(n)]
    got = _run(mccl, ins, mccl.AVG)
    assert_bits_equal(bits(got), oracle_reduce_bits(ins, O.AVG), "avg %s n=%d vs the oracle" % (dtype, n))
    # second witness: the same order of operations in torch on the CPU
    acc_t = torch.float64 if dtype == torch.float64 else torch.float32
    acc = torch.zeros(count, dtype=acc_t)
    for t in ins:
        acc = acc + t.to(acc_t)
    want = (acc / n).to(dtype)
    assert_bits_equal(bits(got), bits(want), "avg %s n=%d" % (dtype, n))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
def test_reduce_avg_special_values(mccl, dtype):
    """AVG over every ordered triple of special values, against the oracle (NaN results of fp32
    arithmetic compared as "is NaN")."""
    v = _special_values(dtype)
    k = v.numel()
    ins = [v.repeat_interleave(k * k).contiguous(), v.repeat_interleave(k).repeat(k).contiguous(), v.repeat(k * k).contiguous()]
    got = bits(_run(mccl, ins, mccl.AVG))
    want = oracle_reduce_bits(ins, O.AVG)
    if dtype == torch.float32:
        nan_g, nan_w = np.isnan(got.view(np.float32)), np.isnan(want.view(np.float32))
        assert np.array_equal(nan_g, nan_w)
        assert_bits_equal(got[~nan_w], want[~nan_w], "avg %s" % dtype)
    else:
        assert_bits_equal(got, want, "avg %s" % dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64], ids=str)
@pytest.mark.parametrize("opname", ["min", "max"])
@pytest.mark.parametrize("n", [2, 3, 8])
def test_min_max_propagate_nan_from_any_rank(mccl, dtype, opname, n):
    """A NaN in any one rank (or in several) makes MIN / MAX NaN: specialised and generic rank
    counts, every launch shape, bit for bit against the oracle."""
    count = 70_001
    for pos in range(n):
        ins = [rank_buffer(count, dtype, r, scale=1.0) for r in range(n)]
        ins[pos][::7] = float("nan")
        ins[(pos + 1) % n][3::11] = -float("nan")
        for variant in (1, 2, 3):  # small, persistent, stream
            got = _run(mccl, ins, OPS[opname], variant=variant)
            assert torch.isnan(got[0]) and torch.isnan(got[7]) and torch.isnan(got[3])
            assert_bits_equal(bits(got), oracle_reduce_bits(ins, OPS[opname]), "%s %s n=%d nan in rank %d" % (dtype, opname, n, pos))


def test_reduce_avg_rejects_integers(mccl):
    t = [torch.ones(8, dtype=torch.int32, device=DEV) for _ in range(2)]
    with pytest.raises(RuntimeError, match="AVG"):
        mccl.reduce_n(t, op=mccl.AVG)


# ---- configs of the headline benchmark, at sizes the oracle finishes in seconds ----

def test_config1_fp32_two_ranks_16mib(mccl):
    """all_reduce SUM fp32, 2 ranks x 4,194,304 elements, uniform[-1,1): bit-exact
    (a two-operand IEEE add has a single possible value)."""
    count = 4_194_304
    ins = [rank_buffer(count, torch.float32, r, dist="uniform") for r in range(2)]
    got = _run(mccl, ins, O.SUM)
    assert_bits_equal(bits(got), bits(ins[0] + ins[1]), "C1 vs torch fp32 add")
    assert_bits_equal(bits(got), oracle_reduce_bits(ins), "C1 vs oracle")


@pytest.mark.parametrize("variant", [1, 2, 3])
def test_config2_bf16_decode_256k(mccl, variant):
    """bf16 [16 x 8192] per rank, 8 ranks, N(0, 0.02), fp32 accumulation."""
    ins = [rank_buffer(16 * 8192, torch.bfloat16, r) for r in range(8)]
    got = _run(mccl, ins, O.SUM, variant)
    assert_bits_equal(bits(got), oracle_reduce_bits(ins), "C2 variant %d" % variant)


def test_config3_bf16_prefill_64mib(mccl):
    """bf16 [4096 x 8192] per rank, 8 ranks: full size, checked against the oracle (OpenMP)
    and against an on-device fp32 chain built from torch ops."""
    count = 4096 * 8192
    ins = [rank_buffer(count, torch.bfloat16, r) for r in range(8)]
    dev = [t.to(DEV) for t in ins]
    acc = torch.zeros(count, dtype=torch.float32, device=DEV)
    for t in dev:
        acc += t.float()
    chain = acc.to(torch.bfloat16).view(torch.int16)
    for variant in (0, 2, 3):
        got = mccl.reduce_n(dev, op=O.SUM, variant=variant)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), chain), "variant %d" % variant
    O.set_threads(min(16, O.max_threads()))
    try:
        want = oracle_reduce_bits(ins)
    finally:
        O.set_threads(1)
    assert_bits_equal(bits(got), want, "C3")


# ---- reduce_scatter ----

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int64], ids=str)
@pytest.mark.parametrize("n,m", [(2, 1), (4, 1000), (8, 65536 + 5), (3, 33)])
def test_reduce_scatter_all_shards(mccl, dtype, n, m):
    ins = [rank_buffer(n * m, dtype, r) for r in range(n)]
    dev = [t.to(DEV) for t in ins]
    outs = [torch.empty(m, dtype=dtype, device=DEV) for _ in range(n)]
    mccl.reduce_scatter_n(dev, outs, op=O.SUM)
    torch.cuda.synchronize()
    code = TORCH_TO_CODE[dtype]
    want = O.reduce_scatter([to_carrier(t) for t in ins], code, O.SUM)
    for s in range(n):
        assert_bits_equal(bits(outs[s]), want[s].view(bits(outs[s]).dtype), "shard %d" % s)
    # one shard at a time (what a single rank does) gives the same answer
    for s in range(n):
        o = torch.empty(m, dtype=dtype, device=DEV)
        mccl.reduce_scatter_n(dev, [o], op=O.SUM, shard_first=s)
        torch.cuda.synchronize()
        assert_bits_equal(bits(o), bits(outs[s]), "single shard %d" % s)


def test_reduce_scatter_matches_allreduce_slices(mccl):
    """Shard s of reduce_scatter == slice s of the allreduce of the same buffers."""
    n, m = 8, 12345
    ins = [rank_buffer(n * m, torch.bfloat16, r) for r in range(n)]
    dev = [t.to(DEV) for t in ins]
    full = mccl.reduce_n(dev, op=O.SUM)
    outs = [torch.empty(m, dtype=torch.bfloat16, device=DEV) for _ in range(n)]
    mccl.reduce_scatter_n(dev, outs, op=O.SUM)
    torch.cuda.synchronize()
    for s in range(n):
        assert_bits_equal(bits(outs[s]), bits(full[s * m:(s + 1) * m]), "shard %d" % s)


def test_reduce_multi_coalesced(mccl):
    """allreduce_coalesced: 5 buckets full((5+i,), rank+1+i) -> W*(i+(W+1)/2)
    (closed form of the reference's test_allreduce_coalesced_basics), one launch group."""
    for W in (2, 4, 8):
        ins = [[torch.full((5 + i,), float(r + 1 + i), device=DEV) for r in range(W)] for i in range(5)]
        outs = [torch.empty(5 + i, device=DEV) for i in range(5)]
        mccl.reduce_multi(ins, outs, op=O.SUM)
        torch.cuda.synchronize()
        for i, o in enumerate(outs):
            assert torch.equal(o.cpu(), torch.full((5 + i,), W * (i + (W + 1.0) / 2.0)))


def test_reduce_multi_random(mccl):
    n = 8
    counts = [1, 17, 4096, 100003, 0, 777]
    ins_cpu = [[rank_buffer(c, torch.bfloat16, r, seed=77 + b) for r in range(n)] for b, c in enumerate(counts)]
    ins = [[t.to(DEV) for t in lst] for lst in ins_cpu]
    outs = [torch.empty(c, dtype=torch.bfloat16, device=DEV) for c in counts]
    mccl.reduce_multi(ins, outs, op=O.SUM)
    torch.cuda.synchronize()
    for b, c in enumerate(counts):
        if c:
            assert_bits_equal(bits(outs[b]), oracle_reduce_bits(ins_cpu[b]), "bucket %d" % b)


# ---- HIP graph capture: the entry points allocate nothing and never synchronise ----

def test_reduce_and_copy_replay_from_a_hip_graph(mccl):
    """Capture one reduction and one allgather into a graph; replay it several times with eager
    work and synchronisations in between; every replay must equal the eager result."""
    n, count = 8, 16 * 8192
    ins = [rank_buffer(count, torch.bfloat16, r).to(DEV) for r in range(n)]
    out = torch.zeros(count, dtype=torch.bfloat16, device=DEV)
    gathered = torch.zeros(n * count, dtype=torch.bfloat16, device=DEV)
    mccl.reduce_n(ins, out=out)          # warm-up outside the capture (device facts are cached)
    mccl.allgather_n(ins, gathered)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        mccl.reduce_n(ins, out=out)
        mccl.allgather_n(ins, gathered)
    for it in range(4):
        for r in range(n):               # eager work between replays: new inputs every time
            ins[r].copy_(rank_buffer(count, torch.bfloat16, r, seed=500 + it))
        out.zero_()
        gathered.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = mccl.reduce_n(ins)        # eager result on the same inputs
        torch.cuda.synchronize()
        assert_bits_equal(bits(out), bits(want), "graph replay %d" % it)
        assert_bits_equal(bits(out), oracle_reduce_bits([t.cpu() for t in ins]), "graph replay %d vs oracle" % it)
        assert_bits_equal(bits(gathered), np.concatenate([bits(t) for t in ins]), "graph allgather %d" % it)


# ---- 64-bit indexing ----

def test_reduce_more_than_4gib_per_buffer(mccl):
    """Two u8 buffers of 2^32 + 1000 elements: element indices and byte offsets exceed 32 bits.
    Inputs are periodic patterns built on the device; the result is checked with torch ops."""
    count = (1 << 32) + 1000
    a = torch.arange(251, dtype=torch.uint8, device=DEV).repeat(count // 251 + 1)[:count]
    b = torch.arange(241, dtype=torch.uint8, device=DEV).repeat(count // 241 + 1)[:count]
    out = mccl.reduce_n([a, b], op=O.SUM)
    torch.cuda.synchronize()
    for lo in (0, (1 << 31) - 5000, (1 << 32) - 5000, count - 9000):
        sl = slice(lo, lo + 9000)
        assert torch.equal(out[sl], a[sl] + b[sl]), "slice at %d" % lo
    # a checksum over everything (uint8 wrap-around sums, reduced in int64)
    assert int(out.sum(dtype=torch.int64)) == int((a + b).sum(dtype=torch.int64))


def test_reduce_scatter_offsets_beyond_4gib(mccl):
    """Shard offsets larger than 4 GiB: 6 shards of 1 GiB (bf16) per rank, 2 ranks; the last
    shard starts 5 GiB into each buffer."""
    n_shards, m = 6, 1 << 29
    ins = []
    for r in range(2):
        g = torch.Generator(device=DEV).manual_seed(1234 * 1_000_003 + r)
        x = torch.empty(n_shards * m, dtype=torch.bfloat16, device=DEV)
        for s in range(n_shards):
            x[s * m:(s + 1) * m] = (torch.randn(m, generator=g, device=DEV) * 1e-3).to(torch.bfloat16)
        ins.append(x)
    out = torch.empty(m, dtype=torch.bfloat16, device=DEV)
    for shard in (0, 5):
        mccl.reduce_scatter_n(ins, [out], op=O.SUM, shard_first=shard)
        torch.cuda.synchronize()
        sl = slice(shard * m, (shard + 1) * m)
        want = (ins[0][sl].float() + ins[1][sl].float()).to(torch.bfloat16)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), "shard %d" % shard


# ---- re-entrancy ----

def test_concurrent_callers_on_their_own_streams(mccl):
    """The entry points are re-entrant: four host threads, each on a stream of its own, run
    reductions and copies of different shapes at the same time; every result matches the oracle."""
    import threading

    shapes = [(8, 131072, torch.bfloat16), (3, 1_000_003, torch.float32), (2, 4_194_304, torch.float16), (5, 77_777, torch.int32)]
    errors = []

    def worker(idx):
        try:
            n, count, dtype = shapes[idx]
            cpu = [rank_buffer(count, dtype, 10 * idx + r) for r in range(n)]
            want = oracle_reduce_bits(cpu)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                dev = [t.to(DEV) for t in cpu]
                out = torch.empty(count, dtype=dtype, device=DEV)
                gathered = torch.empty(n * count, dtype=dtype, device=DEV)
                for it in range(25):
                    out.zero_()
                    mccl.reduce_n(dev, out=out, op=O.SUM, variant=it % 4)
                    mccl.allgather_n(dev, gathered)
                    stream.synchronize()
                    assert_bits_equal(bits(out), want, "thread %d iteration %d" % (idx, it))
                assert_bits_equal(bits(gathered), np.concatenate([bits(t) for t in cpu]), "thread %d allgather" % idx)
        except BaseException as e:  # surfaced in the main thread
            errors.append((idx, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


# ---- large launches write their output with streaming stores: every dtype through that path ----

@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
def test_reduce_streamed_output_all_dtypes(mccl, dtype):
    """Two ranks, a little over 5 MiB per rank (beyond the size up to which outputs stay cacheable),
    odd element count so that the peeled tail runs as well; all three launch shapes."""
    es = torch.empty(0, dtype=dtype).element_size()
    count = (5 << 20) // es + 3
    ins = [rank_buffer(count, dtype, r) for r in range(2)]
    want = oracle_reduce_bits(ins)
    for variant in (0, 1, 2, 3):
        got = _run(mccl, ins, O.SUM, variant)
        assert_bits_equal(bits(got), want, "%s variant %d" % (dtype, variant))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float64], ids=str)
@pytest.mark.parametrize("opname", ["sum", "max"])
def test_reduce_eight_ranks_beyond_the_stream_threshold(mccl, dtype, opname):
    """8 ranks x 16 MiB (144 MiB per launch: the stream shape with its streaming stores), for the
    compile-time rank count (sum) and the generic path (max)."""
    es = torch.empty(0, dtype=dtype).element_size()
    count = (16 << 20) // es
    ins = [rank_buffer(count, dtype, r) for r in range(8)]
    O.set_threads(min(16, O.max_threads()))
    try:
        want = oracle_reduce_bits(ins, OPS[opname])
    finally:
        O.set_threads(1)
    got = _run(mccl, ins, OPS[opname])
    assert_bits_equal(bits(got), want, "%s %s" % (dtype, opname))


# ---- seeded fuzz over every parameter at once ----

@pytest.mark.parametrize("seed", range(6))
def test_reduce_random_combinations(mccl, seed):
    """25 random combinations per seed of dtype, op, rank count (1..20), element count, launch shape
    and independent element offsets of every input and of the output inside padded buffers (so
    that heads, tails, unaligned inputs and canaries all come into play together)."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(25):
        dtype = ALL_DTYPES[int(rng.integers(0, len(ALL_DTYPES)))]
        opname = ["sum", "prod", "min", "max"][int(rng.integers(0, 4))]
        n = int(rng.integers(1, 21))
        count = int(rng.choice([1, 7, 63, 64, 65, 1000, 4097, 70_001, 300_003]))
        variant = int(rng.integers(0, 4))
        pad = 80
        offs = [int(rng.integers(0, pad)) for _ in range(n + 1)]
        scale = 1.0 if opname == "prod" else 0.02
        cpu = [rank_buffer(count, dtype, 100 * case + r, scale=scale) for r in range(n)]
        dev = []
        for r in range(n):
            buf = torch.zeros(count + pad, dtype=dtype, device=DEV)
            buf[offs[r]:offs[r] + count] = cpu[r].to(DEV)
            dev.append(buf[offs[r]:offs[r] + count])
        canary = rank_buffer(count + pad, dtype, 999, scale=scale).to(DEV)
        out_buf = canary.clone()
        out = out_buf[offs[n]:offs[n] + count]
        mccl.reduce_n(dev, out=out, op=OPS[opname], variant=variant)
        torch.cuda.synchronize()
        what = "seed %d case %d: %s %s n=%d count=%d variant=%d offsets=%s" % (seed, case, dtype, opname, n, count, variant, offs)
        assert_bits_equal(bits(out), oracle_reduce_bits(cpu, OPS[opname]), what)
        assert_bits_equal(bits(out_buf[:offs[n]]), bits(canary[:offs[n]]), what + " (bytes before the output)")
        assert_bits_equal(bits(out_buf[offs[n] + count:]), bits(canary[offs[n] + count:]), what + " (bytes after the output)")
