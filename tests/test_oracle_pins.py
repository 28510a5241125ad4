"""Pins for what the reference's tests leave open in the oracle: conversions against library
routines (numpy float16, torch bfloat16), rounding-order known answers chosen so that a
plausible mistake (wrong order, per-step rounding, dropped rank, non-zero start) fails,
and index maps against brute-force Python loops on tagged tiny inputs."""
import numpy as np
import pytest
import torch

from oracle import oracle as O


# ---------------- conversions ----------------

def _float_patterns(rng, n):
    """fp32 bit patterns: uniform random bits plus every exponent crossed with edge mantissas."""
    rnd = rng.integers(0, 2 ** 32, size=n, dtype=np.uint64).astype(np.uint32)
    exps = np.arange(256, dtype=np.uint32) << 23
    mans = np.array([0, 1, 0xfff, 0x1000, 0x1001, 0x1fff, 0x2000, 0x2001, 0x3000, 0x7fff, 0x8000, 0x8001,
                     0xffff, 0x10000, 0x18000, 0x3fffff, 0x400000, 0x7fe000, 0x7ff000, 0x7fffff], dtype=np.uint32)
    edge = (exps[:, None] | mans[None, :]).reshape(-1)
    edge = np.concatenate([edge, edge | np.uint32(0x80000000)])
    return np.concatenate([rnd, edge]).view(np.float32)


def test_f16_to_f32_exhaustive_vs_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = O.f16_to_f32(h).view(np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got.view(np.float32)[nan]).all()


def test_f32_to_f16_vs_numpy():
    x = _float_patterns(np.random.default_rng(1), 4_000_000)
    got = O.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert (got[nan] == 0x7e00).all()  # canonical quiet NaN


def test_f32_to_bf16_vs_torch():
    x = _float_patterns(np.random.default_rng(2), 4_000_000)
    got = O.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert (got[nan] == 0x7fc0).all()
    # and back: widening is exact
    assert np.array_equal(O.bf16_to_f32(got[~nan]).view(np.uint32), got[~nan].astype(np.uint32) << 16)


# ---------------- rounding order and accumulation width ----------------

def test_fp32_sum_is_ascending_rank_order():
    """(((0 + 1e8) + 1) - 1e8) = 0 in fp32, any other order of the three gives 1 or 8."""
    a, b, c = np.float32(1e8), np.float32(1.0), np.float32(-1e8)
    got = O.reduce([np.array([a]), np.array([b]), np.array([c])], O.F32, O.SUM)
    assert got[0] == np.float32(0.0)
    got = O.reduce([np.array([a]), np.array([c]), np.array([b])], O.F32, O.SUM)
    assert got[0] == np.float32(1.0)


def test_fp32_sum_starts_from_positive_zero():
    """result = 0; result += x_r : an all -0 column gives +0 (bit pattern 0), not -0."""
    neg0 = np.array([-0.0], dtype=np.float32)
    for n in (1, 2, 5):
        got = O.reduce([neg0] * n, O.F32, O.SUM)
        assert got.view(np.uint32)[0] == 0
    # MIN/MAX/PRODUCT start from rank 0's value instead
    assert O.reduce([neg0, neg0], O.F32, O.PROD).view(np.uint32)[0] == 0  # (-0)*(-0) = +0
    assert O.reduce([neg0], O.F32, O.MIN).view(np.uint32)[0] == 0x80000000


def test_fp32_two_rank_sum_matches_numpy():
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, 100000).astype(np.float32)
    b = rng.uniform(-1, 1, 100000).astype(np.float32)
    assert np.array_equal(O.reduce([a, b], O.F32, O.SUM).view(np.uint32), (a + b).view(np.uint32))


def test_bf16_accumulates_in_fp32_and_rounds_once():
    """1 + 3 * 2^-9: fp32 accumulation gives 1 + 0.75 ulp -> rounds up to 0x3F81; rounding to
    bf16 after every add would stay at 1.0 (0x3F80)."""
    one = O.f32_to_bf16(np.array([1.0], dtype=np.float32))
    tiny = O.f32_to_bf16(np.array([2.0 ** -9], dtype=np.float32))
    assert O.reduce([one, tiny, tiny, tiny], O.BF16, O.SUM)[0] == 0x3F81
    # tie: 1 + 2 * 2^-9 = 1 + 0.5 ulp -> round to even -> 1.0
    assert O.reduce([one, tiny, tiny], O.BF16, O.SUM)[0] == 0x3F80
    # tie above an odd mantissa rounds up: (1 + ulp) + 0.5 ulp -> 1 + 2 ulp
    odd = np.array([0x3F81], dtype=np.uint16)
    assert O.reduce([odd, tiny, tiny], O.BF16, O.SUM)[0] == 0x3F82


def test_f16_accumulates_in_fp32_and_rounds_once():
    """Same construction for fp16 (ulp at 1.0 is 2^-10): 1 + 3 * 2^-12 -> 0x3C01."""
    one = O.f32_to_f16(np.array([1.0], dtype=np.float32))
    tiny = O.f32_to_f16(np.array([2.0 ** -12], dtype=np.float32))
    assert O.reduce([one, tiny, tiny, tiny], O.F16, O.SUM)[0] == 0x3C01
    assert O.reduce([one, tiny, tiny], O.F16, O.SUM)[0] == 0x3C00
    # overflow to infinity happens only at the final rounding: 60000 + 60000 - 60000 = 60000
    big = O.f32_to_f16(np.array([60000.0], dtype=np.float32))
    nbig = O.f32_to_f16(np.array([-60000.0], dtype=np.float32))
    assert O.reduce([big, big, nbig], O.F16, O.SUM)[0] == big[0]
    assert O.reduce([big, big], O.F16, O.SUM)[0] == 0x7C00


def test_bf16_chain_matches_torch_fp32_chain():
    """An independent restatement with torch CPU ops: fp32 running sum, one cast at the end."""
    rng = np.random.default_rng(4)
    n, count = 8, 50000
    ins = [O.f32_to_bf16((rng.standard_normal(count) * 0.02).astype(np.float32)) for _ in range(n)]
    acc = torch.zeros(count, dtype=torch.float32)
    for x in ins:
        acc = acc + torch.from_numpy(x.view(np.int16).copy()).view(torch.bfloat16).float()
    want = acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.reduce(ins, O.BF16, O.SUM), want)


@pytest.mark.parametrize("dtype,np_t", [(O.U8, np.uint8), (O.I8, np.int8), (O.I16, np.int16),
                                        (O.I32, np.int32), (O.I64, np.int64)])
def test_integer_sum_and_product_wrap(dtype, np_t):
    rng = np.random.default_rng(5)
    info = np.iinfo(np_t)
    ins = [rng.integers(info.min, info.max, size=1000, dtype=np_t, endpoint=True) for _ in range(7)]
    with np.errstate(over="ignore"):
        s = np.zeros(1000, dtype=np_t)
        p = np.ones(1000, dtype=np_t)
        for x in ins[::-1]:  # wrap-around arithmetic is associative and commutative: any order
            s = s + x
            p = p * x
    assert np.array_equal(O.reduce(ins, dtype, O.SUM), s)
    assert np.array_equal(O.reduce(ins, dtype, O.PROD), p)
    assert np.array_equal(O.reduce(ins, dtype, O.MIN), np.minimum.reduce(ins))
    assert np.array_equal(O.reduce(ins, dtype, O.MAX), np.maximum.reduce(ins))


def test_threads_do_not_change_results():
    rng = np.random.default_rng(6)
    ins = [O.f32_to_bf16(rng.standard_normal(300001).astype(np.float32)) for _ in range(8)]
    one = O.reduce(ins, O.BF16, O.SUM)
    O.set_threads(4)
    try:
        four = O.reduce(ins, O.BF16, O.SUM)
    finally:
        O.set_threads(1)
    assert np.array_equal(one, four)


# ---------------- index maps: brute force on tagged inputs ----------------

def test_reduce_scatter_is_sliced_reduce():
    rng = np.random.default_rng(7)
    n, m = 5, 37
    ins = [rng.integers(-1000, 1000, size=n * m).astype(np.int32) for _ in range(n)]
    full = O.reduce(ins, O.I32, O.SUM)
    outs = O.reduce_scatter(ins, O.I32, O.SUM)
    for s in range(n):
        assert np.array_equal(outs[s], full[s * m:(s + 1) * m])
    assert np.array_equal(O.reduce_scatter(ins, O.I32, O.SUM, shard_first=3, shard_num=1)[0], full[3 * m:4 * m])


@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_alltoallv_brute_force(n):
    """Every element is tagged (source rank, row, column); the receive side is rebuilt with
    plain Python loops from the definition: rank d's segment r = rank r's segment d."""
    rng = np.random.default_rng(n)
    row = 3
    S = rng.integers(0, 5, size=(n, n))
    ins = []
    for r in range(n):
        rows = int(S[r].sum())
        ins.append(np.array([[r * 1_000_000 + i * 10 + c for c in range(row)] for i in range(rows)],
                            dtype=np.int32).reshape(-1))
    outs = O.alltoallv(ins, S, row * 4)
    for d in range(n):
        want = []
        for r in range(n):
            start = sum(int(S[r][dd]) for dd in range(d))
            for i in range(start, start + int(S[r][d])):
                want.extend(r * 1_000_000 + i * 10 + c for c in range(row))
        assert outs[d].view(np.int32).tolist() == want


def test_allgather_pack_unpack_brute_force():
    ins = [np.arange(5, dtype=np.int16) + 100 * r for r in range(4)]
    assert O.allgather(ins).view(np.int16).tolist() == [100 * r + i for r in range(4) for i in range(5)]
    parts = [np.arange(k + 1, dtype=np.uint8) + 10 * k for k in range(6)]
    flat = O.pack(parts)
    assert flat.tolist() == [10 * k + i for k in range(6) for i in range(k + 1)]
    back = O.unpack(flat, [k + 1 for k in range(6)])
    assert all(np.array_equal(a, b) for a, b in zip(back, parts))


def test_alltoall_counts_equal_and_empty():
    counts, displs = O.alltoall_counts(4, 48, 12, None)      # equal split: numel / world
    assert counts.tolist() == [12] * 4 and displs.tolist() == [0, 12, 24, 36]
    counts, displs = O.alltoall_counts(3, 60, 10, [1, 0, 9])  # rowLen = 60/10 = 6
    assert counts.tolist() == [6, 0, 54] and displs.tolist() == [0, 6, 6]
    counts, displs = O.alltoall_counts(3, 0, 0, [0, 0, 0])    # empty tensor: no division
    assert counts.tolist() == [0, 0, 0]


# ---------------- MoE steps: brute force and closed forms ----------------

def test_gather_and_dispatch_brute_force():
    from moe_helpers import route
    n, tokens, topk, n_exp, row = 4, 9, 2, 8, 3
    S, send_tok, send_exp = route(n, tokens, n_exp, topk)
    hidden = [np.array([[r * 10000 + t * 10 + c for c in range(row)] for t in range(tokens)], dtype=np.int32)
              for r in range(n)]
    outs = O.moe_dispatch(hidden, [t.numpy() for t in send_tok], S, row * 4)
    per_rank = n_exp // n
    for d in range(n):
        want = []
        for r in range(n):  # plain loops from the definition: rows for experts owned by d, by (expert, token)
            pairs = sorted((int(e), int(t)) for t, e in zip(send_tok[r].tolist(), send_exp[r].tolist())
                           if e // per_rank == d)
            for e, t in pairs:
                want.extend(r * 10000 + t * 10 + c for c in range(row))
        assert outs[d].view(np.int32).tolist() == want
    g = O.gather_rows(hidden[1], [5, 0, 5, 8], row * 4).view(np.int32).reshape(4, row)
    assert g.tolist() == [hidden[1][5].tolist(), hidden[1][0].tolist(), hidden[1][5].tolist(), hidden[1][8].tolist()]


def test_combine_closed_forms():
    """One-hot weights return the selected row; weights 0.5/0.25/0.25 on rows 8, 4, 4 give 6;
    the chain is fp32 with a rounded product: (2^-9 * 1) three times on top of 1.0 rounds up."""
    x0 = O.f32_to_bf16(np.array([[8.0, 1.0], [4.0, 2.0 ** -9]], dtype=np.float32)).reshape(-1)
    x1 = O.f32_to_bf16(np.array([[4.0, 2.0 ** -9]], dtype=np.float32)).reshape(-1)
    sr = np.array([[0, 0, 1]], dtype=np.int32)
    so = np.array([[0, 1, 0]], dtype=np.int64)
    y = O.moe_combine([x0, x1], sr, so, np.array([[1.0, 0.0, 0.0]], dtype=np.float32), 1, 3, 2, O.BF16)
    assert O.bf16_to_f32(y).tolist() == [8.0, 1.0]
    y = O.moe_combine([x0, x1], sr, so, np.array([[0.5, 0.25, 0.25]], dtype=np.float32), 1, 3, 2, O.BF16)
    assert O.bf16_to_f32(y)[0] == 6.0
    # column 1: 1*1.0 + 1*2^-9 + 1*2^-9 = 1 + 2^-8: a tie in bf16 -> stays 1.0 (even)
    y = O.moe_combine([x0, x1], sr, so, np.array([[1.0, 1.0, 1.0]], dtype=np.float32), 1, 3, 2, O.BF16)
    assert y[1] == 0x3F80
    # with weight 1.5 on the two small terms: 1 + 3*2^-9 -> rounds up (fp32 accumulation, one rounding)
    y = O.moe_combine([x0, x1], sr, so, np.array([[1.0, 1.5, 1.5]], dtype=np.float32), 1, 3, 2, O.BF16)
    assert y[1] == 0x3F81
    # out-of-range entries contribute nothing
    y = O.moe_combine([x0, x1], np.array([[0, 5, 1]], dtype=np.int32), np.array([[0, 0, 9]], dtype=np.int64),
                      np.array([[1.0, 1.0, 1.0]], dtype=np.float32), 1, 3, 2, O.BF16)
    assert O.bf16_to_f32(y).tolist() == [8.0, 1.0]


def test_combine_matches_torch_fp32():
    rng = np.random.default_rng(12)
    n, rows, hidden, tokens, topk = 3, 20, 16, 11, 4
    x = [O.f32_to_bf16(rng.standard_normal((rows, hidden)).astype(np.float32)).reshape(-1) for _ in range(n)]
    sr = rng.integers(0, n, size=(tokens, topk)).astype(np.int32)
    so = rng.integers(0, rows, size=(tokens, topk)).astype(np.int64)
    w = rng.random((tokens, topk)).astype(np.float32)
    y = O.moe_combine(x, sr, so, w, tokens, topk, hidden, O.BF16)
    xs = [torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).view(rows, hidden).float() for a in x]
    acc = torch.zeros(tokens, hidden)
    for k in range(topk):
        rows_k = torch.stack([xs[sr[t, k]][so[t, k]] for t in range(tokens)])
        acc = acc + torch.from_numpy(w[:, k:k + 1]) * rows_k
    want = acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).reshape(-1)
    assert np.array_equal(y, want)


# ---------------- AVG: where the division and the roundings sit ----------------

def _rne(x, mant_bits, emin):
    """Exact rational -> nearest value with `mant_bits` fraction bits (ties to even, gradual
    underflow below 2**emin); overflow is not needed here.  Pure integer / Fraction arithmetic."""
    from fractions import Fraction
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = 0
    while Fraction(2) ** (e + 1) <= x:
        e += 1
    while Fraction(2) ** e > x:
        e -= 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - mant_bits)
    q, r = divmod(x, ulp)
    if r * 2 > ulp or (r * 2 == ulp and q % 2 == 1):
        q += 1
    return sign * q * ulp


def _f32(x):
    return _rne(x, 23, -126)


def _bf16(x):
    return _rne(x, 7, -126)


def _bf16_bits(x):
    """Bit pattern of an exactly representable bf16 value."""
    return int(np.array([float(x)], dtype=np.float32).view(np.uint32)[0] >> 16)


def _avg_orders(xs):
    """The defined result and three plausible wrong ones, all in exact arithmetic:
    right  fp32 chain in rank order, ONE division in fp32, one rounding to bf16
    a      the sum is rounded to bf16 before the division
    b      every input is divided first, the quotients are summed
    c      the sum is multiplied by the rounded reciprocal instead of divided"""
    from fractions import Fraction
    n = len(xs)
    s = Fraction(0)
    for x in xs:
        s = _f32(s + x)
    right = _bf16(_f32(s / n))
    a = _bf16(_f32(_bf16(s) / n))
    sb = Fraction(0)
    for x in xs:
        sb = _f32(sb + _f32(x / n))
    b = _bf16(sb)
    c = _bf16(_f32(s * _f32(Fraction(1, n))))
    return right, a, b, c


def test_avg_is_one_division_of_the_fp32_chain_then_one_rounding():
    """AVG of bf16 inputs against exact rational arithmetic, on vectors picked so that each wrong
    order of divide and round (sum rounded to bf16 first; inputs divided first; multiplication by
    the rounded reciprocal) gives different bits than the defined order, plus random vectors."""
    from fractions import Fraction
    rng = np.random.default_rng(5)
    need = {"a": 3, "b": 3, "c": 3}  # discriminating vectors still wanted per wrong order
    checked = 0
    for trial in range(4000):
        n = int(rng.choice([3, 5, 6, 7]))
        vals = torch.tensor(rng.normal(0, 1, size=n).astype(np.float32) * np.float32(2.0) ** int(rng.integers(-3, 3)))
        vals = vals.to(torch.bfloat16)
        xs = [Fraction(float(v)) for v in vals.float()]
        right, a, b, c = _avg_orders(xs)
        hits = [k for k, w in (("a", a), ("b", b), ("c", c)) if w != right and need[k] > 0]
        if not hits and trial >= 300:
            continue
        for k in hits:
            need[k] -= 1
        carriers = [vals[r:r + 1].view(torch.int16).numpy().view(np.uint16) for r in range(n)]
        got = int(O.reduce(carriers, O.BF16, O.AVG)[0])
        assert got == _bf16_bits(right), (n, [hex(int(c_[0])) for c_ in carriers], hex(got), hex(_bf16_bits(right)))
        checked += 1
    assert all(v == 0 for v in need.values()), need  # every wrong order was told apart at least three times
    assert checked >= 300


def test_avg_fp32_and_fp64_divide_once_in_their_own_type():
    """fp32: (1 + 1 + 1e-8...) style: the chain, then one division; checked against numpy scalars
    of the same type evaluated in the same order, and against the exact-arithmetic model."""
    from fractions import Fraction
    rng = np.random.default_rng(6)
    for n in (2, 3, 7):
        x = rng.normal(0, 1, size=(n, 257)).astype(np.float32)
        got = O.reduce([x[r].copy() for r in range(n)], O.F32, O.AVG)
        for i in range(0, 257, 16):
            s = Fraction(0)
            for r in range(n):
                s = _f32(s + Fraction(float(x[r, i])))
            assert Fraction(float(got[i])) == _f32(s / n), (n, i)
        xd = x.astype(np.float64)
        gd = O.reduce([xd[r].copy() for r in range(n)], O.F64, O.AVG)
        acc = np.zeros(257)
        for r in range(n):
            acc = acc + xd[r]
        assert np.array_equal(gd, acc / n)
    # integers have no AVG
    with pytest.raises(Exception):
        O.reduce([np.ones(4, np.int32), np.ones(4, np.int32)], O.I32, O.AVG)


def test_min_max_propagate_nan_whatever_the_rank_order():
    """A NaN in any rank makes MIN and MAX NaN (torch.min / torch.max semantics); for fp32 the bits
    are those of the highest rank's NaN, quiet or signalling, either sign; bf16 / f16 results are
    the canonical quiet NaN."""
    nans = np.array([0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001, 0x7fc12345], dtype=np.uint32).view(np.float32)
    one = np.array([1.0], dtype=np.float32)
    for op in (O.MIN, O.MAX):
        for k, nan in enumerate(nans):
            v = np.array([nan], dtype=np.float32)
            for order in ([v, one, one], [one, v, one], [one, one, v]):
                got = O.reduce([a.copy() for a in order], O.F32, op)
                assert got.view(np.uint32)[0] == v.view(np.uint32)[0], (op, k)
            other = np.array([nans[(k + 1) % len(nans)]], dtype=np.float32)
            got = O.reduce([v.copy(), one.copy(), other.copy()], O.F32, op)
            assert got.view(np.uint32)[0] == other.view(np.uint32)[0]  # the highest rank's NaN
        for code, qnan, canon, one16 in ((O.BF16, 0x7fc1, 0x7fc0, 0x3f80), (O.F16, 0x7e01, 0x7e00, 0x3c00)):
            for pos in range(3):
                ins = [np.array([one16], dtype=np.uint16) for _ in range(3)]
                ins[pos] = np.array([qnan], dtype=np.uint16)
                assert int(O.reduce(ins, code, op)[0]) == canon
    # and without NaN they are still the minimum / maximum, signed zeros compared as equal
    got = O.reduce([np.array([3.0, -0.0], np.float32), np.array([-2.0, 0.0], np.float32), np.array([5.0, -0.0], np.float32)], O.F32, O.MIN)
    assert got.tolist()[0] == -2.0 and got.view(np.uint32)[1] == 0x80000000  # first of the equal zeros is kept


def test_route_counts_vs_numpy_bincount():
    """oracle_route_counts against numpy's bincount (ids out of range dropped), empty input included."""
    rng = np.random.default_rng(9)
    for n_experts, npairs in ((1, 10), (8, 0), (64, 1000), (256, 32768), (4096, 100000)):
        ids = rng.integers(-3, n_experts + 3, size=npairs).astype(np.int32)
        keep = ids[(ids >= 0) & (ids < n_experts)]
        want = np.bincount(keep, minlength=n_experts).astype(np.int64)
        assert np.array_equal(O.route_counts(ids, n_experts), want)
