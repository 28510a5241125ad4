"""Property-based checks of the oracle's index maps (hypothesis): random split matrices, ragged and
empty segments, arbitrary row lengths.  Each property is checked against an independent formulation
(numpy fancy indexing / concatenation), not against the oracle's own loops."""
import numpy as np
from hypothesis import given, settings, strategies as st

from oracle import oracle as O


@st.composite
def split_case(draw):
    n = draw(st.integers(1, 8))
    row = draw(st.sampled_from([1, 2, 3, 8, 16, 20]))
    S = np.array(draw(st.lists(st.lists(st.integers(0, 6), min_size=n, max_size=n), min_size=n, max_size=n)),
                 dtype=np.int64)
    return n, row, S


@settings(max_examples=150, deadline=None)
@given(split_case())
def test_alltoallv_equals_numpy_slicing(case):
    n, row, S = case
    ins = []
    for r in range(n):
        rows = int(S[r].sum())
        ins.append(np.arange(rows * row, dtype=np.int32) + r * 1_000_000)
    outs = O.alltoallv(ins, S, row * 4)
    offs = np.concatenate([np.zeros((n, 1), dtype=np.int64), np.cumsum(S, axis=1)], axis=1)  # send displacements
    for d in range(n):
        want = np.concatenate([ins[r].reshape(-1, row)[offs[r, d]:offs[r, d + 1]].reshape(-1) for r in range(n)]
                              or [np.zeros(0, dtype=np.int32)])
        assert outs[d].view(np.int32).tolist() == want.tolist()
    # conservation: every sent element arrives exactly once
    sent = np.sort(np.concatenate(ins)) if n else np.zeros(0)
    got = np.sort(np.concatenate([o.view(np.int32) for o in outs]))
    assert np.array_equal(sent, got)


@settings(max_examples=100, deadline=None)
@given(st.lists(st.integers(0, 40), min_size=1, max_size=12))
def test_pack_unpack_are_inverse_and_match_concatenate(sizes):
    rng = np.random.default_rng(sum(sizes) + len(sizes))
    parts = [rng.integers(0, 256, size=s, dtype=np.uint8) for s in sizes]
    flat = O.pack(parts)
    assert np.array_equal(flat, np.concatenate(parts))
    back = O.unpack(flat, sizes)
    assert all(np.array_equal(a, b) for a, b in zip(back, parts))


@settings(max_examples=100, deadline=None)
@given(st.integers(1, 8), st.integers(0, 50), st.sampled_from([O.I32, O.F32, O.BF16]))
def test_reduce_scatter_and_allgather_compose_to_allreduce(n, m, dtype):
    """allgather(reduce_scatter(x)) == allreduce(x): shards are disjoint and in rank order."""
    rng = np.random.default_rng(n * 100 + m)
    lim = 15 if dtype == O.BF16 else 50  # bf16 holds integers exactly only up to 256
    raw = [rng.integers(-lim, lim, size=n * m) for _ in range(n)]
    if dtype == O.I32:
        ins = [r.astype(np.int32) for r in raw]
    elif dtype == O.F32:
        ins = [r.astype(np.float32) for r in raw]
    else:
        ins = [O.f32_to_bf16(r.astype(np.float32)) for r in raw]
    full = O.reduce(ins, dtype, O.SUM)
    shards = O.reduce_scatter(ins, dtype, O.SUM)
    if m:
        gathered = O.allgather(shards).view(full.dtype)
        assert np.array_equal(gathered, full)
    # small integers are exact in every dtype: the sum equals numpy's integer sum
    want = np.sum(raw, axis=0)
    got = O.bf16_to_f32(full) if dtype == O.BF16 else full.astype(np.float64)
    assert np.array_equal(np.asarray(got, dtype=np.float64), want.astype(np.float64))


@settings(max_examples=100, deadline=None)
@given(st.integers(1, 8), st.integers(1, 30), st.lists(st.integers(0, 9), min_size=1, max_size=8))
def test_alltoall_counts_are_prefix_sums(world, row_len, splits):
    splits = (splits * world)[:world]
    dim0 = sum(splits)
    counts, displs = O.alltoall_counts(world, dim0 * row_len, dim0, splits)
    if dim0:
        assert counts.tolist() == [s * row_len for s in splits]
    assert displs.tolist() == [int(x) for x in np.concatenate([[0], np.cumsum(counts)[:-1]])]
