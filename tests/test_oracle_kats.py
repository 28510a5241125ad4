"""The CPU oracle against the known-answer cases of the reference's own tests
(tests/golden/c10d_kats.json, closed forms of tests/test_c10d_ccl.py) for world sizes 2..8."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

with open(os.path.join(os.path.dirname(__file__), "golden", "c10d_kats.json")) as f:
    KATS = json.load(f)["world_sizes"]

WORLDS = sorted(int(w) for w in KATS)
OPS = {"SUM": O.SUM, "PRODUCT": O.PROD, "MIN": O.MIN, "MAX": O.MAX}


@pytest.mark.parametrize("W", WORLDS)
@pytest.mark.parametrize("dtype", [O.F32, O.F64, O.BF16, O.F16, O.I32, O.I64])
def test_allreduce_closed_forms(W, dtype):
    case = KATS[str(W)]["allreduce"]
    for opname, want in case["expected"].items():
        if opname == "PRODUCT" and dtype in (O.BF16, O.F16) and W > 5:
            continue  # W! is not representable in 8/11 significand bits beyond 5! = 120
        ins = [_encode(np.array(v, dtype=np.float64), dtype) for v in case["inputs"]]
        got = _decode(O.reduce(ins, dtype, OPS[opname]), dtype)
        assert got.tolist() == want, (W, opname)


@pytest.mark.parametrize("W", WORLDS)
def test_allreduce_coalesced_closed_form(W):
    case = KATS[str(W)]["allreduce_coalesced"]
    for i, want in enumerate(case["expected"]):
        ins = [np.array(case["inputs"][r][i], dtype=np.float32) for r in range(W)]
        assert O.reduce(ins, O.F32, O.SUM).tolist() == want


@pytest.mark.parametrize("W", WORLDS)
def test_reduce_scatter_base_closed_form(W):
    case = KATS[str(W)]["reduce_scatter_base"]
    ins = [np.array(v, dtype=np.float32) for v in case["inputs"]]
    outs = O.reduce_scatter(ins, O.F32, O.SUM)
    assert [o.tolist() for o in outs] == case["expected"]


@pytest.mark.parametrize("W", WORLDS)
def test_reduce_scatter_list_closed_form(W):
    """List form = stack the W tensors of each rank, then the same shard reduction."""
    case = KATS[str(W)]["reduce_scatter_list"]
    ins = [np.concatenate([np.array(t, dtype=np.int64) for t in case["inputs"][r]]) for r in range(W)]
    outs = O.reduce_scatter(ins, O.I64, O.SUM)
    assert [o.tolist() for o in outs] == case["expected"]


@pytest.mark.parametrize("W", WORLDS)
def test_reduce_scatter_variable_closed_form(W):
    """Unequal slots degrade to one reduction per destination rank (slot i of every rank)."""
    case = KATS[str(W)]["reduce_scatter_list_variable"]
    for dest in range(W):
        ins = [np.array(case["inputs"][r][dest], dtype=np.int64) for r in range(W)]
        assert O.reduce(ins, O.I64, O.SUM).tolist() == case["expected"][dest]


@pytest.mark.parametrize("W", WORLDS)
def test_allgather_closed_forms(W):
    case = KATS[str(W)]["allgather_base"]
    out = O.allgather([np.array(v, dtype=np.int64) for v in case["inputs"]]).view(np.int64)
    assert out.tolist() == case["expected"]
    for sub in KATS[str(W)]["allgather_list"]:
        out = O.allgather([np.array(v, dtype=np.int64) for v in sub["inputs"]]).view(np.int64)
        assert [[x] for x in out.tolist()] == sub["expected"]


@pytest.mark.parametrize("W", WORLDS)
def test_alltoall_equal_closed_form(W):
    case = KATS[str(W)]["alltoall_base_equal"]
    ins = [np.array(v, dtype=np.float32) for v in case["inputs"]]
    counts, displs = O.alltoall_counts(W, W * W, W, None)
    assert counts.tolist() == [W] * W and displs.tolist() == [W * i for i in range(W)]
    outs = O.alltoallv(ins, np.ones((W, W), dtype=np.int64), W * 4)
    for d in range(W):
        assert outs[d].view(np.float32).reshape(W, W).tolist() == case["expected"][d]


@pytest.mark.parametrize("W", WORLDS)
def test_alltoall_unequal_closed_form(W):
    case = KATS[str(W)]["alltoall_base_unequal"]
    S = np.array(case["in_splits"], dtype=np.int64)  # S[r][d] = rows r -> d
    assert (S.T == np.array(case["out_splits"])).all()  # rank d's out_splits[r] == rank r's in_splits[d]
    # count arithmetic: rowLen = numel / dim0 = W, sendCounts[i] = in_splits[i] * W
    rows = int(S[0].sum())
    counts, displs = O.alltoall_counts(W, rows * W, rows, S[0])
    assert counts.tolist() == [(i + 1) * W for i in range(W)]
    assert displs.tolist() == [W * sum(range(1, i + 1)) for i in range(W)]
    ins = [np.array(v, dtype=np.float32) for v in case["inputs"]]
    outs = O.alltoallv(ins, S, W * 4)
    for d in range(W):
        assert outs[d].view(np.float32).reshape(-1, W).tolist() == case["expected"][d]


@pytest.mark.parametrize("W", WORLDS)
def test_alltoall_list_closed_form(W):
    """List form = pack the W input tensors, alltoallv, unpack into the W output tensors."""
    case = KATS[str(W)]["alltoall_list"]
    S = np.array([[i + 1 for i in range(W)] for _ in range(W)], dtype=np.int64)
    packed = []
    for r in range(W):
        tensors = [np.array(t, dtype=np.float32) for t in case["inputs"][r]]
        packed.append(O.pack(tensors))
    outs = O.alltoallv(packed, S, W * 4)
    for d in range(W):
        parts = O.unpack(outs[d], [(d + 1) * W * 4] * W)
        for i in range(W):
            assert parts[i].view(np.float32).reshape(-1, W).tolist() == case["expected"][d][i]


@pytest.mark.parametrize("W", WORLDS)
def test_coalescing_identities(W):
    c = KATS[str(W)]["coalesced_allreduce_ones"]
    small = [O.reduce([np.ones(c["size_per_coll"], dtype=np.float32)] * W, O.F32, O.SUM) for _ in range(c["num_colls"])]
    big = O.reduce([np.ones(c["num_colls"] * c["size_per_coll"], dtype=np.float32)] * W, O.F32, O.SUM)
    assert np.concatenate(small).tolist() == big.tolist() == [c["expected_value"]] * big.size
    r = KATS[str(W)]["reduce_scatter_tensor_ones"]
    outs = O.reduce_scatter([np.ones(W * 4, dtype=np.float32)] * W, O.F32, O.SUM)
    assert all(o.tolist() == [r["expected_value"]] * 4 for o in outs)


def _encode(x, dtype):
    if dtype == O.BF16:
        return O.f32_to_bf16(x.astype(np.float32))
    if dtype == O.F16:
        return O.f32_to_f16(x.astype(np.float32))
    return x.astype(O.CARRIER[dtype])


def _decode(x, dtype):
    if dtype == O.BF16:
        return O.bf16_to_f32(x).astype(np.float64)
    if dtype == O.F16:
        return O.f16_to_f32(x).astype(np.float64)
    return x.astype(np.float64)


def test_fixture_matches_its_generator():
    """tests/golden/c10d_kats.json is exactly what tests/golden/make_kat_fixture.py writes."""
    import importlib.util
    here = os.path.dirname(__file__)
    spec = importlib.util.spec_from_file_location("make_kat_fixture", os.path.join(here, "golden", "make_kat_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    with open(os.path.join(here, "golden", "c10d_kats.json")) as f:
        committed = json.load(f)
    assert committed["world_sizes"] == json.loads(json.dumps({str(W): mod.cases_for(W) for W in range(2, 9)}))
    assert committed["p2p"] == json.loads(json.dumps(mod.p2p_cases()))
