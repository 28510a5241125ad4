"""Writes tests/golden/c10d_kats.json: the known-answer cases of the reference's own functional
tests (tests/test_c10d_ccl.py), instantiated for world sizes 2..8.

The reference's tests state their expectations as closed forms in the world size W and the
rank; this script evaluates exactly those closed forms (cited per case) into plain
input/expected-output vectors.  Nothing of the reference is imported or run, and the oracle
is not used: the expectations come from the reference's formulas, so they pin the oracle
rather than restate it.
"""
import json
import math
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def cases_for(W):
    c = {}
    # simple_reduce_tests, tests/test_c10d_ccl.py:70-93: every rank contributes [rank + 1.0]
    inputs = [[r + 1.0] for r in range(W)]
    c["allreduce"] = {
        "inputs": inputs,
        "expected": {"SUM": [W * (W + 1) / 2.0], "PRODUCT": [float(math.factorial(W))],
                     "MIN": [1.0], "MAX": [float(W)]},
    }
    # allreduce_coalesced, :200-209: tensor i of rank r = full((5+i,), r+1+i) -> W*(i+(W+1)/2)
    c["allreduce_coalesced"] = {
        "inputs": [[[float(r + 1 + i)] * (5 + i) for i in range(5)] for r in range(W)],
        "expected": [[W * (i + (W + 1.0) / 2.0)] * (5 + i) for i in range(5)],
    }
    # _reduce_scatter_base, :550-566: every rank's input arange(W) -> rank r receives r*W
    c["reduce_scatter_base"] = {
        "inputs": [[float(j) for j in range(W)] for _ in range(W)],
        "expected": [[float(r * W)] for r in range(W)],
    }
    # reduce_scatter (list), :579-610: rank r's list = [[r+i+1] for i] -> rank r gets (1+W)W/2 + W*r
    c["reduce_scatter_list"] = {
        "inputs": [[[r + i + 1] for i in range(W)] for r in range(W)],
        "expected": [[(1 + W) * W // 2 + W * r] for r in range(W)],
    }
    # variable-length variant, :623-653: slot i of rank r = [r+i+1]*(i+1); rank r gets (r+1) copies
    c["reduce_scatter_list_variable"] = {
        "inputs": [[[r + i + 1] * (i + 1) for i in range(W)] for r in range(W)],
        "expected": [[(1 + W) * W // 2 + W * r] * (r + 1) for r in range(W)],
    }
    # _allgather_base, :377-391: rank r contributes [r] -> arange(W)
    c["allgather_base"] = {"inputs": [[r] for r in range(W)], "expected": list(range(W))}
    # allgather (list), :345-364: for n in range(W): rank r contributes [n*r] -> [[i*n] for i]
    c["allgather_list"] = [{"inputs": [[n * r] for r in range(W)], "expected": [[i * n] for i in range(W)]}
                           for n in range(W)]
    # alltoall_base equal split, :443-456: rank r sends ones[W,W]*r -> everybody receives rows i
    c["alltoall_base_equal"] = {
        "inputs": [[[float(r)] * W for _ in range(W)] for r in range(W)],
        "expected": [[[float(i)] * W for i in range(W)] for _ in range(W)],
    }
    # alltoall_base uneven, :458-473: in_splits = [i+1], out_splits = [rank+1]*W
    c["alltoall_base_unequal"] = {
        "in_splits": [[i + 1 for i in range(W)] for _ in range(W)],
        "out_splits": [[r + 1] * W for r in range(W)],
        "inputs": [[[float(r)] * W for _ in range(sum(i + 1 for i in range(W)))] for r in range(W)],
        "expected": [[[float(i)] * W for i in range(W) for _ in range(r + 1)] for r in range(W)],
    }
    # alltoall (list), :498-518: same data as the uneven base case, as lists of tensors
    c["alltoall_list"] = {
        "inputs": [[[[float(r)] * W for _ in range(i + 1)] for i in range(W)] for r in range(W)],
        "expected": [[[[float(i)] * W for _ in range(r + 1)] for i in range(W)] for r in range(W)],
    }
    # reduce to every root in turn, :221-237: the allreduce cases, checked on the root only
    c["reduce"] = {"inputs": inputs, "expected": c["allreduce"]["expected"], "roots": list(range(W))}
    # gather, :254-277: rank r contributes [r]; every rank is root once and then holds [[0], [1], ...]
    c["gather"] = {"inputs": [[r] for r in range(W)], "expected": [[r] for r in range(W)], "roots": list(range(W))}
    # scatter, :290-308: every root in turn scatters [[0], [1], ...]; rank r receives [r]
    c["scatter"] = {"inputs": [[r] for r in range(W)], "expected": [[r] for r in range(W)], "roots": list(range(W))}
    # coalescing manager, :667-693: two 8-element allreduces of ones == one 16-element allreduce
    c["coalesced_allreduce_ones"] = {"num_colls": 2, "size_per_coll": 8, "expected_value": float(W)}
    # reduce_scatter_tensor of ones, :716-733: -> W
    c["reduce_scatter_tensor_ones"] = {"shape": [2, 2], "expected_value": float(W)}
    return c


def p2p_cases():
    """tests/test_c10d_p2p.py (world size 6): rank r owns a cube of side r+1 filled with r+1
    (:29-36).  A pair 0 -> 1 (:38-68), a relay 1 -> 3 -> 5 (:73-109), every rank to every other in
    turn (:114-147), and cubes of side 10 filled with the sender's rank, tagged (:152-183)."""
    W = 6
    return {
        "world_size": W,
        "cube": [{"side": r + 1, "value": float(r + 1)} for r in range(W)],
        "pair": {"src": 0, "dst": 1},
        "relay": [{"src": 1, "dst": 3}, {"src": 3, "dst": 5}],
        "all_pairs": [{"src": s, "dst": d} for s in range(W) for d in range(W) if s != d],
        "tagged": {"side": 10, "messages": [{"src": s, "dst": d, "tag": s, "value": float(s)}
                                            for d in range(W) for s in range(W) if s != d]},
    }


def main():
    data = {"source": "closed forms of intel/torch-ccl tests/test_c10d_ccl.py and tests/test_c10d_p2p.py "
                      "(lines cited in make_kat_fixture.py)",
            "world_sizes": {str(W): cases_for(W) for W in range(2, 9)},
            "p2p": p2p_cases()}
    with open(os.path.join(HERE, "c10d_kats.json"), "w") as f:
        json.dump(data, f, separators=(",", ":"))
    print("wrote c10d_kats.json")


if __name__ == "__main__":
    main()
