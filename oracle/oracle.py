"""ctypes front end of the CPU oracle (oracle/mccl_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  Arrays are numpy arrays; bf16 and fp16 buffers travel as uint16 bit patterns
(numpy has no bf16), everything else in its natural numpy dtype.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# dtype / op codes, identical to include/mccl.h
U8, I8, I16, I32, I64, F16, F32, F64, BF16 = range(9)
SUM, AVG, PROD, MIN, MAX = 0, 1, 2, 3, 4

DTYPE_SIZE = {U8: 1, I8: 1, I16: 2, I32: 4, I64: 8, F16: 2, F32: 4, F64: 8, BF16: 2}
# numpy carrier dtype for each code (bit patterns for the 16-bit floats)
CARRIER = {U8: np.uint8, I8: np.int8, I16: np.int16, I32: np.int32, I64: np.int64,
           F16: np.uint16, F32: np.float32, F64: np.float64, BF16: np.uint16}


def build(force=False):
    """Compile liboracle.so with the Makefile beside it (gcc, a second or two)."""
    src = os.path.join(_HERE, "mccl_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)
             or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src))
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        L.oracle_reduce.argtypes = [vp, i32, vp, sz, i32, i32]
        L.oracle_reduce_scatter.argtypes = [vp, i32, vp, sz, i32, i32, i32, i32]
        L.oracle_allgather.argtypes = [vp, i32, vp, sz]
        L.oracle_alltoall_counts.argtypes = [i32, ctypes.c_int64, ctypes.c_int64, vp, vp, vp]
        L.oracle_alltoallv.argtypes = [vp, vp, i32, vp, sz]
        L.oracle_pack.argtypes = [vp, vp, i32, vp]
        L.oracle_unpack.argtypes = [vp, vp, vp, i32]
        L.oracle_gather_rows.argtypes = [vp, sz, vp, sz, sz, vp]
        L.oracle_moe_dispatch.argtypes = [vp, vp, vp, vp, i32, vp, sz]
        L.oracle_moe_combine.argtypes = [vp, vp, i32, vp, vp, vp, sz, i32, sz, i32, vp]
        L.oracle_route_counts.argtypes = [vp, sz, i32, vp]
        L.oracle_set_threads.argtypes = [i32]
        for name in ("f32_to_bf16", "f32_to_f16", "f16_to_f32", "bf16_to_f32"):
            getattr(L, "oracle_%s_array" % name).argtypes = [vp, vp, sz]
        _lib = L
    return _lib


def set_threads(n):
    lib().oracle_set_threads(int(n))


def max_threads():
    return int(lib().oracle_max_threads())


def _ptr_array(arrays):
    return (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])


def _check(arrays, dtype):
    out = []
    for a in arrays:
        a = np.ascontiguousarray(a)
        assert a.dtype == CARRIER[dtype], (a.dtype, CARRIER[dtype])
        out.append(a)
    return out


def reduce(inputs, dtype, op=SUM):
    """Reduce N equal-length 1-D arrays; returns a new array."""
    ins = _check(inputs, dtype)
    count = ins[0].size
    assert all(a.size == count for a in ins)
    out = np.empty(count, dtype=CARRIER[dtype])
    rc = lib().oracle_reduce(_ptr_array(ins), len(ins), out.ctypes.data, count, dtype, op)
    assert rc == 0, rc
    return out


def reduce_scatter(inputs, dtype, op=SUM, shard_first=0, shard_num=None):
    """inputs: N arrays of N*M elements; returns the list of reduced shards."""
    ins = _check(inputs, dtype)
    n = len(ins)
    assert ins[0].size % n == 0
    m = ins[0].size // n
    if shard_num is None:
        shard_num = n - shard_first
    outs = [np.empty(m, dtype=CARRIER[dtype]) for _ in range(shard_num)]
    rc = lib().oracle_reduce_scatter(_ptr_array(ins), n, _ptr_array(outs), m,
                                     shard_first, shard_num, dtype, op)
    assert rc == 0, rc
    return outs


def allgather(inputs):
    """inputs: N byte-equal-sized arrays; returns the concatenation rank-major (uint8)."""
    ins = [np.ascontiguousarray(a).view(np.uint8).reshape(-1) for a in inputs]
    b = ins[0].size
    assert all(a.size == b for a in ins)
    out = np.empty(b * len(ins), dtype=np.uint8)
    lib().oracle_allgather(_ptr_array(ins), len(ins), out.ctypes.data, b)
    return out


def alltoall_counts(world, numel, dim0, split=None):
    """Split arithmetic of alltoall_base: (counts, displacements) in elements."""
    counts = np.zeros(world, dtype=np.int64)
    displs = np.zeros(world, dtype=np.int64)
    sp = None
    if split is not None:
        sp = np.ascontiguousarray(split, dtype=np.int64)
    rc = lib().oracle_alltoall_counts(world, numel, dim0,
                                      sp.ctypes.data if sp is not None else None,
                                      counts.ctypes.data, displs.ctypes.data)
    assert rc == 0, rc
    return counts, displs


def alltoallv(inputs, split_rows, row_bytes):
    """inputs: N uint8 arrays (rank r's send buffer); split_rows[r][d] = rows r -> d.
    Returns the N receive buffers as uint8 arrays."""
    ins = [np.ascontiguousarray(a).view(np.uint8).reshape(-1) for a in inputs]
    n = len(ins)
    S = np.ascontiguousarray(split_rows, dtype=np.int64).reshape(n, n)
    outs = [np.empty(int(S[:, d].sum()) * row_bytes, dtype=np.uint8) for d in range(n)]
    for r in range(n):
        assert ins[r].size == int(S[r].sum()) * row_bytes
    lib().oracle_alltoallv(_ptr_array(ins), _ptr_array(outs), n, S.ctypes.data, row_bytes)
    return outs


def pack(srcs):
    ins = [np.ascontiguousarray(a).view(np.uint8).reshape(-1) for a in srcs]
    sizes = (ctypes.c_size_t * len(ins))(*[a.size for a in ins])
    out = np.empty(sum(a.size for a in ins), dtype=np.uint8)
    lib().oracle_pack(_ptr_array(ins), sizes, len(ins), out.ctypes.data)
    return out


def unpack(src, sizes):
    src = np.ascontiguousarray(src).view(np.uint8).reshape(-1)
    outs = [np.empty(int(s), dtype=np.uint8) for s in sizes]
    csz = (ctypes.c_size_t * len(outs))(*[int(s) for s in sizes])
    lib().oracle_unpack(src.ctypes.data, _ptr_array(outs), csz, len(outs))
    return outs


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16_array(x.ctypes.data, out.ctypes.data, x.size)
    return out


def f32_to_f16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_f16_array(x.ctypes.data, out.ctypes.data, x.size)
    return out


def f16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_f16_to_f32_array(h.ctypes.data, out.ctypes.data, h.size)
    return out


def bf16_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_bf16_to_f32_array(h.ctypes.data, out.ctypes.data, h.size)
    return out


def gather_rows(src, idx, row_bytes):
    """dst row j = src row idx[j] (uint8 arrays); out-of-range indices leave zeros."""
    src = np.ascontiguousarray(src).view(np.uint8).reshape(-1)
    idx = np.ascontiguousarray(idx, dtype=np.int64)
    out = np.zeros(idx.size * row_bytes, dtype=np.uint8)
    lib().oracle_gather_rows(src.ctypes.data, src.size // row_bytes, idx.ctypes.data, idx.size, row_bytes,
                             out.ctypes.data)
    return out


def moe_dispatch(hidden, idx, split_rows, row_bytes):
    """hidden[r]: rank r's rows (uint8); idx[r]: its send order; returns the n receive buffers."""
    hs = [np.ascontiguousarray(h).view(np.uint8).reshape(-1) for h in hidden]
    ix = [np.ascontiguousarray(i, dtype=np.int64) for i in idx]
    n = len(hs)
    S = np.ascontiguousarray(split_rows, dtype=np.int64).reshape(n, n)
    outs = [np.zeros(int(S[:, d].sum()) * row_bytes, dtype=np.uint8) for d in range(n)]
    rows = (ctypes.c_size_t * n)(*[h.size // row_bytes for h in hs])
    lib().oracle_moe_dispatch(_ptr_array(hs), rows, _ptr_array(ix), _ptr_array(outs), n, S.ctypes.data, row_bytes)
    return outs


def moe_combine(x, src_rank, src_row, w, tokens, topk, hidden, dtype):
    """x[r]: rank r's expert-output rows in the carrier dtype; returns y [tokens*hidden] carrier."""
    xs = _check(x, dtype)
    n = len(xs)
    sr = np.ascontiguousarray(src_rank, dtype=np.int32)
    so = np.ascontiguousarray(src_row, dtype=np.int64)
    ww = np.ascontiguousarray(w, dtype=np.float32)
    assert sr.size == so.size == ww.size == tokens * topk
    rows = (ctypes.c_size_t * n)(*[a.size // hidden for a in xs])
    y = np.empty(tokens * hidden, dtype=CARRIER[dtype])
    rc = lib().oracle_moe_combine(_ptr_array(xs), rows, n, sr.ctypes.data, so.ctypes.data, ww.ctypes.data,
                                  tokens, topk, hidden, dtype, y.ctypes.data)
    assert rc == 0, rc
    return y


def route_counts(expert_ids, n_experts):
    """counts[e] = number of entries of expert_ids equal to e (ids out of range ignored)."""
    ids = np.ascontiguousarray(expert_ids, dtype=np.int32).reshape(-1)
    out = np.zeros(n_experts, dtype=np.int64)
    rc = lib().oracle_route_counts(ids.ctypes.data, ids.size, n_experts, out.ctypes.data)
    if rc != 0:
        raise ValueError("oracle_route_counts failed")
    return out
