"""ctypes binding of libmi355ccl.so (the C ABI declared in include/mccl.h).

torch is imported first on purpose: the library's HIP runtime dependency then resolves to
the runtime torch already loaded, so both share streams and allocations.  There is no CPU
fallback anywhere in this module: a missing library is an ImportError, a failed call is a
RuntimeError carrying mccl_last_error().
"""
import ctypes
import os

import torch  # noqa: F401  (must precede the CDLL below)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmi355ccl.so")

# dtype codes (mccl_dtype_t), mirroring cclDatatypes of the reference (src/utils.cpp:46-58)
U8, I8, I16, I32, I64, F16, F32, F64, BF16 = range(9)
# op codes (mccl_op_t), numbered like c10d::ReduceOp
SUM, AVG, PROD, MIN, MAX = 0, 1, 2, 3, 4
VARIANT_AUTO, VARIANT_SMALL, VARIANT_PERSISTENT, VARIANT_STREAM = 0, 1, 2, 3
(TUNE_PERSISTENT_BLOCKS_PER_CU, TUNE_STREAM_WAVES_PER_CU, TUNE_SMALL_MAX_BYTES,
 TUNE_COPY_WAVES_PER_CU, TUNE_STREAM_MIN_TOTAL_BYTES, TUNE_COMBINE_PIECES_PER_WAVE,
 TUNE_COMBINE_WAVES_PER_CU, TUNE_XRANK_WAVES_ALL_RANKS, TUNE_COPY_VECTORS_PER_LANE, TUNE_COPY_STREAM_STORES,
 TUNE_COPY_LARGE_MIN_BYTES, TUNE_GATHER_WAVES_PER_CU, TUNE_XRANK_CACHED_LOADS, TUNE_XRANK_FRESH_WAVES_PER_CU,
 TUNE_XRANK_FRESH_MAX_WAVES) = range(15)
COPY_SHARED_SOURCES = 1  # flag of mccl_copy_segments_sync
FUSED_WORK_ONLY, FUSED_SYNC_ONLY = 1, 2  # flags of mccl_allreduce_fused_replayable
FUSED_STATE_BYTES = 128
MAX_RANKS = 64

TORCH_DTYPE = {
    torch.uint8: U8, torch.int8: I8, torch.int16: I16, torch.int32: I32, torch.int64: I64,
    torch.float16: F16, torch.float32: F32, torch.float64: F64, torch.bfloat16: BF16,
    torch.bool: U8,
}

EXPORTS = (
    "mccl_version", "mccl_last_error", "mccl_dtype_size", "mccl_reduce_n",
    "mccl_reduce_scatter_n", "mccl_reduce_multi", "mccl_copy_segments", "mccl_allgather_n",
    "mccl_alltoallv_n", "mccl_alltoallv_pull", "mccl_pack", "mccl_unpack",
    "mccl_query_launch", "mccl_set_tuning", "mccl_get_tuning",
    "mccl_gather_rows", "mccl_moe_dispatch_n", "mccl_moe_combine",
    "mccl_rank_barrier", "mccl_rank_barrier_offers", "mccl_rank_barrier_offers_each", "mccl_import_table_update", "mccl_allreduce_sync_resolved", "mccl_allreduce_sync_offers",
    "mccl_reduce_sync_resolved", "mccl_reduce_sync_offers", "mccl_fanout_sync_resolved", "mccl_fanout_sync_offers", "mccl_allreduce_fused", "mccl_allreduce_fused_replayable", "mccl_fanout_sync",
    "mccl_copy_segments_sync", "mccl_copy_segments_sync_resolved", "mccl_alltoall_sync_offers", "mccl_reduce_sync", "mccl_allreduce_sync_shard", "mccl_allreduce_sync",
    "mccl_route_counts", "mccl_route_counts_noalloc", "mccl_placement_check",
)


class XSync(ctypes.Structure):
    """mccl_xsync_t"""
    _fields_ = [("words", ctypes.c_void_p), ("n", ctypes.c_int), ("rank", ctypes.c_int),
                ("ready_epoch", ctypes.c_uint64), ("done_epoch", ctypes.c_uint64), ("done_counter", ctypes.c_void_p),
                ("timeout_us", ctypes.c_uint64), ("status", ctypes.c_void_p),
                ("max_compute_units", ctypes.c_uint), ("reserved", ctypes.c_uint)]


OFFER_RANKS, OFFER_ENTRIES, OFFER_STAGED, STATUS_UNMAPPED = 8, 32, 0xffffffff, 0xfffffffe
OFFER_SLOTS, OFFER_SLOT_OUTBOX, STATUS_MISMATCH = 4, 2, 0xfffffffd


class Offer(ctypes.Structure):
    """mccl_offer_t"""
    _fields_ = [("entry", ctypes.c_uint32), ("slot", ctypes.c_uint32), ("generation", ctypes.c_uint64),
                ("offset", ctypes.c_uint64), ("bytes", ctypes.c_uint64)]


class ImportTable(ctypes.Structure):
    """mccl_import_table_t"""
    _fields_ = [("base", ctypes.c_uint64 * OFFER_ENTRIES * OFFER_RANKS),
                ("generation", ctypes.c_uint64 * OFFER_ENTRIES * OFFER_RANKS),
                ("staging", ctypes.c_uint64 * OFFER_SLOTS * OFFER_RANKS)]


class ImportUpdate(ctypes.Structure):
    """mccl_import_update_t"""
    _fields_ = [("rank", ctypes.c_uint32), ("entry", ctypes.c_uint32), ("slot", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
                ("base", ctypes.c_uint64), ("generation", ctypes.c_uint64)]


class Segment(ctypes.Structure):
    _fields_ = [("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("bytes", ctypes.c_size_t)]


_lib = None


def lib():
    """Loads the shared library once; raises ImportError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libmi355ccl.so is not built (%s); run `python torch-ccl_amd/csrc/build.py`" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    L.mccl_version.restype = i32
    L.mccl_last_error.restype = ctypes.c_char_p
    L.mccl_dtype_size.restype = sz
    L.mccl_dtype_size.argtypes = [i32]
    L.mccl_reduce_n.argtypes = [vp, i32, vp, sz, i32, i32, i32, vp]
    L.mccl_reduce_scatter_n.argtypes = [vp, i32, vp, sz, i32, i32, i32, i32, vp]
    L.mccl_reduce_multi.argtypes = [vp, i32, vp, vp, i32, i32, i32, vp]
    L.mccl_copy_segments.argtypes = [vp, i32, vp]
    L.mccl_allgather_n.argtypes = [vp, i32, vp, sz, vp]
    L.mccl_alltoallv_n.argtypes = [vp, vp, i32, vp, sz, vp]
    L.mccl_alltoallv_pull.argtypes = [vp, i32, vp, vp, vp, vp]
    L.mccl_pack.argtypes = [vp, vp, i32, vp, vp]
    L.mccl_unpack.argtypes = [vp, vp, vp, i32, vp]
    L.mccl_gather_rows.argtypes = [vp, sz, vp, sz, sz, vp, vp]
    L.mccl_moe_dispatch_n.argtypes = [vp, vp, vp, vp, i32, vp, sz, vp]
    L.mccl_moe_combine.argtypes = [vp, vp, i32, vp, vp, vp, sz, i32, sz, i32, vp, vp]
    L.mccl_rank_barrier.argtypes = [vp, i32, i32, ctypes.c_uint64, ctypes.c_uint64, vp, vp]
    L.mccl_rank_barrier_offers.argtypes = [vp, i32, i32, ctypes.c_uint64, ctypes.c_uint64, vp, vp, vp, vp, vp, vp, vp]
    L.mccl_rank_barrier_offers_each.argtypes = [vp, i32, i32, ctypes.c_uint64, ctypes.c_uint64, vp, vp, vp, vp, vp, vp, vp, vp]
    L.mccl_allreduce_sync_resolved.argtypes = [vp, sz, i32, i32, vp, vp]
    L.mccl_import_table_update.argtypes = [vp, vp, i32, vp]
    L.mccl_allreduce_sync_offers.argtypes = [sz, i32, i32, vp, vp, vp, vp, vp, vp]
    L.mccl_reduce_sync_resolved.argtypes = [vp, sz, vp, sz, i32, i32, vp, vp]
    L.mccl_reduce_sync_offers.argtypes = [sz, vp, sz, i32, i32, vp, vp, vp, vp, vp, vp]
    L.mccl_fanout_sync_resolved.argtypes = [vp, vp, sz, sz, i32, vp, vp]
    L.mccl_fanout_sync_offers.argtypes = [vp, sz, sz, i32, vp, vp, vp, vp, vp, vp]
    L.mccl_allreduce_fused.argtypes = [vp, vp, sz, i32, i32, vp, vp, i32, i32, ctypes.c_uint32, ctypes.c_uint64, vp, ctypes.c_uint, vp]
    L.mccl_allreduce_fused_replayable.argtypes = [vp, vp, sz, i32, i32, vp, vp, sz, sz, vp, i32, i32, ctypes.c_uint64, vp, ctypes.c_uint, ctypes.c_uint, vp]
    L.mccl_copy_segments_sync.argtypes = [vp, i32, ctypes.c_uint, vp, vp]
    L.mccl_copy_segments_sync_resolved.argtypes = [vp, vp, i32, vp, ctypes.c_uint, vp, vp]
    L.mccl_alltoall_sync_offers.argtypes = [vp, i32, vp, vp, i32, vp, vp, vp, vp, vp, vp, vp]
    L.mccl_fanout_sync.argtypes = [vp, vp, i32, sz, vp, vp]
    L.mccl_reduce_sync.argtypes = [vp, vp, sz, i32, i32, vp, vp]
    L.mccl_allreduce_sync.argtypes = [vp, sz, i32, i32, vp, vp]
    L.mccl_allreduce_sync_shard.argtypes = [sz, i32]
    L.mccl_allreduce_sync_shard.restype = sz
    L.mccl_placement_check.argtypes = [vp, i32, sz]
    L.mccl_route_counts.argtypes = [vp, sz, i32, vp, vp, vp]
    L.mccl_route_counts_noalloc.argtypes = [vp, sz, i32, vp, vp]
    L.mccl_query_launch.argtypes = [sz, i32, i32, i32, i32, vp, vp]
    L.mccl_set_tuning.argtypes = [i32, ctypes.c_longlong]
    L.mccl_get_tuning.argtypes = [i32]
    L.mccl_get_tuning.restype = ctypes.c_longlong
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise RuntimeError("mccl error %d: %s" % (rc, lib().mccl_last_error().decode()))


def ptr_table(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)


def size_table(sizes):
    return (ctypes.c_size_t * len(sizes))(*[int(s) for s in sizes])
