"""No-GPU checks of the native boundary: the shared libraries load, export every symbol the
headers declare, and the entry points that need no device behave.  Also guards the product
tree against routing through the CPU oracle."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "torch-ccl_amd")


def _declared(header, folder="include"):
    text = open(os.path.join(ROOT, folder, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mcclb?_[a-z0-9_]+)\s*\(", text)))


def test_libmi355ccl_exports_every_declared_symbol(mccl):
    from torch_ccl_amd import capi
    L = capi.lib()
    names = _declared("mccl.h")
    assert len(names) >= 14
    for name in names:
        assert hasattr(L, name), "libmi355ccl.so does not export %s" % name
    assert sorted(capi.EXPORTS) == names


def test_libmcclbench_exports_every_declared_symbol(mccl):
    import sys
    sys.path.insert(0, os.path.join(ROOT, "bench"))
    import benchlib
    L = benchlib.lib()
    names = [n for n in _declared("mccl_bench.h", "bench") if n.startswith("mcclb_")]
    assert len(names) >= 12
    for name in names:
        assert hasattr(L, name), "libmcclbench.so does not export %s" % name


def test_device_free_entry_points(mccl):
    from torch_ccl_amd import capi
    L = capi.lib()
    assert L.mccl_version() >= 100
    sizes = {capi.U8: 1, capi.I8: 1, capi.I16: 2, capi.I32: 4, capi.I64: 8,
             capi.F16: 2, capi.F32: 4, capi.F64: 8, capi.BF16: 2}
    for code, size in sizes.items():
        assert L.mccl_dtype_size(code) == size
    assert L.mccl_dtype_size(99) == 0
    assert L.mccl_set_tuning(99, 1) == -1
    assert b"unknown tuning knob" in L.mccl_last_error()
    default = L.mccl_get_tuning(capi.TUNE_COPY_WAVES_PER_CU)
    assert L.mccl_set_tuning(capi.TUNE_COPY_WAVES_PER_CU, 12) == 0
    assert L.mccl_get_tuning(capi.TUNE_COPY_WAVES_PER_CU) == 12
    assert L.mccl_set_tuning(capi.TUNE_COPY_WAVES_PER_CU, 0) == 0
    assert L.mccl_get_tuning(capi.TUNE_COPY_WAVES_PER_CU) == default


def test_argument_errors_need_no_device(mccl):
    """Validation happens before any HIP call: bad arguments come back as status codes."""
    from torch_ccl_amd import capi
    L = capi.lib()
    one = capi.ptr_table([0x1000])
    assert L.mccl_reduce_n(None, 2, None, 8, capi.F32, capi.SUM, 0, None) == -1
    assert L.mccl_reduce_n(one, 0, None, 8, capi.F32, capi.SUM, 0, None) == -1
    assert L.mccl_reduce_n(one, 65, None, 8, capi.F32, capi.SUM, 0, None) == -1
    assert L.mccl_reduce_n(one, 1, None, 8, 42, capi.SUM, 0, None) == -1
    assert L.mccl_reduce_n(one, 1, None, 8, capi.F32, 7, 0, None) == -1
    assert L.mccl_reduce_n(one, 1, None, 8, capi.I32, capi.AVG, 0, None) == -3
    assert b"AVG" in L.mccl_last_error()
    assert L.mccl_reduce_n(one, 1, None, 0, capi.F32, capi.SUM, 0, None) == 0  # empty message: no-op
    assert L.mccl_allgather_n(one, 1, None, 0, None) == 0
    assert L.mccl_copy_segments(None, 0, None) == 0
    assert L.mccl_copy_segments(None, 3, None) == -1


def test_overlapping_buffers_are_rejected_before_any_launch(mccl):
    """In place means: the output is exactly the range the reduction reads from one rank.  Any other
    overlap between an output and something the same launch reads or writes is refused."""
    from torch_ccl_amd import capi
    L = capi.lib()
    base, nbytes = 0x10000000, 4096 * 4
    ins = capi.ptr_table([base, base + 0x100000])
    out = ctypes.c_void_p
    # partial overlap with input 1
    assert L.mccl_reduce_n(ins, 2, out(base + 0x100000 + 64), 4096, capi.F32, capi.SUM, 0, None) == -1
    assert b"partially overlaps input 1" in L.mccl_last_error()
    assert L.mccl_reduce_n(ins, 2, out(base - nbytes + 4), 4096, capi.F32, capi.SUM, 0, None) == -1
    assert b"partially overlaps input 0" in L.mccl_last_error()
    # reduce_scatter: shard 0's output inside the range shard 1 reads from rank 0
    outs = capi.ptr_table([base + 0x200000, base + 1024 * 4 + 16])
    assert L.mccl_reduce_scatter_n(ins, 2, outs, 1024, 0, 2, capi.F32, capi.SUM, None) == -1
    assert b"overlaps input 0 of reduction 1" in L.mccl_last_error()
    # two outputs of one coalesced launch overlapping each other
    tab = capi.ptr_table([base, base + 0x100000, base + 0x200000, base + 0x300000])
    outs = capi.ptr_table([base + 0x400000, base + 0x400000 + 512])
    counts = (ctypes.c_size_t * 2)(1024, 1024)
    assert L.mccl_reduce_multi(tab, 2, outs, counts, 2, capi.F32, capi.SUM, None) == -1
    assert b"outputs" in L.mccl_last_error() and b"overlap" in L.mccl_last_error()


def test_one_launch_collectives_reject_partial_overlap(mccl):
    """mccl_reduce_sync: the output may be exactly one of the inputs, nothing else of them;
    mccl_allreduce_sync: two ranks' tensors may be the same memory, never partly so."""
    from torch_ccl_amd import capi
    L = capi.lib()
    base = 0x10000000
    ins = capi.ptr_table([base, base + 0x100000])
    sy = capi.XSync(None, 2, 0, 0, 0, None, 0, None)  # no waits: words, counters and status are not used
    assert L.mccl_reduce_sync(ins, ctypes.c_void_p(base + 0x100000 + 64), 4096, capi.F32, capi.SUM, ctypes.byref(sy), None) == -1
    assert b"partially overlaps input 1" in L.mccl_last_error()
    assert L.mccl_reduce_sync(ins, ctypes.c_void_p(base - 4096 * 4 + 4), 4096, capi.F32, capi.SUM, ctypes.byref(sy), None) == -1
    assert b"partially overlaps input 0" in L.mccl_last_error()
    tens = capi.ptr_table([base, base + 4096 * 4 - 8])
    assert L.mccl_allreduce_sync(tens, 4096, capi.F32, capi.SUM, ctypes.byref(sy), None) == -1
    assert b"tensors 0 and 1 partially overlap" in L.mccl_last_error()


def test_offer_entry_points_reject_bad_arguments_without_a_device(mccl):
    """mccl_rank_barrier_offers(_each), mccl_import_table_update, the `_resolved` and `_offers` forms and
    mccl_allreduce_fused_replayable: every refusal that depends on arguments only."""
    from torch_ccl_amd import capi
    L = capi.lib()
    err = lambda: L.mccl_last_error().decode()
    vp = ctypes.c_void_p
    two = capi.ptr_table([0x10000, 0x20000])
    nine = capi.ptr_table([0x10000 + 64 * i for i in range(9)])
    offer = capi.Offer(3, 0, 7, 0, 0)
    tab, res = vp(0x40000), vp(0x50000)
    assert L.mccl_rank_barrier_offers(nine, 9, 0, 1, 0, None, ctypes.byref(offer), vp(0x1000), nine, tab, res, None) == -3 and "1 to 8 ranks" in err()
    assert L.mccl_rank_barrier_offers(two, 2, 2, 1, 0, None, ctypes.byref(offer), vp(0x1000), two, tab, res, None) == -1 and "rank 2" in err()
    assert L.mccl_rank_barrier_offers(two, 2, 0, 1, 0, None, None, vp(0x1000), two, tab, res, None) == -1 and "null" in err()
    assert L.mccl_rank_barrier_offers(two, 2, 0, 1, 0, None, ctypes.byref(offer), vp(0x1000), two, vp(0x40004), res, None) == -1 and "8-byte" in err()
    assert L.mccl_rank_barrier_offers(two, 2, 0, 1, 0, None, ctypes.byref(offer), vp(0x1000), capi.ptr_table([0x10000, 0x20004]), tab, res, None) == -1
    assert "offer pointer 1" in err()
    bad = capi.Offer(32, 0, 7, 0, 0)
    assert L.mccl_rank_barrier_offers(two, 2, 0, 1, 0, None, ctypes.byref(bad), vp(0x1000), two, tab, res, None) == -1 and "entry 32" in err()
    # table updates
    ups = (capi.ImportUpdate * 9)()
    assert L.mccl_import_table_update(tab, ups, 0, None) == 0
    assert L.mccl_import_table_update(tab, ups, 9, None) == -1 and "at most 8" in err()
    ups[0] = capi.ImportUpdate(8, 0, 0, 0, 0x1000, 1)
    assert L.mccl_import_table_update(tab, ups, 1, None) == -1 and "rank 8" in err()
    ups[0] = capi.ImportUpdate(1, 40, 0, 0, 0x1000, 1)
    assert L.mccl_import_table_update(tab, ups, 1, None) == -1 and "entry 40" in err()
    ups[0] = capi.ImportUpdate(1, 5, 0, 0, 0x1000, 1)
    ups[1] = capi.ImportUpdate(1, 5, 0, 0, 0x2000, 2)
    assert L.mccl_import_table_update(tab, ups, 2, None) == -1 and "same entry" in err()
    ups[0] = capi.ImportUpdate(1, capi.OFFER_STAGED, 0, 0, 0x1000, 0)
    ups[1] = capi.ImportUpdate(1, capi.OFFER_STAGED, 1, 0, 0x2000, 0)  # the two staging slots of one rank: different entries
    assert L.mccl_import_table_update(None, ups, 2, None) == -1 and "null" in err()
    # the forms behind a barrier want no opening epoch and a closing one; the one-launch forms want all three
    words = capi.ptr_table([0x60000, 0x60040])
    behind = capi.XSync(ctypes.cast(words, vp), 2, 0, 0, 7, vp(0x70000), 0, None, 0, 0)
    opening = capi.XSync(ctypes.cast(words, vp), 2, 0, 5, 7, vp(0x70000), 0, None, 0, 0)
    one = capi.XSync(ctypes.cast(words, vp), 2, 0, 5, 7, vp(0x70000), 0, None, 16, 0)
    assert L.mccl_allreduce_sync_resolved(res, 64, capi.F32, capi.SUM, ctypes.byref(opening), None) == -1 and "behind a barrier" in err()
    assert L.mccl_allreduce_sync_resolved(None, 64, capi.F32, capi.SUM, ctypes.byref(behind), None) == -1 and "null" in err()
    assert L.mccl_reduce_sync_resolved(res, 0, vp(0x80000), 64, capi.F32, capi.SUM, ctypes.byref(opening), None) == -1 and "behind a barrier" in err()
    assert L.mccl_reduce_sync_resolved(res, 2, vp(0x80000), 64, capi.F32, capi.SUM, ctypes.byref(behind), None) == -1 and "offset" in err()
    assert L.mccl_fanout_sync_resolved(vp(0x90000), res, 0, 64, 0, ctypes.byref(opening), None) == -1 and "behind a barrier" in err()
    assert L.mccl_allreduce_sync_offers(64, capi.F32, capi.SUM, ctypes.byref(opening), ctypes.byref(offer), vp(0x1000), two, tab, None) == -1
    assert "max_compute_units" in err()
    assert L.mccl_reduce_sync_offers(0, vp(0x80000), 64, capi.F32, capi.SUM, ctypes.byref(behind), ctypes.byref(offer), vp(0x1000), two, tab, None) == -1
    assert "max_compute_units" in err()
    assert L.mccl_fanout_sync_offers(vp(0x90000), 0, 64, 0, ctypes.byref(one), ctypes.byref(bad), vp(0x1000), two, tab, None) == -1 and "entry 32" in err()
    assert L.mccl_reduce_sync_offers(0, vp(0x80000), 64, capi.I32, capi.AVG, ctypes.byref(one), ctypes.byref(offer), vp(0x1000), two, tab, None) == -3
    # a row of offers per rank (alltoall): the same refusals, per offer
    rows = (capi.Offer * 2)(capi.Offer(3, 0, 7, 0, 64), capi.Offer(capi.OFFER_STAGED, capi.OFFER_SLOT_OUTBOX, 0, 0, 64))
    expect = (ctypes.c_uint64 * 2)(64, 64)
    each = lambda n, rank, mine, exp, offers, imports=tab, flags=two: L.mccl_rank_barrier_offers_each(
        flags, n, rank, 1, 0, None, mine, exp, vp(0x1000), offers, imports, res, None)
    assert each(9, 0, rows, expect, nine, flags=nine) == -3 and "1 to 8 ranks" in err()
    assert each(2, 2, rows, expect, two) == -1 and "rank 2" in err()
    assert each(2, 0, None, expect, two) == -1 and "null" in err()
    assert each(2, 0, rows, None, two) == -1 and "null" in err()
    assert each(2, 0, rows, expect, two, imports=vp(0x40004)) == -1 and "8-byte" in err()
    assert each(2, 0, rows, expect, capi.ptr_table([0x10000, 0x20004])) == -1 and "offer pointer 1" in err()
    rows[1] = capi.Offer(40, 0, 7, 0, 64)
    assert each(2, 0, rows, expect, two) == -1 and "offer 1 names entry 40" in err()
    rows[1] = capi.Offer(capi.OFFER_STAGED, 4, 0, 0, 64)
    assert each(2, 0, rows, expect, two) == -1 and "staging buffer 4" in err()
    ups[0] = capi.ImportUpdate(1, capi.OFFER_STAGED, 4, 0, 0x1000, 0)
    assert L.mccl_import_table_update(tab, ups, 1, None) == -1 and "staging buffer 4" in err()
    # the pulls behind it
    segs = (capi.Segment * 2)(capi.Segment(0, 0xa0000, 4096), capi.Segment(0x100, 0xb0000, 4096))
    from_ = (ctypes.c_int * 2)(0, 1)
    pull = lambda sy, table=res, ranks=from_, n=2: L.mccl_copy_segments_sync_resolved(segs, ranks, n, table, 0, ctypes.byref(sy), None)
    assert pull(opening) == -1 and "behind a barrier" in err()
    assert pull(behind, table=None) == -1 and "null" in err()
    assert pull(behind, table=vp(0x50004)) == -1 and "8-byte" in err()
    assert pull(behind, ranks=None) == -1 and "source rank table" in err()
    assert pull(behind, ranks=(ctypes.c_int * 2)(0, 2)) == -1 and "rank 2 of 2" in err()
    segs[1] = capi.Segment(0x100, 0, 4096)
    assert pull(behind) == -1 and "null pointer" in err()
    segs[1] = capi.Segment(0, 0xb0000, 4096)
    assert pull(behind, ranks=(ctypes.c_int * 2)(0, -1)) == -1 and "null pointer" in err()  # a plain address must not be null
    # the same as one launch
    copies = (capi.Segment * 1)(capi.Segment(0xc0000, 0xd0000, 4096))
    segs[1] = capi.Segment(0x100, 0xb0000, 4096)
    rows[1] = capi.Offer(capi.OFFER_STAGED, capi.OFFER_SLOT_OUTBOX, 0, 0, 64)
    a2a = lambda sy, stage=copies, ns=1, mine=rows, exp=expect, offers=two, imports=tab: L.mccl_alltoall_sync_offers(
        stage, ns, segs, from_, 2, ctypes.byref(sy), mine, exp, vp(0x1000), offers, imports, None)
    assert a2a(behind) == -1 and "max_compute_units" in err()
    assert a2a(opening) == -1 and "max_compute_units" in err()
    assert a2a(one, mine=None) == -1 and "null" in err()
    assert a2a(one, exp=None) == -1 and "null" in err()
    assert a2a(one, imports=vp(0x40004)) == -1 and "8-byte" in err()
    assert a2a(one, ns=9) == -1 and "0 to 8 segments" in err()
    assert a2a(one, stage=(capi.Segment * 1)(capi.Segment(0, 0xd0000, 4096))) == -1 and "outboxes: segment 0 has a null pointer" in err()
    assert a2a(one, offers=capi.ptr_table([0x10000, 0x20004])) == -1 and "offer pointer 1" in err()
    rows[0] = capi.Offer(40, 0, 7, 0, 64)
    assert a2a(one) == -1 and "offer 0 names entry 40" in err()
    # the small allreduce with its epoch on the device
    stage = capi.ptr_table([0x100000, 0x300000])
    tf = capi.ptr_table([0x500000, 0x510000])
    call = lambda state, ss, fs, flags, count=1024: L.mccl_allreduce_fused_replayable(
        vp(0x600000), vp(0x600000), count, capi.F32, capi.SUM, stage, tf, ss, fs, state, 2, 0, 0, None, 0, flags, None)
    assert call(None, 1 << 20, 8192, 0) == -1 and "state is null" in err()
    assert call(vp(0x700020), 1 << 20, 8192, 0) == -1 and "64-byte" in err()
    assert call(vp(0x700000), (1 << 20) + 8, 8192, 0) == -1 and "multiple of 16" in err()
    assert call(vp(0x700000), 1 << 20, 8190, 0) == -1 and "multiple of 4" in err()
    assert call(vp(0x700000), 2048, 8192, 0) == -1 and "does not fit" in err()
    assert call(vp(0x700000), 1 << 20, 8192, 4) == -1 and "unknown flags" in err()
    assert call(vp(0x700000), 1 << 20, 8192, capi.FUSED_WORK_ONLY | capi.FUSED_SYNC_ONLY) == -1 and "exclude each other" in err()
    assert call(vp(0x700000), 1 << 20, 8192, 0, count=0) == 0  # empty message: no launch


def test_pack_and_unpack_reject_a_null_flat_buffer(mccl):
    from torch_ccl_amd import capi
    L = capi.lib()
    tab = capi.ptr_table([0x1000, 0x2000])
    sizes = (ctypes.c_size_t * 2)(16, 16)
    assert L.mccl_pack(tab, sizes, 2, None, None) == -1
    assert L.mccl_unpack(None, tab, sizes, 2, None) == -1
    zero = (ctypes.c_size_t * 2)(0, 0)
    assert L.mccl_pack(tab, zero, 2, None, None) == 0


def test_alignment_and_range_errors_need_no_device(mccl):
    """Every refusal that depends on addresses, sizes or enum values only."""
    from torch_ccl_amd import capi
    L = capi.lib()
    err = lambda: L.mccl_last_error().decode()
    vp = ctypes.c_void_p
    two = capi.ptr_table([0x10000, 0x20000])
    # element alignment of inputs and output
    assert L.mccl_reduce_n(capi.ptr_table([0x10000, 0x20002]), 2, vp(0x30000), 64, capi.F32, capi.SUM, 0, None) == -1
    assert "input pointer 1 not aligned" in err()
    assert L.mccl_reduce_n(two, 2, vp(0x30001), 64, capi.BF16, capi.SUM, 0, None) == -1
    assert "output pointer not aligned" in err()
    assert L.mccl_reduce_n(two, 2, vp(0x30000), 64, capi.F32, capi.SUM, 9, None) == -1 and "variant" in err()
    assert L.mccl_reduce_n(capi.ptr_table([0x10000, 0]), 2, vp(0x30000), 64, capi.F32, capi.SUM, 0, None) == -1
    assert "input pointer 1 is null" in err()
    # shard and bucket ranges
    outs = capi.ptr_table([0x30000])
    assert L.mccl_reduce_scatter_n(two, 2, outs, 16, -1, 1, capi.F32, capi.SUM, None) == -1 and "negative shard" in err()
    assert L.mccl_reduce_scatter_n(two, 2, outs, 16, 0, 0, capi.F32, capi.SUM, None) == 0  # nothing to do
    assert L.mccl_reduce_multi(two, 2, outs, (ctypes.c_size_t * 1)(4), -3, capi.F32, capi.SUM, None) == -1
    # alltoallv: negative splits, rank count
    splits = (ctypes.c_int64 * 4)(1, -1, 0, 2)
    assert L.mccl_alltoallv_n(two, two, 2, splits, 16, None) == -1 and "negative split" in err()
    assert L.mccl_alltoallv_n(two, two, 0, splits, 16, None) == -1 and "rank count" in err()
    assert L.mccl_allgather_n(two, 65, vp(0x30000), 16, None) == -1
    # copies: a null end of a non-empty segment
    seg = (capi.Segment * 2)(capi.Segment(0x10000, 0x20000, 16), capi.Segment(0x10000, None, 16))
    assert L.mccl_copy_segments(seg, 2, None) == -1 and "segment 1 has a null pointer" in err()
    # gather: index table alignment, row length, row counts
    assert L.mccl_gather_rows(vp(0x10000), 10, vp(0x20004), 5, 64, vp(0x30000), None) == -1 and "8-byte aligned" in err()
    assert L.mccl_gather_rows(vp(0x10000), 10, vp(0x20000), 5, 1 << 31, vp(0x30000), None) == -1 and "too long" in err()
    assert L.mccl_gather_rows(vp(0x10000), 1 << 32, vp(0x20000), 5, 64, vp(0x30000), None) == -1 and "too many rows" in err()
    assert L.mccl_gather_rows(None, 10, vp(0x20000), 5, 64, vp(0x30000), None) == -1 and "null pointer" in err()
    assert L.mccl_gather_rows(None, 10, None, 0, 64, None, None) == 0
    # combine: dtype, top-k range, row length, alignment of every operand
    x = capi.ptr_table([0x10000, 0x20000])
    rows = (ctypes.c_size_t * 2)(8, 8)
    args = lambda **kw: [kw.get("x", x), rows, 2, vp(kw.get("rank", 0x40000)), vp(kw.get("row", 0x50000)), vp(kw.get("w", 0x60000)),
                         4, kw.get("topk", 2), kw.get("hidden", 64), kw.get("dtype", capi.BF16), vp(kw.get("y", 0x70000)), None]
    assert L.mccl_moe_combine(*args(dtype=capi.I32)) == -3 and "bf16, f16 and f32" in err()
    assert L.mccl_moe_combine(*args(topk=0)) == -1 and L.mccl_moe_combine(*args(topk=65)) == -1 and "topk" in err()
    assert L.mccl_moe_combine(*args(hidden=63)) == -3 and "multiple of 16 bytes" in err()
    assert L.mccl_moe_combine(*args(y=0x70008)) == -1 and "output is not 16-byte aligned" in err()
    assert L.mccl_moe_combine(*args(x=capi.ptr_table([0x10000, 0x20008]))) == -1 and "input 1 is not 16-byte aligned" in err()
    assert L.mccl_moe_combine(*args(row=0x50004)) == -1 and "misaligned" in err()
    assert L.mccl_moe_combine(*args(w=0x60002)) == -1 and "misaligned" in err()


def test_tensor_front_end_rejects_cpu_tensors(mccl):
    import torch
    with pytest.raises(RuntimeError, match="must be on the GPU"):
        mccl.reduce_n([torch.zeros(4), torch.zeros(4)])


def test_product_tree_never_touches_the_oracle():
    """The oracle is the checker; nothing that ships may import, load or call it."""
    offenders = []
    for base, _, files in os.walk(PKG):
        for name in files:
            if name.endswith((".py", ".hip", ".cpp", ".h", ".hpp")):
                text = open(os.path.join(base, name), errors="ignore").read()
                if re.search(r"\boracle\b", text):
                    offenders.append(os.path.join(base, name))
    assert not offenders, offenders


def test_isa_guard_flags_nothing():
    """Compiles the device code to assembly and scans for the stale-SCC select pattern."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("check_isa", os.path.join(PKG, "csrc", "check_isa.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert mod.main() == 0


def test_placement_check_needs_no_device(mccl):
    """The advisory placement test flags equal spacings of 256 MiB and more that are multiples of
    2 MiB on large messages (what a caching allocator gives equal tensors of 1 GiB and more), and
    nothing else: small messages, irregular spacings, the same spacing 4 KiB further apart."""
    from torch_ccl_amd import capi
    L = capi.lib()
    GiB, MiB = 1 << 30, 1 << 20
    base = 0x7f0000000000

    def check(spacings, nbytes):
        ptrs, p = [], base
        for d in [0] + list(spacings):
            p += d
            ptrs.append(p)
        return L.mccl_placement_check(capi.ptr_table(ptrs), len(ptrs), nbytes)

    assert check([GiB + 2 * MiB] * 7, GiB) == 1
    assert check([256 * MiB] * 7, 256 * MiB) == 1
    assert check([-(GiB + 2 * MiB)] * 7, GiB) == 1            # descending addresses too
    assert check([GiB + 2 * MiB + 4096] * 7, GiB) == 0         # staggered
    assert check([GiB + 2 * MiB] * 6 + [GiB + 4 * MiB], GiB) == 0  # not regular
    assert check([66 * MiB] * 7, 64 * MiB) == 0                # small messages have not shown the effect
    assert check([GiB + 2 * MiB] * 7, 64 * MiB) == 0
    assert L.mccl_placement_check(None, 8, GiB) == 0


def test_ctypes_structures_match_the_header(mccl, tmp_path):
    """The ctypes mirrors of the header's structures have the compiler's size and field offsets
    (a plain-C program that includes include/mccl.h prints them)."""
    import subprocess
    from torch_ccl_amd import capi
    layouts = {"mccl_xsync_t": (capi.XSync, [f[0] for f in capi.XSync._fields_]),
               "mccl_segment_t": (capi.Segment, [f[0] for f in capi.Segment._fields_]),
               "mccl_offer_t": (capi.Offer, [f[0] for f in capi.Offer._fields_]),
               "mccl_import_table_t": (capi.ImportTable, [f[0] for f in capi.ImportTable._fields_]),
               "mccl_import_update_t": (capi.ImportUpdate, [f[0] for f in capi.ImportUpdate._fields_])}
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "mccl.h"', 'int main(void) {']
    for cname, (_, fields) in layouts.items():
        lines.append('  printf("%s %%zu", sizeof(%s));' % (cname, cname))
        for f in fields:
            lines.append('  printf(" %%zu", offsetof(%s, %s));' % (cname, f))
        lines.append('  printf("\\n");')
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    for line in filter(None, out):
        cname, size, *offsets = line.split()
        ctype, fields = layouts[cname]
        assert ctypes.sizeof(ctype) == int(size), cname
        assert [getattr(ctype, f).offset for f in fields] == [int(o) for o in offsets], cname
