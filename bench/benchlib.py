"""ctypes binding of libmcclbench.so: HIP-event timing loops around the C ABI
(mccl_bench.h beside this file).  Benchmark support; not needed to use the library."""
import ctypes
import os

import torch

from torch_ccl_amd import capi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmcclbench.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        capi.lib()
        if not os.path.exists(LIB_PATH):
            raise ImportError("libmcclbench.so is not built; run `python torch-ccl_amd/csrc/build.py`")
        L = ctypes.CDLL(LIB_PATH)
        vp, sz, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        L.mcclb_last_error.restype = ctypes.c_char_p
        L.mcclb_reduce_latency.argtypes = [vp, i32, vp, i32, sz, i32, i32, i32, vp, i32, i32, vp]
        L.mcclb_reduce_throughput.argtypes = [vp, i32, vp, i32, sz, i32, i32, i32, vp, i32, i32, vp]
        L.mcclb_loop_create.argtypes = [ctypes.POINTER(vp)]
        L.mcclb_loop_reduce.argtypes = [vp, vp, i32, vp, i32, sz, i32, i32, i32, vp, i32]
        L.mcclb_loop_elapsed_us.argtypes = [vp, vp]
        L.mcclb_loop_destroy.argtypes = [vp]
        L.mcclb_loop_destroy.restype = None
        L.mcclb_reduce_scatter_throughput.argtypes = [vp, i32, vp, sz, i32, i32, i32, i32, vp, i32, i32, vp]
        L.mcclb_copy_latency.argtypes = [vp, i32, vp, i32, i32, vp]
        L.mcclb_copy_throughput.argtypes = [vp, i32, vp, i32, i32, vp]
        L.mcclb_alltoallv_throughput.argtypes = [vp, vp, i32, vp, sz, vp, i32, i32, vp]
        L.mcclb_probe_stream.argtypes = [vp, i32, vp, i32, sz, i32, i32, vp, i32, i32, vp]
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError("mccl bench error %d: %s" % (rc, lib().mcclb_last_error().decode()))


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _sets(input_sets, outputs):
    n = len(input_sets[0])
    flat = [t.data_ptr() for s in input_sets for t in s]
    return n, capi.ptr_table(flat), capi.ptr_table([o.data_ptr() for o in outputs])


def reduce_latency(input_sets, outputs, op=capi.SUM, variant=capi.VARIANT_AUTO, warmup=100, iters=1000):
    """Per-call microseconds (list of floats); call i uses buffer set i % len(input_sets)."""
    n, ins, outs = _sets(input_sets, outputs)
    us = (ctypes.c_float * iters)()
    o = outputs[0]
    _check(lib().mcclb_reduce_latency(ins, n, outs, len(input_sets), o.numel(),
                                      capi.TORCH_DTYPE[o.dtype], op, variant, _stream(), warmup, iters, us))
    return list(us)


def reduce_throughput(input_sets, outputs, op=capi.SUM, variant=capi.VARIANT_AUTO, warmup=5, iters=20):
    """Average microseconds per call over `iters` back-to-back calls."""
    n, ins, outs = _sets(input_sets, outputs)
    total = ctypes.c_float(0)
    o = outputs[0]
    _check(lib().mcclb_reduce_throughput(ins, n, outs, len(input_sets), o.numel(),
                                         capi.TORCH_DTYPE[o.dtype], op, variant, _stream(), warmup, iters,
                                         ctypes.byref(total)))
    return total.value / iters


class ReduceLoop:
    """`iters` back-to-back calls of mccl_reduce_n with everything that is not a launch done up front:
    the library handle, the pointer tables and the event pair exist before the caller starts its
    clock.  run() only records, enqueues and records; elapsed_us() (after the caller's own
    synchronisation) is the time between the two events."""

    def __init__(self, input_sets, outputs, op=capi.SUM, variant=capi.VARIANT_AUTO):
        self._lib = lib()
        self._keep = (input_sets, outputs)
        self._n, self._ins, self._outs = _sets(input_sets, outputs)
        o = outputs[0]
        self._args = (len(input_sets), o.numel(), capi.TORCH_DTYPE[o.dtype], op, variant)
        self._h = ctypes.c_void_p()
        _check(self._lib.mcclb_loop_create(ctypes.byref(self._h)))
        self._stream = _stream()

    def run(self, iters):
        nsets, count, dtype, op, variant = self._args
        rc = self._lib.mcclb_loop_reduce(self._h, self._ins, self._n, self._outs, nsets, count, dtype, op, variant,
                                         self._stream, iters)
        if rc != 0:
            _check(rc)

    def elapsed_us(self):
        total = ctypes.c_float(0)
        _check(self._lib.mcclb_loop_elapsed_us(self._h, ctypes.byref(total)))
        return total.value

    def close(self):
        if self._h:
            self._lib.mcclb_loop_destroy(self._h)
            self._h = ctypes.c_void_p()


def reduce_scatter_throughput(inputs, outputs, shard_first=0, op=capi.SUM, warmup=3, iters=10):
    total = ctypes.c_float(0)
    o = outputs[0]
    _check(lib().mcclb_reduce_scatter_throughput(
        capi.ptr_table([t.data_ptr() for t in inputs]), len(inputs),
        capi.ptr_table([t.data_ptr() for t in outputs]), o.numel(), shard_first, len(outputs),
        capi.TORCH_DTYPE[o.dtype], op, _stream(), warmup, iters, ctypes.byref(total)))
    return total.value / iters


def _segs(segments):
    segs = list(segments)
    return (capi.Segment * len(segs))(*[capi.Segment(s, d, b) for (s, d, b) in segs]), len(segs)


def copy_latency(segments, warmup=100, iters=1000):
    arr, n = _segs(segments)
    us = (ctypes.c_float * iters)()
    _check(lib().mcclb_copy_latency(arr, n, _stream(), warmup, iters, us))
    return list(us)


def copy_throughput(segments, warmup=3, iters=10):
    arr, n = _segs(segments)
    total = ctypes.c_float(0)
    _check(lib().mcclb_copy_throughput(arr, n, _stream(), warmup, iters, ctypes.byref(total)))
    return total.value / iters


def alltoallv_throughput(inputs, outputs, split_rows, row_bytes, warmup=2, iters=5):
    n = len(inputs)
    S = torch.as_tensor(split_rows, dtype=torch.int64).reshape(n, n).contiguous()
    total = ctypes.c_float(0)
    _check(lib().mcclb_alltoallv_throughput(
        capi.ptr_table([t.data_ptr() for t in inputs]), capi.ptr_table([t.data_ptr() for t in outputs]), n,
        ctypes.c_void_p(S.data_ptr()), row_bytes, _stream(), warmup, iters, ctypes.byref(total)))
    return total.value / iters


def probe_stream(inputs, output, write, block=64, workgroups_per_cu=0, warmup=3, iters=20):
    """Bare streaming kernel of the bench library (no product code): reads len(inputs) buffers, writes
    `output` when `write`; returns microseconds per launch."""
    nbytes = output.numel() * output.element_size()
    total = ctypes.c_float(0)
    ins = capi.ptr_table([t.data_ptr() for t in inputs]) if inputs else None
    _check(lib().mcclb_probe_stream(ins, len(inputs), ctypes.c_void_p(output.data_ptr()), int(bool(write)), nbytes,
                                    block, workgroups_per_cu, _stream(), warmup, iters, ctypes.byref(total)))
    return total.value / iters
