"""Tensor-level front end of the C ABI: the N "peer" buffers are N torch tensors on one GPU.

These functions only marshal pointers and sizes; the work is done by the HIP kernels in
libmi355ccl.so on the current torch stream.  Argument checks follow the reference's
(src/utils.cpp:217-255: contiguous, same dtype) with the device test inverted: tensors must
live on the GPU.
"""
import ctypes

import torch

from . import capi


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check_tensors(tensors, what):
    first = tensors[0]
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("%s: tensors must be on the GPU (got %s)" % (what, t.device))
        if not t.is_contiguous():
            raise RuntimeError("input dense tensor has to be contiguous")
        if t.dtype != first.dtype:
            raise RuntimeError("Tensors are not equal in data type")
        if t.device != first.device:
            raise RuntimeError("%s: tensors must share one device" % what)


def _dtype_code(dtype):
    try:
        return capi.TORCH_DTYPE[dtype]
    except KeyError:
        raise RuntimeError("unsupported data type %s" % dtype) from None


def reduce_n(inputs, out=None, op=capi.SUM, variant=capi.VARIANT_AUTO):
    """out[i] = inputs[0][i] op ... op inputs[N-1][i] in ascending rank order.
    out may be one of the inputs (the in-place allreduce of the reference)."""
    if out is None:
        out = torch.empty_like(inputs[0])
    _check_tensors(list(inputs) + [out], "reduce_n")
    count = out.numel()
    for t in inputs:
        if t.numel() != count:
            raise RuntimeError("reduce_n: all buffers must have the same number of elements")
    with torch.cuda.device(out.device):
        rc = capi.lib().mccl_reduce_n(capi.ptr_table([t.data_ptr() for t in inputs]), len(inputs),
                                      out.data_ptr(), count, _dtype_code(out.dtype), op, variant,
                                      _stream())
    capi.check(rc)
    return out


_placement_warned = False


def placement_check(tensors):
    """True when the rank buffers sit at a spacing measured to cost 6-10 % of bandwidth on large
    reductions (see mccl_placement_check); `staggered_copies` / `empty_staggered` avoid it."""
    if len(tensors) < 2:
        return False
    nbytes = tensors[0].numel() * tensors[0].element_size()
    return bool(capi.lib().mccl_placement_check(capi.ptr_table([t.data_ptr() for t in tensors]), len(tensors), nbytes))


def _warn_about_placement(tensors):
    global _placement_warned
    if not _placement_warned and placement_check(tensors):
        _placement_warned = True
        import warnings
        warnings.warn("torch_ccl_amd: the rank buffers of this reduction sit at a regular spacing that costs 6-10 % of "
                      "HBM bandwidth on MI355X (DRAM bank conflicts); torch_ccl_amd.staggered_copies / empty_staggered "
                      "place them 4 KiB further apart per rank", stacklevel=3)


def reduce_scatter_n(inputs, outputs, op=capi.SUM, shard_first=0):
    """outputs[s] = reduction over ranks of inputs[k][(shard_first+s)*M : (shard_first+s+1)*M]."""
    _check_tensors(list(inputs) + list(outputs), "reduce_scatter_n")
    m = outputs[0].numel()
    for o in outputs:
        if o.numel() != m:
            raise RuntimeError("reduce_scatter_n: shard outputs must have equal sizes")
    for t in inputs:
        if t.numel() < (shard_first + len(outputs)) * m:
            raise RuntimeError("input tensor must be the same size as output size times world size")
    _warn_about_placement(inputs)
    with torch.cuda.device(outputs[0].device):
        rc = capi.lib().mccl_reduce_scatter_n(
            capi.ptr_table([t.data_ptr() for t in inputs]), len(inputs),
            capi.ptr_table([o.data_ptr() for o in outputs]), m, shard_first, len(outputs),
            _dtype_code(outputs[0].dtype), op, _stream())
    capi.check(rc)
    return outputs


def reduce_multi(input_lists, outputs, op=capi.SUM):
    """Coalesced reductions: input_lists[b] is the list of N rank buffers of bucket b."""
    n = len(input_lists[0])
    flat = []
    for b, ins in enumerate(input_lists):
        if len(ins) != n:
            raise RuntimeError("reduce_multi: every bucket needs the same rank count")
        _check_tensors(list(ins) + [outputs[b]], "reduce_multi")
        for t in ins:
            if t.numel() != outputs[b].numel():
                raise RuntimeError("reduce_multi: bucket %d size mismatch" % b)
            flat.append(t.data_ptr())
    for o in outputs:
        if o.dtype != outputs[0].dtype:
            raise RuntimeError("Tensors are not equal in data type")
    with torch.cuda.device(outputs[0].device):
        rc = capi.lib().mccl_reduce_multi(
            capi.ptr_table(flat), n, capi.ptr_table([o.data_ptr() for o in outputs]),
            capi.size_table([o.numel() for o in outputs]), len(outputs),
            _dtype_code(outputs[0].dtype), op, _stream())
    capi.check(rc)
    return outputs


def allgather_n(inputs, out):
    """out[k*M:(k+1)*M] = inputs[k]."""
    _check_tensors(list(inputs) + [out], "allgather_n")
    m = inputs[0].numel()
    for t in inputs:
        if t.numel() != m:
            raise RuntimeError("allgather_n: inputs must have equal sizes")
    if out.numel() != m * len(inputs):
        raise RuntimeError("output tensor size must be equal to world_size times input tensor size")
    with torch.cuda.device(out.device):
        rc = capi.lib().mccl_allgather_n(capi.ptr_table([t.data_ptr() for t in inputs]), len(inputs),
                                         out.data_ptr(), m * out.element_size(), _stream())
    capi.check(rc)
    return out


def alltoallv_n(inputs, outputs, split_rows):
    """All ranks' alltoall(v): split_rows[r][d] = dim-0 rows rank r sends to rank d."""
    _check_tensors(list(inputs) + list(outputs), "alltoallv_n")
    n = len(inputs)
    S = torch.as_tensor(split_rows, dtype=torch.int64).reshape(n, n).contiguous()
    row_bytes = None
    for t in list(inputs) + list(outputs):
        if t.numel():
            rb = t.numel() // t.shape[0] * t.element_size()
            if row_bytes is None:
                row_bytes = rb
            elif rb != row_bytes:
                raise RuntimeError("alltoallv_n: all tensors need the same row length")
    if row_bytes is None:
        return outputs
    for r in range(n):
        if inputs[r].shape[0] != int(S[r].sum()):
            raise RuntimeError("Tensor's dim 0 does not match sum of splits")
        if outputs[r].shape[0] != int(S[:, r].sum()):
            raise RuntimeError("Tensor's dim 0 does not match sum of splits")
    with torch.cuda.device(outputs[0].device):
        rc = capi.lib().mccl_alltoallv_n(capi.ptr_table([t.data_ptr() for t in inputs]),
                                         capi.ptr_table([t.data_ptr() for t in outputs]), n,
                                         ctypes.c_void_p(S.data_ptr()), row_bytes, _stream())
    capi.check(rc)
    return outputs


def copy_segments(segments):
    """segments: iterable of (src_ptr, dst_ptr, nbytes); raw device addresses, so the copy runs on the
    current stream of the current device (the other front ends switch to their tensors' device)."""
    segs = list(segments)
    arr = (capi.Segment * len(segs))(*[capi.Segment(s, d, b) for (s, d, b) in segs])
    capi.check(capi.lib().mccl_copy_segments(arr, len(segs), _stream()))


def pack(srcs, dst):
    """dst = concatenation of the flattened srcs (byte-exact)."""
    _check_tensors(list(srcs) + [dst], "pack")
    sizes = [t.numel() * t.element_size() for t in srcs]
    if sum(sizes) != dst.numel() * dst.element_size():
        raise RuntimeError("pack: destination size does not match the sources")
    with torch.cuda.device(dst.device):
        capi.check(capi.lib().mccl_pack(capi.ptr_table([t.data_ptr() for t in srcs]),
                                        capi.size_table(sizes), len(srcs), dst.data_ptr(), _stream()))
    return dst


def unpack(src, dsts):
    """Inverse of pack: scatter consecutive byte ranges of src into dsts."""
    _check_tensors([src] + list(dsts), "unpack")
    sizes = [t.numel() * t.element_size() for t in dsts]
    if sum(sizes) != src.numel() * src.element_size():
        raise RuntimeError("unpack: source size does not match the destinations")
    with torch.cuda.device(src.device):
        capi.check(capi.lib().mccl_unpack(src.data_ptr(), capi.ptr_table([t.data_ptr() for t in dsts]),
                                          capi.size_table(sizes), len(dsts), _stream()))
    return dsts


def _row_bytes(t):
    return (t.numel() // t.shape[0] if t.shape[0] else 0) * t.element_size()


def gather_rows(src, row_index, out=None):
    """out[j] = src[row_index[j]] (token permute); row_index is an int64 tensor on the GPU."""
    _check_tensors([src] + ([out] if out is not None else []), "gather_rows")
    if row_index.dtype != torch.int64 or not row_index.is_cuda or not row_index.is_contiguous():
        raise RuntimeError("gather_rows: row_index must be a contiguous int64 tensor on the GPU")
    if out is None:
        out = torch.empty((row_index.numel(),) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
    if out.shape[0] != row_index.numel() or tuple(out.shape[1:]) != tuple(src.shape[1:]):
        raise RuntimeError("gather_rows: output shape does not match the index and the source rows")
    rb = (src.numel() // src.shape[0] if src.shape[0] else 0) * src.element_size()
    with torch.cuda.device(src.device):
        capi.check(capi.lib().mccl_gather_rows(src.data_ptr(), src.shape[0], row_index.data_ptr(),
                                               row_index.numel(), rb, out.data_ptr(), _stream()))
    return out


def moe_dispatch_n(hidden, row_index, outputs, split_rows):
    """Fused token permute + alltoallv for all ranks: outputs[d] segment r = hidden[r][row_index[r][...]]."""
    _check_tensors(list(hidden) + list(outputs), "moe_dispatch_n")
    n = len(hidden)
    S = torch.as_tensor(split_rows, dtype=torch.int64).reshape(n, n).contiguous()
    rb = None
    for t in list(hidden) + list(outputs):
        if t.numel():
            b = _row_bytes(t)
            if rb is None:
                rb = b
            elif b != rb:
                raise RuntimeError("moe_dispatch_n: all tensors need the same row length")
    if rb is None:
        return outputs
    for r in range(n):
        ix = row_index[r]
        if ix.dtype != torch.int64 or not ix.is_cuda or not ix.is_contiguous():
            raise RuntimeError("moe_dispatch_n: row_index must be contiguous int64 tensors on the GPU")
        if ix.numel() != int(S[r].sum()):
            raise RuntimeError("moe_dispatch_n: row_index[%d] does not match the split sizes" % r)
        if outputs[r].shape[0] != int(S[:, r].sum()):
            raise RuntimeError("Tensor's dim 0 does not match sum of splits")
    with torch.cuda.device(outputs[0].device):
        capi.check(capi.lib().mccl_moe_dispatch_n(
            capi.ptr_table([t.data_ptr() for t in hidden]), capi.size_table([t.shape[0] for t in hidden]),
            capi.ptr_table([t.data_ptr() for t in row_index]), capi.ptr_table([t.data_ptr() for t in outputs]),
            n, ctypes.c_void_p(S.data_ptr()), rb, _stream()))
    return outputs


def moe_combine(x, src_rank, src_row, weights, out=None):
    """out[t] = sum_k weights[t, k] * x[src_rank[t, k]][src_row[t, k]] with fp32 accumulation."""
    _check_tensors(list(x) + ([out] if out is not None else []), "moe_combine")
    tokens, topk = weights.shape
    for t, dt in ((src_rank, torch.int32), (src_row, torch.int64), (weights, torch.float32)):
        if t.dtype != dt or not t.is_cuda or not t.is_contiguous() or tuple(t.shape) != (tokens, topk):
            raise RuntimeError("moe_combine: src_rank int32, src_row int64, weights fp32, all [tokens, topk] on the GPU")
    hidden = x[0].numel() // x[0].shape[0] if x[0].shape[0] else 0
    if out is None:
        out = torch.empty((tokens, hidden), dtype=x[0].dtype, device=x[0].device)
    with torch.cuda.device(out.device):
        capi.check(capi.lib().mccl_moe_combine(
            capi.ptr_table([t.data_ptr() for t in x]), capi.size_table([t.shape[0] for t in x]), len(x),
            src_rank.data_ptr(), src_row.data_ptr(), weights.data_ptr(), tokens, topk, hidden,
            _dtype_code(out.dtype), out.data_ptr(), _stream()))
    return out


def route_counts(expert_ids, n_experts, workspace=None, out=None):
    """counts[e] = number of entries of expert_ids (int32, on the GPU) equal to e, as an int64 tensor
    on the GPU; ids outside [0, n_experts) are ignored.  The per-rank sums of it are the split
    sizes of the dispatch all_to_all_single."""
    if expert_ids.dtype != torch.int32 or not expert_ids.is_cuda or not expert_ids.is_contiguous():
        raise RuntimeError("route_counts: expert_ids must be a contiguous int32 tensor on the GPU")
    if workspace is None:
        workspace = torch.empty(n_experts, dtype=torch.int32, device=expert_ids.device)
    if workspace.dtype != torch.int32 or workspace.numel() < n_experts or not workspace.is_cuda:
        raise RuntimeError("route_counts: workspace must hold n_experts int32 counters on the GPU")
    if out is None:
        out = torch.empty(n_experts, dtype=torch.int64, device=expert_ids.device)
    with torch.cuda.device(out.device):
        capi.check(capi.lib().mccl_route_counts(expert_ids.data_ptr(), expert_ids.numel(), n_experts,
                                                workspace.data_ptr(), out.data_ptr(), _stream()))
    return out


def empty_staggered(n, shape, dtype, device="cuda", stagger_bytes=4096):
    """n uninitialised tensors of one shape carved from a single allocation, buffer k starting
    stagger_bytes past the end of buffer k-1 (rounded up to 256 bytes): rank buffers allocated this
    way never sit at one of the spacings that map element i of every rank to the same DRAM bank
    (which is where a caching allocator puts equal tensors of 1 GiB and more)."""
    numel = 1
    for d in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,)):
        numel *= int(d)
    nbytes = numel * torch.empty(0, dtype=dtype).element_size()
    offs, pos = [], 0
    for k in range(n):
        pos = (pos + (stagger_bytes if k else 0) + 255) // 256 * 256
        offs.append(pos)
        pos += nbytes
    slab = torch.empty(max(pos, 1), dtype=torch.uint8, device=device)
    return [slab[off:off + nbytes].view(dtype).view(shape) for off in offs]


def staggered_copies(tensors, stagger_bytes=4096):
    """Copies of `tensors` carved from one allocation so that buffer k starts k * stagger_bytes past
    the end of buffer k-1 (rounded up to 256 bytes).  Rank buffers that sit an exact power of two
    apart (what a caching allocator tends to hand out for equal sizes) make every wavefront's loads
    hit the same DRAM banks at the same time; measured cost 6-20 % of bandwidth, gone with a 4 KiB
    stagger.  For callers who place the rank buffers themselves."""
    _check_tensors(list(tensors), "staggered_copies")
    sizes = [t.numel() * t.element_size() for t in tensors]
    offs, pos = [], 0
    for k, sz in enumerate(sizes):
        pos = (pos + (stagger_bytes if k else 0) + 255) // 256 * 256
        offs.append(pos)
        pos += sz
    slab = torch.empty(pos, dtype=torch.uint8, device=tensors[0].device)
    out = []
    for t, off, sz in zip(tensors, offs, sizes):
        v = slab[off:off + sz].view(t.dtype).view(t.shape)
        v.copy_(t)
        out.append(v)
    return out
