"""Guard against a code-generation hazard seen with hipcc on gfx950: a uniform 64-bit
compare + select lowered to `v_cmp_*_u64 vcc` ... `s_cselect_b32` where the instruction
that should turn vcc into SCC has been dropped, so the select consumes the carry bit of an
unrelated scalar add/sub.  The kernels avoid the source pattern (uniform 64-bit min/max);
this script compiles the device code to assembly and scans every kernel for a scalar
select or SCC branch whose nearest SCC writer in the same straight-line region is an
arithmetic instruction rather than a compare or mask operation.

The same scan enforces two numeric rules of the kernels: no packed-fp32 arithmetic
(v_pk_add/mul/fma_f32) anywhere, and no fused multiply-add outside the AVG kernels (whose
division by the rank count expands to a correctly rounded sequence that uses v_fma_f32): every
add and every product of the reduction chains must round on its own.  Scratch (register spill)
instructions are flagged as well.

A third scan audits the cache hints of the 16-byte vector accesses, which decide several percent
of bandwidth and which the compiler has dropped silently before (the `nt` of a non-temporal
store vanished on one path of the tile loop, and byte-typed kernels lost it on some loads): in the
reduction kernels every vector load must be non-temporal, each tile path must hold the
streaming store (a hand-written `sc1` instruction) beside the cacheable one, and that store must be
followed by the wait state the compiler cannot know it needs; the full-chunk
path of the copy kernel, the combine kernel and the stores of the row gather must be non-temporal.

A fourth scan covers the kernels that wait for other ranks inside a launch: each must use at most
128 vector registers, because the wavefront budget of all ranks (4096) is sized for four
wavefronts per SIMD -- with fewer, the waiting workgroups of seven ranks could fill the GPU and
keep the eighth rank's first workgroup out for good -- and the reduction among them must read the
peers' tensors with `buffer_load_dwordx4 ... sc0 sc1 nt` (coherent and streaming) and write
them back with `buffer_store_dwordx4 ... sc0 sc1`.

Usage: python torch-ccl_amd/csrc/check_isa.py   (exit status 1 if anything is flagged)
"""
import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as _build  # noqa: E402

_COMPARE = re.compile(r"^(s_cmp|s_cmpk|s_bitcmp|s_and_b|s_or_b|s_xor_b|s_andn2_b|s_orn2_b|s_lshr_b|s_bfe_|"
                      r"s_and_saveexec|s_or_saveexec|s_andn2_saveexec|s_not_b)")
_ARITH = re.compile(r"^(s_add_|s_sub_|s_addc_|s_subb_|s_lshl_b|s_ashr_|s_min_|s_max_|s_abs_|s_absdiff_|"
                    r"s_lshl[1-4]_add_)")
_USER = re.compile(r"^(s_cselect_|s_cbranch_scc)")
_PACKED = re.compile(r"^v_pk_(add|mul|fma)_f32")
_FMA = re.compile(r"^(v_fma_f32|v_fmac_f32|v_mad_f32|v_fma_f64|v_fmac_f64)")
_AVG_KERNEL = re.compile(r"(reduce_(vec|elem)_kernel|allreduce_fused_kernel|xrank_reduce_kernel)ILi\d+ELi1E")  # second template argument = MCCL_AVG
_SCRATCH = re.compile(r"^scratch_")


def device_asm(out_path):
    """Device assembly of every translation unit of the kernel library, concatenated into out_path."""
    flags = [f for f in _build.HIP_FLAGS if f != "-fPIC"] + ["-I", HERE]
    parts, cmds = [], []
    for src, extra, tag in _build.kernel_units():
        part = "%s.%s.s" % (out_path, tag)
        parts.append(part)
        cmds.append([_build.HIPCC] + flags + list(extra) + ["--cuda-device-only", "-S", "-o", part, src])
    _build._run_parallel(cmds)
    with open(out_path, "w") as out:
        for part in parts:
            with open(part) as f:
                out.write(f.read())
            os.remove(part)


def scan(asm_path):
    """Returns a list of (line_no, instruction, scc_source, function)."""
    flagged = []
    fn, last = None, None
    with open(asm_path) as f:
        for ln, line in enumerate(f, 1):
            t = line.strip()
            if not t or t.startswith(";"):
                continue
            if t.startswith(".LBB"):
                last = None  # SCC may arrive from another block: left alone
                continue
            if t.startswith("."):
                continue
            if re.match(r"^[A-Za-z_][\w.$]*:", t):
                fn, last = t.split(":")[0], None
                continue
            op = t.split()[0]
            if _PACKED.match(op):
                flagged.append((ln, t, "packed fp32 arithmetic", fn))
            if _FMA.match(op) and not _AVG_KERNEL.search(fn or ""):
                flagged.append((ln, t, "fused multiply-add outside the AVG kernels", fn))
            if _SCRATCH.match(op):
                flagged.append((ln, t, "scratch access (register spill)", fn))
            if _USER.match(op) and last is not None and _ARITH.match(last[0]):
                flagged.append((ln, t, last[1], fn))
            if _COMPARE.match(op) or _ARITH.match(op):
                last = (op, t)
    return flagged


_REDUCE_VEC = re.compile(r"reduce_vec_kernelILi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELb[01]E")


def _hint(instruction):
    """Cache-policy flags of a global load/store ('plain' if none)."""
    words = instruction.split(";")[0].replace(",", " ").split()
    flags = [w for w in words if w in ("sc0", "sc1", "nt")]
    return " ".join(flags) if flags else "plain"


def scan_hints(asm_path):
    """Returns a list of (function, problem) for vector accesses whose cache hint is not the intended one."""
    counts, fn, pending, unguarded = {}, None, None, []
    with open(asm_path) as f:
        for line in f:
            t = line.strip()
            m = re.match(r"^(_Z[\w.$]*):", t)
            if m:
                fn = m.group(1)
                continue
            if pending and t and not t.startswith((";", ".")):
                # the hand-written store carries its own wait state (the compiler cannot know it needs one)
                if not t.startswith("s_nop"):
                    unguarded.append((pending, "vector store of the reduction is not followed by s_nop"))
                pending = None
            if fn and _REDUCE_VEC.search(fn) and t.startswith("global_store_dwordx4") and _hint(t) == "sc1":
                pending = fn
            if fn and (t.startswith("global_load_dwordx4") or t.startswith("global_store_dwordx4")):
                t = t.split(";")[0].strip()
                key = ("load" if t.startswith("global_load") else "store", _hint(t))
                c = counts.setdefault(fn, {})
                c[key] = c.get(key, 0) + 1
    bad, seen_reduce = list(unguarded), 0
    for fn, c in counts.items():
        get = lambda kind, hint: c.get((kind, hint), 0)
        if _REDUCE_VEC.search(fn):
            seen_reduce += 1
            if get("store", "plain") != get("store", "sc1") or not get("store", "sc1"):
                bad.append((fn, "streamed (sc1) and cacheable vector stores do not pair up: %r" % c))
            if set(k for k in c if k[0] == "load") != {("load", "nt")}:
                bad.append((fn, "vector loads must all be nt: %r" % c))
            if set(k for k in c if k[0] == "store") != {("store", "plain"), ("store", "sc1")}:
                bad.append((fn, "unexpected vector store flavour: %r" % c))
        elif "moe_combine_kernel" in fn:
            if get("load", "plain") or get("store", "plain"):
                bad.append((fn, "combine kernel has vector accesses without nt: %r" % c))
        elif "gather_rows_kernel" in fn:
            if get("store", "plain"):
                bad.append((fn, "row gather has vector stores without nt: %r" % c))
        elif "copy_segments_kernel" in fn:
            # full chunks: nt loads; nt stores, or written-through (sc1) ones in the STREAM variants
            if get("load", "nt") < 2 or max(get("store", "nt"), get("store", "sc1")) < 2:
                bad.append((fn, "copy kernel lost its cache hints: %r" % c))
    if not seen_reduce:
        bad.append(("reduce_vec_kernel", "no reduction kernel recognised (name mangling changed?)"))
    return bad


_WAITING_KERNEL = re.compile(r"(xrank_reduce_kernel|copy_segments_sync_kernel|fanout_sync_kernel|fanout_indirect_kernel|allreduce_fused_kernel|"
                             r"rank_barrier_kernel|rank_barrier_offers_kernel|rank_barrier_offers_each_kernel|copy_segments_resolved_kernel|exchange_offers_kernel)")
_MAX_VGPRS_OF_WAITING_KERNELS = 128


def scan_waiting_kernels(asm_path):
    """Returns a list of (function, problem) for the kernels that wait for other ranks."""
    bad, seen, fn, acc = [], 0, None, {}
    with open(asm_path) as f:
        for line in f:
            t = line.strip()
            m = re.match(r"^(_Z[\w.$]*):", t)
            if m:
                fn = m.group(1)
                continue
            m = re.match(r"^\.set (_Z[\w.$]*)\.num_vgpr, (\d+)", t)
            if m and _WAITING_KERNEL.search(m.group(1)):
                seen += 1
                if int(m.group(2)) > _MAX_VGPRS_OF_WAITING_KERNELS:
                    bad.append((m.group(1), "%s vector registers: fewer than four wavefronts per SIMD" % m.group(2)))
            if fn and "xrank_reduce_kernel" in fn and t.startswith(("buffer_load_dwordx4", "buffer_store_dwordx4")):
                kind = "load" if t.startswith("buffer_load") else "store"
                acc.setdefault(fn, set()).add((kind, " ".join(sorted(_hint(t).split()))))
    for fn, kinds in acc.items():
        if kinds != {("load", "nt sc0 sc1"), ("store", "sc0 sc1")}:
            bad.append((fn, "coherent accesses of the cross-rank reduction changed flavour: %r" % sorted(kinds)))
    if not seen or not acc:
        bad.append(("xrank_reduce_kernel", "no waiting kernel recognised (name mangling changed?)"))
    return bad


def main():
    with tempfile.TemporaryDirectory() as d:
        asm = os.path.join(d, "mccl_kernels.s")
        device_asm(asm)
        flagged = scan(asm)
        hints = scan_hints(asm) + scan_waiting_kernels(asm)
    for fn, problem in hints:
        print("cache hint in %s: %s" % (fn, problem))
    print("cache hints flagged: %d" % len(hints))
    if hints:
        return 1
    for ln, ins, src, fn in flagged:
        print("line %d in %s: `%s` <- %s" % (ln, fn, ins, src))
    print("flagged: %d" % len(flagged))
    return 1 if flagged else 0


if __name__ == "__main__":
    sys.exit(main())
