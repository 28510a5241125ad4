"""Builds the native pieces in-tree for gfx950.

  libmi355ccl.so   HIP kernels + C ABI (include/mccl.h); depends on the HIP runtime only.
  libmcclbench.so  HIP-event timing loops around that ABI (bench/mccl_bench.h; lands in bench/).
  _C.*.so          the c10d backend (process_group_ccl.cpp: the group and how a collective runs;
                   pg_sharing.cpp: staging, shared allocations, standing offers; pg_collectives.cpp;
                   pg_p2p.cpp) and its Python module; host code only, links torch's c10d and
                   libmi355ccl.so.

Usage: python torch-ccl_amd/csrc/build.py [--force]
Outputs land in torch-ccl_amd/torch_ccl_amd/lib/.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(os.path.dirname(HERE), "torch_ccl_amd", "lib")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

KERNEL_SRC = os.path.join(HERE, "mccl_kernels.hip")          # planning, C ABI, copy and MoE kernels
REDUCE_SRC = os.path.join(HERE, "mccl_reduce_dtype.hip")     # reduction kernels, one object per dtype
REDUCE_DTYPES = range(9)                                      # mccl_dtype_t codes
KERNEL_LIB = os.path.join(LIB_DIR, "libmi355ccl.so")
KERNEL_HDRS = [os.path.join(INCLUDE, "mccl.h")] + [
    os.path.join(HERE, h) for h in ("kernels_common.hpp", "kernels_reduce.hpp", "kernels_copy.hpp",
                                    "kernels_moe.hpp", "kernels_sync.hpp", "kernels_fused.hpp", "kernels_xrank.hpp", "reduce_launch.hpp")]

# -ffp-contract=off / no fast-math: the reduction chain must round add by add.
# packed-fp32 ops are switched off for all device code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I", INCLUDE,
]


def _stale(out, srcs):
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    return any(os.path.getmtime(s) > t for s in srcs)


def kernel_units():
    """(source, extra flags, tag) of every translation unit of libmi355ccl.so."""
    units = [(KERNEL_SRC, [], "main")]
    units += [(REDUCE_SRC, ["-DMCCL_REDUCE_DT=%d" % dt], "dt%d" % dt) for dt in REDUCE_DTYPES]
    return units


def _run_parallel(cmds, jobs=8):
    """Runs the command lines concurrently; raises with the first failure."""
    from concurrent.futures import ThreadPoolExecutor
    def run(cmd):
        p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        return cmd, p.returncode, p.stdout
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(run, cmds))
    for cmd, rc, out in results:
        if rc != 0:
            sys.stderr.write(out)
            raise subprocess.CalledProcessError(rc, cmd)


def build_kernels(force=False, extra_flags=(), out=KERNEL_LIB):
    os.makedirs(os.path.dirname(out), exist_ok=True)
    if not (force or _stale(out, [KERNEL_SRC, REDUCE_SRC] + KERNEL_HDRS)):
        return out
    obj_dir = out + ".objs"
    os.makedirs(obj_dir, exist_ok=True)
    objs, cmds = [], []
    for src, flags, tag in kernel_units():
        obj = os.path.join(obj_dir, tag + ".o")
        objs.append(obj)
        cmds.append([HIPCC] + HIP_FLAGS + list(flags) + list(extra_flags) + ["-c", "-o", obj, src])
    _run_parallel(cmds)
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    for obj in objs:
        os.remove(obj)
    os.rmdir(obj_dir)
    return out


BENCH_DIR = os.path.join(ROOT, "bench")
BENCH_SRC = os.path.join(BENCH_DIR, "mccl_bench.cpp")
BENCH_LIB = os.path.join(BENCH_DIR, "libmcclbench.so")


def build_bench(force=False):
    srcs = [BENCH_SRC, os.path.join(BENCH_DIR, "mccl_bench.h"), os.path.join(INCLUDE, "mccl.h"), KERNEL_LIB]
    if force or _stale(BENCH_LIB, srcs):
        cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", INCLUDE, "-I", BENCH_DIR, "-o", BENCH_LIB, BENCH_SRC,
               "-L", LIB_DIR, "-lmi355ccl", "-Wl,-rpath,$ORIGIN/../torch-ccl_amd/torch_ccl_amd/lib"]
        subprocess.check_call(cmd)
    return BENCH_LIB


BACKEND_SRCS = [os.path.join(HERE, f) for f in ("process_group_ccl.cpp", "pg_sharing.cpp", "pg_collectives.cpp", "pg_p2p.cpp", "python_module.cpp")]
BACKEND_HDRS = [os.path.join(HERE, "process_group_ccl.hpp"), os.path.join(HERE, "pg_internal.hpp"), os.path.join(INCLUDE, "mccl.h")]


def backend_lib_path():
    import sysconfig
    return os.path.join(os.path.dirname(LIB_DIR), "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_backend(force=False):
    """The c10d backend is host-only C++ (no device code): g++ against torch's headers."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ext
    out = backend_lib_path()
    if not (force or _stale(out, BACKEND_SRCS + BACKEND_HDRS)):
        return out
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for d in ext.include_paths("cuda") + [sysconfig.get_paths()["include"], INCLUDE, HERE]:
        inc += ["-isystem" if "torch" in d or "rocm" in d or "python" in d else "-I", d]
    objs, cmds = [], []
    for src in BACKEND_SRCS:
        obj = os.path.join(LIB_DIR, os.path.basename(src) + ".o")
        cmds.append(["g++", "-c", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unknown-pragmas",
                     "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
                     "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)] + inc + ["-o", obj, src])
        objs.append(obj)
    _run_parallel(cmds)
    cmd = ["g++", "-shared", "-o", out] + objs + [
        "-L", torch_lib, "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python", "-lc10_hip", "-ltorch_hip",
        "-lamdhip64", "-L", LIB_DIR, "-lmi355ccl", "-lrt", "-lpthread",
        "-Wl,-rpath,$ORIGIN/lib", "-Wl,-rpath," + torch_lib]
    subprocess.check_call(cmd)
    for obj in objs:
        os.remove(obj)
    return out


C_CALLER_SRC = os.path.join(ROOT, "tests", "c_abi", "caller.c")
C_CALLER_BIN = os.path.join(ROOT, "tests", "c_abi", "caller")


def build_c_caller(force=False):
    """The plain-C host of tests/c_abi: gcc in C mode against include/mccl.h and the HIP runtime's
    C API; proves that the boundary needs no C++ and no torch."""
    if force or _stale(C_CALLER_BIN, [C_CALLER_SRC, os.path.join(INCLUDE, "mccl.h"), KERNEL_LIB]):
        subprocess.check_call(["gcc", "-std=c11", "-O1", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__=1",
                               "-I", INCLUDE, "-isystem", "/opt/rocm/include", "-o", C_CALLER_BIN, C_CALLER_SRC,
                               "-L", LIB_DIR, "-lmi355ccl", "-L", "/opt/rocm/lib", "-lamdhip64",
                               "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,$ORIGIN/../../torch-ccl_amd/torch_ccl_amd/lib",
                               "-Wl,-rpath,/opt/rocm/lib"])
    return C_CALLER_BIN


def build_all(force=False):
    return [build_kernels(force), build_bench(force), build_backend(force), build_c_caller(force)]


def stale_outputs():
    """Built libraries that are older than one of their sources."""
    checks = [(KERNEL_LIB, [KERNEL_SRC, REDUCE_SRC] + KERNEL_HDRS),
              (BENCH_LIB, [BENCH_SRC, os.path.join(BENCH_DIR, "mccl_bench.h")]),
              (backend_lib_path(), BACKEND_SRCS + BACKEND_HDRS)]
    return [out for out, srcs in checks if os.path.exists(out) and _stale(out, srcs)]


def ensure_built():
    """Builds only what does not exist yet: for tests, smoke() and bench.py, which use the libraries
    that are there and compile only when nothing is.  A library older than its sources is used as
    it is, with a warning on stderr, so that an edit without a rebuild does not pass unnoticed."""
    for out in stale_outputs():
        sys.stderr.write("warning: %s is older than its sources; run `python torch-ccl_amd/csrc/build.py`\n" % out)
    built = []
    if not os.path.exists(KERNEL_LIB):
        built.append(build_kernels(force=True))
    if not os.path.exists(BENCH_LIB):
        built.append(build_bench(force=True))
    if not os.path.exists(backend_lib_path()):
        built.append(build_backend(force=True))
    if not os.path.exists(C_CALLER_BIN):
        built.append(build_c_caller(force=True))
    return built


if __name__ == "__main__":
    for path in build_all(force="--force" in sys.argv):
        print(path)
