"""Builds the native pieces in-tree for gfx950.

  libmi355ccl.so   HIP kernels + C ABI (include/mccl.h); depends on the HIP runtime only.
  libmcclbench.so  HIP-event timing loops around that ABI (include/mccl_bench.h).

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

KERNEL_SRC = os.path.join(HERE, "mccl_kernels.hip")
KERNEL_LIB = os.path.join(LIB_DIR, "libmi355ccl.so")

# -ffp-contract=off / no fast-math: the reduction chain must round add by add.
# packed-fp32 ops are switched off for all device code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
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


def build_kernels(force=False, extra_flags=(), out=KERNEL_LIB):
    os.makedirs(os.path.dirname(out), exist_ok=True)
    srcs = [KERNEL_SRC, os.path.join(INCLUDE, "mccl.h")]
    if force or _stale(out, srcs):
        cmd = [HIPCC] + HIP_FLAGS + list(extra_flags) + ["-o", out, KERNEL_SRC]
        subprocess.check_call(cmd)
    return out


BENCH_SRC = os.path.join(HERE, "mccl_bench.cpp")
BENCH_LIB = os.path.join(LIB_DIR, "libmcclbench.so")


def build_bench(force=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = [BENCH_SRC, os.path.join(INCLUDE, "mccl_bench.h"), os.path.join(INCLUDE, "mccl.h")]
    if force or _stale(BENCH_LIB, srcs):
        cmd = [HIPCC, "-x", "hip", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-I", INCLUDE, "-o", BENCH_LIB, BENCH_SRC,
               "-L", LIB_DIR, "-lmi355ccl", "-Wl,-rpath,$ORIGIN"]
        subprocess.check_call(cmd)
    return BENCH_LIB


def build_all(force=False):
    return [build_kernels(force), build_bench(force)]


if __name__ == "__main__":
    for path in build_all(force="--force" in sys.argv):
        print(path)
