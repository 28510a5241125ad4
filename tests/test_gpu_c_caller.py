"""The C ABI from a host written in plain C (tests/c_abi/caller.c, built by build() with gcc in C
mode against include/mccl.h and the HIP runtime's C API): no C++, no torch, no Python between the
caller and libmi355ccl.so."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CALLER = os.path.join(HERE, "c_abi", "caller")


@pytest.mark.gpu
def test_plain_c_host_drives_the_library(mccl):
    assert os.path.exists(CALLER), "tests/c_abi/caller is not built; run __graft_entry__.build()"
    p = subprocess.run([CALLER], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert p.returncode == 0, (p.returncode, p.stdout, p.stderr)
    assert "c abi ok" in p.stdout


def test_plain_c_host_links_only_the_library_and_the_hip_runtime(mccl):
    """No GPU needed: the binary's dynamic dependencies name neither torch nor a C++ runtime of its own."""
    assert os.path.exists(CALLER), "tests/c_abi/caller is not built; run __graft_entry__.build()"
    out = subprocess.run(["readelf", "-d", CALLER], stdout=subprocess.PIPE, text=True, check=True).stdout
    needed = [line.split("[")[1].rstrip("]") for line in out.splitlines() if "(NEEDED)" in line]
    assert "libmi355ccl.so" in needed and any(n.startswith("libamdhip64") for n in needed), needed
    assert not any("torch" in n or "c10" in n or "stdc++" in n or "python" in n for n in needed), needed
