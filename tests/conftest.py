import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "torch-ccl_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def _ensure_built():
    """Use the native libraries that are there; compile only when nothing is built."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("mccl_build", os.path.join(ROOT, "torch-ccl_amd", "csrc", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.ensure_built()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    _ensure_built()


@pytest.fixture(scope="session")
def mccl():
    """The product package; importing it loads libmi355ccl.so or fails."""
    import torch_ccl_amd
    return torch_ccl_amd
