"""Import-name compatibility: code written for the reference does
`import torch; import oneccl_bindings_for_pytorch` and then uses backend "ccl"
(README.md:176-190 of the reference).  With this directory on sys.path the same two lines load the
MI355X library and register the same backend name; nothing else lives here."""
import os

import torch_ccl_amd
from torch_ccl_amd import ProcessGroupCCL, __version__  # noqa: F401

cwd = os.path.dirname(os.path.abspath(torch_ccl_amd.__file__))

__all__ = ["ProcessGroupCCL", "is_available"]


def is_available(tensors):
    """True when the tensors could take part in one collective call: all contiguous and no two on
    the same device (oneccl_bindings_for_pytorch/__init__.py:38-49 of the reference)."""
    seen = set()
    for t in tensors:
        if not t.is_contiguous() or t.get_device() in seen:
            return False
        seen.add(t.get_device())
    return True
