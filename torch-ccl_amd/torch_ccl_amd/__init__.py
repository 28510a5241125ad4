"""MI355X-native collective data path behind the torch-ccl c10d API.

Importing this package
  * loads libmi355ccl.so (HIP kernels for gfx950 + C ABI) -- there is no CPU or eager
    fallback: if the library is missing the import fails;
  * registers the c10d backend "ccl" (and the alias "mccl") for ROCm tensors (device type
    "cuda") and exposes torch.distributed.ProcessGroupCCL, mirroring what
    `import oneccl_bindings_for_pytorch` does in the reference
    (oneccl_bindings_for_pytorch/csrc/init.cpp:123-154).
"""
import torch.distributed as _dist

from . import capi
from .capi import (AVG, MAX, MIN, PROD, SUM, VARIANT_AUTO, VARIANT_PERSISTENT,  # noqa: F401
                   VARIANT_SMALL, VARIANT_STREAM)
from .ops import (allgather_n, alltoallv_n, copy_segments, empty_staggered, gather_rows, moe_combine,  # noqa: F401
                  moe_dispatch_n, pack, placement_check, reduce_multi, reduce_n, reduce_scatter_n, route_counts, staggered_copies,
                  unpack)

capi.lib()  # fail loudly at import time when the native library is absent

from . import _C  # noqa: E402  (the c10d backend; needs libmi355ccl.so loaded first)

ProcessGroupCCL = _C.ProcessGroupCCL


def _register():
    for name in ("ccl", "mccl"):
        if name.upper() not in getattr(_dist.Backend, "backend_list", []) and \
                name not in getattr(_dist.Backend, "backend_list", []):
            _C.register(name)
    _dist.ProcessGroupCCL = ProcessGroupCCL


_register()

__version__ = "0.1.0"
