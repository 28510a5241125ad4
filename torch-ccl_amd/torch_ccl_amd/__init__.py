"""MI355X-native collective data path behind the torch-ccl c10d API.

Importing this package loads libmi355ccl.so (HIP kernels for gfx950 + C ABI).  The kernels
are the product; there is no CPU or eager fallback: if the library is missing the import
fails.
"""
from . import capi
from .capi import (AVG, MAX, MIN, PROD, SUM, VARIANT_AUTO, VARIANT_PERSISTENT,  # noqa: F401
                   VARIANT_SMALL, VARIANT_STREAM)
from .ops import (allgather_n, alltoallv_n, copy_segments, pack, reduce_multi,  # noqa: F401
                  reduce_n, reduce_scatter_n, unpack)

capi.lib()  # fail loudly at import time when the native library is absent

__version__ = "0.1.0"
