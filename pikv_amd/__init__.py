"""pikv_amd - PiKV's routed, compressed KV-cache data path on MI355X (gfx950).

The compute path is libpikv_hip.so (hand-written HIP kernels behind a C ABI,
include/pikv_hip.h).  `pikv_amd.ops` exposes it on torch tensors;
`pikv_amd.routing`, `.compression`, `.scheduling`, `.kernels`, `.moe`, `.attention`, `.pyramid`
mirror the reference's Python interfaces for this path.
"""
from . import _native  # noqa: F401

__version__ = "0.1.0"
