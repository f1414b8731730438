"""MI355X (gfx950) implementation of the BlitzScale worker's paged-attention compute path.

The product is blitz_scale_amd/lib/libbz_hip.so (C ABI: include/bz_hip.h); `kernel` mirrors the
reference's blitz::kernel operator interface on top of it.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib", "kernel", "build"]
