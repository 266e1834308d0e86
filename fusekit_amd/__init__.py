"""fusekit_amd: MI355X (gfx950) decode backend behind FuseKit's runtime interface.

The compute lives in libfusekit_hip.so (hand-written HIP, C ABI declared in
include/fusekit_hip.h).  This package is the thin host-side mirror of the
reference's Python-facing runtime; it never computes on the CPU.
"""
from . import native  # noqa: F401

__all__ = ["native"]
__version__ = "0.1.0"
