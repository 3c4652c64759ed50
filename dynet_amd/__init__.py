"""dynet_amd: MI355X (gfx950) device layer and fused-layer kernels for DyNet's GPU path.

The product is ``libdynet_hip.so`` (hand-written HIP behind the C-ABI declared in
``include/dynet_hip.h``).  This package is the thin host side used by the tests
and the benchmark: ``lib`` binds the C-ABI with ctypes, ``device`` mirrors
DyNet's Device / pools / Tensor plumbing on top of it.  There is no CPU fallback:
importing works anywhere (so that the symbol table can be checked), but creating
a device without a GPU raises.
"""
from . import lib  # noqa: F401
from .device import Device, DevTensor, DyhipError, PinnedArray  # noqa: F401

__all__ = ["lib", "Device", "DevTensor", "DyhipError", "PinnedArray"]
