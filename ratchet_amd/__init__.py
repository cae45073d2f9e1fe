"""ratchet_amd: MI355X (gfx950) device backend for ratchet-core's memory-bound tensor ops.

The product is the C ABI in include/ratchet_hip.h, implemented by hand-written HIP kernels in ratchet_amd/csrc and built
in-tree into ratchet_amd/libratchet_hip.so.  This package is the thin Python binding used by the tests and the benchmark.
"""
from . import _lib
from ._lib import RatchetError
from .runtime import Buffer, BufferView, Device, Event

__all__ = ["Device", "Buffer", "BufferView", "Event", "RatchetError", "_lib"]
