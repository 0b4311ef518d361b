"""MI355X (gfx950) implementation of the SMaLL layer hot path.

csrc/      hand-written HIP kernels + the C ABI (include/small_hip.h) -> lib/libsmall_hip.so
capi.py    ctypes binding of that ABI
layout.py  packed-layout helpers (numpy)
synth.py   seeded synthetic tensors
models.py  the benchmark topologies expressed as sequences of layer calls
"""
from . import capi, layout, synth  # noqa: F401

__all__ = ["capi", "layout", "synth"]
