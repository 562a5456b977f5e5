"""granite_amd -- MI355X (gfx950) attention backend for Granite.

Holds only what the attention hot path needs: the HIP kernels and C ABI
(csrc/ -> lib/libgranite_hip.so), the C++ host layer that plugs them into
Granite's backend / compute / operator interfaces (host/), and a thin ctypes
mirror of that interface for tests and the benchmark.
"""
from ._capi import GraniteHipError, LIB_PATH  # noqa: F401
from .hip_compute import (DeviceBuffer, HipCompute, get_hip_compute, F16, F32, MASK_CAUSAL,  # noqa: F401
                          MASK_NONE, MASK_TREE, ROUND_NEAREST, ROUND_TRUNCATE)
