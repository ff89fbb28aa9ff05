"""MI355X-native execution and fingerprint-verification backend for Mirage mugraphs.

The product is native: HIP kernels for gfx950 behind the C ABI of
include/mi355_abi.h, and the mirage::kernel / mirage::threadblock C++ host API
above it.  This package holds their sources (csrc/), the build recipe, a ctypes
mirror of the host API (graph.py) and the workload catalogue (workloads.py).
"""
from . import workloads  # noqa: F401  (pure data, no native code needed)

__all__ = ["workloads"]
