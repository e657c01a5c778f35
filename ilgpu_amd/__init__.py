"""MI355X-native (gfx950) implementation of ILGPU.Algorithms' data-parallel
primitives: radix sort (keys, pairs), scan, reduce and histogram.

The product is the C-ABI shared library built from ``csrc/`` (declared in
``include/ilgpu_hip_algorithms.h``) plus the C++ host layer in ``host/`` that
mirrors the reference's C# surface.  ``capi`` is a ctypes binding of the same
C ABI used by the tests and the benchmark; torch only supplies device memory
and streams there.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
