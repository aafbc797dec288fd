"""MI355X (gfx950) implementation of NeuZephyr's tensor-core GEMM path.

The product is ``libnzhip.so`` (hand-written HIP kernels behind the C-ABI declared in
``include/nzhip.h``) plus the C++ host layer that mirrors the ``nz::`` API.  This Python
package only carries the build driver and a ctypes view of the C-ABI used by the tests and
the benchmark; it contains no compute fallback: without the built library every call raises.
"""
from .capi import NzHipError, lib_path, load  # noqa: F401
