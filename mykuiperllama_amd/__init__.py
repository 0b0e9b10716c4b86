"""MI355X-native INT4 AWQ dequantise+GEMV path behind the kuiper matmul operator.

The product is native code: HIP kernels with a C ABI (include/kx_hip.h, csrc/) and the C++ host
API that mirrors the kuiper tensor / allocator / layer interfaces (kuiper/).  The Python in this
package is plumbing for tests and the benchmark: a ctypes binding and seeded input generators.
"""
from . import synth  # noqa: F401

__all__ = ["synth", "capi", "build"]
