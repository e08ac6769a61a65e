"""MI355X (gfx950) implementation of MLcompiler's paged-KV attention hot path.

The product is the native library csrc/libmlc_hip.so (hand-written HIP kernels
behind the C ABI of include/mlc_hip.h) and the C++ HipExecutor above it.  This
package is the thin Python face of the same ABI, used by the tests and the
benchmark; it never falls back to a CPU or PyTorch implementation: if the
native library is missing or no gfx950 device is present, calls raise.
"""
from .executor import HipExecutor, NativeLibraryError  # noqa: F401

__all__ = ["HipExecutor", "NativeLibraryError"]
