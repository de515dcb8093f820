"""MI355X (gfx950) inference kernels behind nnForge's layer_tester surface.

The product is the native library ``libnnforge_hip.so`` (hand-written HIP kernels behind the C ABI
declared in ``include/nnforge_hip.h``) and the C++ backend above it. This Python package only
holds the build recipe and a ctypes binding of that C ABI used by the tests and the benchmark;
it contains no arithmetic of its own and no CPU fallback.
"""

__all__ = ["build", "capi"]
