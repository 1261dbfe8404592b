"""MI355X (gfx950) implementation of the seblas fp32 GEMM / linear / convolution hot path.

The product is the C-ABI shared library ``lib/libcrusader_hip.so`` (declared in ``include/crusader_hip.h``)
and the C++ ``seblas`` / ``seann`` host layer built on it; ``capi`` is a ctypes binding used by the tests
and the benchmark.
"""
__all__ = ["capi"]
