"""iom_amd — MI355X (gfx950) backend for IOM's memory-bound tensor operations.

The product is `libiomx.so` (hand-written HIP kernels behind the C ABI of
`include/iomx.h`) plus the C++ `iom::Device` backend under `iom_amd/host/`.
This Python package is plumbing for tests and benchmarks: a ctypes binding of
the C ABI.  There is no CPU fallback: importing `iom_amd.iomx` fails when the
library has not been built.
"""
__all__ = ["iomx", "build"]
