"""skl_amd - Python binding of libskl_gfx950.so, the MI355X implementation of
SKL's gemm / pack / cvt entry points (see include/skl-gfx950.h).

The binding is plumbing for tests and benchmarks: it loads the shared library
with ctypes and exposes every C entry point under its C name. Array arguments
may be numpy arrays (ordinary host memory: the library stages them) or
:class:`DeviceBuffer` objects (device memory: asynchronous launch). There is no
CPU fallback: if the library is not built, importing the entry points fails.
"""
from .binding import (DeviceBuffer, Epilogue, LibraryNotBuilt, check_error, lib, library_path, load)  # noqa: F401
