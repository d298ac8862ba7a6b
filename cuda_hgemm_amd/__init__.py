"""MI355X (gfx950) half-precision GEMM library -- Python binding of the C ABI.

The product is the native library ``lib/libhgemm.so`` (hand-written HIP kernels behind
``include/hgemm.h``) and the C++ driver ``bin/hgemm``.  This package only loads the
library through ctypes so that tests and the benchmark can call the same entry points a
C++ caller links against.  PyTorch is used for device memory and nothing else.

There is no fallback: if the library has not been built, importing a symbol raises.
"""
from .binding import (HgemmLibrary, VendorLibrary, hgemm, library, vendor_library, lib_path,  # noqa: F401
                      vendor_lib_path, driver_path)

__all__ = ["HgemmLibrary", "VendorLibrary", "hgemm", "library", "vendor_library", "lib_path", "vendor_lib_path",
           "driver_path"]
