"""MI355X (gfx950) weight-only quantized linear path for cccc: Python access to the C-ABI library.

The product is libcccc_hip_quant.so (HIP kernels behind the `hip_*` C entry points declared in
include/cccc_hip_quant.h).  This package only loads it with ctypes so that tests, the smoke test and
the benchmark can call the same entry points a C++ host would.  There is no fallback: if the
library is missing, loading raises.

The directory name is not a Python identifier; load it as module `cccc_lite_amd` with
`__graft_entry__.load_package()`.
"""
from .capi import DataType, QuantLibrary, library, library_path  # noqa: F401
from . import host_api  # noqa: F401
