"""MI355X-native matmul path for dfdx: ctypes front-end over ``libdfdx_rocm.so``.

The product is the shared library (hand-written HIP kernels for gfx950 behind the
C ABI in ``include/dfdx_rocm.h``).  This package only loads it and mirrors, in
Python, the kernel-trait interface a dfdx device implements for ``matmul`` so
that tests and the benchmark read like the reference's own tests.  There is no
CPU fallback: if the library is missing or no gfx950 GPU is present, calls fail.
"""
from .rocm import DTYPES, Rocm, RocmError, View, lib_path, load_library  # noqa: F401
from .encoder import EncoderBlock  # noqa: F401
