"""saga_amd - MI355X (gfx950) compute backend for the Saga graph/program API.

The product is native: `lib/libsaga_hip.so` (HIP kernels behind the C ABI of
include/saga_hip.h) and `lib/libsaga.so` (the C++ front end and the "hip" engine).  The Python
modules here are thin ctypes bindings used by the tests and by bench.py; torch only provides
device memory and streams.
"""
from . import kernels  # noqa: F401
