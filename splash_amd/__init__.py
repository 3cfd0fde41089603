"""MI355X-native speculative-decoding verify step of Splash: Python bindings of the C ABI.

The product is ``splash_amd/lib/libsplash_hip.so`` (HIP backend, gfx950 kernels, C++ operators);
this package only binds it with ctypes. There is no CPU fallback: importing works without a GPU
(so the ABI can be inspected), but every call that computes needs the library and a device.
"""
from ._native import lib, library_path, SplashError, check  # noqa: F401
from .backend import Backend, Buffer, CommandGraph, STORAGE_PRIVATE, STORAGE_SHARED  # noqa: F401
from . import ops  # noqa: F401
from . import verify  # noqa: F401
