"""MI355X-native FP8 hot path: ctypes access to libcf_fp8.so (hand-written HIP, gfx950).

The library is the product; this package only loads it and checks return codes.
There is no CPU fallback: if the shared library is missing, loading raises.
"""
from .native import CfError, Lib, lib, lib_path  # noqa: F401
