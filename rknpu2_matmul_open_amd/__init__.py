"""MI355X-native quantized-linear hot path behind the rk_npu_* C API.

The product is ``librk_npu_matmul.so`` (HIP kernels + C++ host layer, built by
``rknpu2_matmul_open_amd.build``).  This package only locates and loads it and
mirrors the C structs for Python callers (tests, smoke check, benchmark).
There is no CPU fallback: loading fails loudly if the library is not built.
"""
from .capi import load_library, lib_path  # noqa: F401
