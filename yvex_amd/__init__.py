"""yvex_amd: MI355X (gfx950) backend for YVEX's quantized-weight matmul path.

The product is ``libyvex_rocm.so`` (HIP kernels + a C11 host layer behind a C ABI, declared in
``include/yvex_rocm.h`` and ``include/yvex_rocm_kernels.h``). This package only loads that
library for Python callers (tests, the benchmark); it holds no compute path of its own and
raises if the library is missing instead of falling back to anything.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libyvex_rocm.so")

_lib = None


class LibraryMissing(RuntimeError):
    pass


def load_library() -> ctypes.CDLL:
    """Load the in-tree shared library. Never builds, never falls back."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is not built; run `python -m yvex_amd.build` "
                "(hipcc cross-compiles gfx950 without a GPU)")
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib
