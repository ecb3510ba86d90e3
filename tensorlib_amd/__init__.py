"""tensorlib_amd: MI355X (gfx950) backend for tensorLib's matrix-multiplication hot path.

The product is the C-ABI shared library ``lib/libtensorlib_amd.so`` built from ``csrc/``
(declared in ``include/tensorlib_amd.h``).  This Python package is only the ctypes binding
used by the tests and the benchmark; it holds no compute of its own and has no CPU
fallback: every call fails loudly when the library or a GPU is missing.
"""
from ._lib import LIB_PATH, TensorLibError, build_library, lib  # noqa: F401
from .device import HipDevice  # noqa: F401

__all__ = ["HipDevice", "TensorLibError", "build_library", "lib", "LIB_PATH"]
