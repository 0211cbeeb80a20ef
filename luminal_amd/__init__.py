"""luminal_amd — MI355X (gfx950) quantized-matmul backend for Luminal.

The product is the C-ABI shared library ``libluminal_hip.so`` built from
``csrc/`` (hand-written HIP kernels; header in ``include/luminal_hip.h``).
This package holds its build recipe, a ctypes binding, and a thin host-side
mirror of the reference's quantized operators used by the tests and the
benchmark.  There is no CPU fallback: every operator raises if the library has
not been built.
"""
from . import capi  # noqa: F401
from .capi import LhipError, load_library  # noqa: F401

__version__ = "0.1.0"
