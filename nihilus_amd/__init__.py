"""MI355X (gfx950) implementation of Nihilus's Q8_0 mat-mul hot path.

``csrc/`` holds the HIP kernels and their C ABI (``include/nihilus_amd/q8_0_abi.h``);
``q8_0`` wraps that ABI for torch-held device memory; the C++23 dispatch surface is
``include/nihilus_amd/mul_mat_dispatch.hpp``.
"""
from . import _lib  # noqa: F401
from ._lib import Q8Error  # noqa: F401

__all__ = ["Q8Error", "q8_0", "build"]
