"""MI355X (gfx950) fused-dequant GEMM and flash-decode attention.

The product is the C-ABI shared library lib/libw4amd.so (see include/w4_abi.h)
and the C++ headers under include/w4/.  `capi` is a thin ctypes view of the C
ABI that takes device pointers; it allocates nothing and has no CPU fallback.
"""
from . import capi  # noqa: F401
from .build import build  # noqa: F401
