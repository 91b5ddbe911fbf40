"""blok_amd -- MI355X (gfx950) implementation of blok's kimi_exec forward hot path.

The product is the C-ABI library ``libkx.so`` (declared in ``include/kx.h``).
This package only locates and loads it; there is no Python fallback for any
operator, and loading fails loudly when the library has not been built.
"""
from .lib import KxError, DevBuf, kx, lib_path  # noqa: F401
