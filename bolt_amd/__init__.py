"""MI355X (gfx950) implementation of Bolt's quantized matrix-product path.

`capi` declares the C-ABI of libbolt_gfx950.so; `host` mirrors the reference's call sequences on
top of it. All computation happens in the HIP library.
"""
from . import capi  # noqa: F401
