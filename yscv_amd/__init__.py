"""MI355X (gfx950) backend for YSCV's quantized-matmul path.

The product is the C-ABI library ``lib/libyscv_hip.so`` (sources in ``csrc/``, contract in
``include/yscv_hip.h``).  This package is the thin Python binding used by the tests, the
benchmark and the decode harness: it loads the library, checks status codes and passes raw
device pointers; it contains no arithmetic of its own and has no CPU fallback.
"""
from .capi import (  # noqa: F401
    BF16,
    F16,
    F32,
    NIBBLE_SIGNED,
    NIBBLE_UNSIGNED,
    ROUND_HALF_AWAY,
    ROUND_TIES_EVEN,
    YscvHipError,
    lib,
    library_path,
)
