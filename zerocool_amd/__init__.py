"""MI355X-native implementation of ZeroCool's mixture-of-experts layer path.

The product is libzc_hip.so (hand-written HIP for gfx950 behind a C ABI,
include/zc_hip.h).  This package is the thin Python face of that ABI used by the
tests and the benchmark; it has no CPU fallback and raises if the library is missing.
"""
from .hip import Context, Config, Linear, Layer, Trace, StackTrace, Store, ZcError, load_library, LIB_PATH  # noqa: F401
