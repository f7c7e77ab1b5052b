"""MI355X-native paged KV-cache path with RichEngine's KV data-plane interface.

The product is ``libkvx.so`` (hand-written HIP kernels for gfx950 behind the C
ABI declared in ``include/kvx.h``).  This package only loads it and wraps the
calls for Python callers; torch supplies device memory and streams.
"""
from . import kvx  # noqa: F401
