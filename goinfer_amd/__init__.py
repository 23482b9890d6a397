"""goinfer_amd — MI355X (gfx950) decode backend for goinfer: hand-written HIP kernels behind a C ABI.

The product is goinfer_amd/lib/librocmdecode.so + rocmdecode_gfx950.hsaco (see include/rocmdecode.h).
This package is the thin Python harness over that C ABI used by the tests and the benchmark; it fails loudly
when the native library is missing or no GPU is present — there is no CPU fallback.
"""
from . import capi  # noqa: F401
