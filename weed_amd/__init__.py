"""weed_amd -- MI355X (gfx950) device layer for Weed's quantized-KV attention path.

The product is the C-ABI shared library `weed_amd/lib/libweed_hip.so` (declared in `include/weed_hip.h`).
This package only builds it (`weed_amd.build`) and binds it with ctypes (`weed_amd.capi`) for tests and
benchmarks; there is no CPU fallback: loading fails loudly when the library has not been built.
"""
from .build import build_library, library_path  # noqa: F401
