"""alignedkv_amd -- MI355X (gfx950) implementation of AlignedKV's split-precision KV cache and
decode attention.  The compute lives in libalignedkv_hip.so (hand-written HIP, C ABI declared in
include/alignedkv.h); this package holds the loader and the Python host layer that mirrors the
reference's extension/ and model/ modules."""

__all__ = ["build", "load_library"]

from ._lib import build, load_library  # noqa: E402
