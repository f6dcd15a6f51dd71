"""MI355X-native KV-cache / attention hot path behind the reference's dispatch interface.

The product is ``libvfkv.so`` (hand-written HIP for gfx950 behind the C ABI in ``include/vfkv.h``).
This package is the thin Python host side used by the tests and the benchmark: it mirrors the
reference's ``KvCache`` (src/backend/vulkan/kv_cache.rs) and ``Forward::run_*`` helpers
(src/backend/vulkan/forward/runs.rs), borrows device memory and streams from PyTorch, and forwards
everything through ctypes.  There is no CPU or eager fallback: importing works anywhere, calling a
compute entry point without the built library or without a GPU raises.
"""
from ._ffi import VfkvError, lib, lib_path  # noqa: F401
from .kv_cache import (KvCache, KvCacheConfig, KvDtype, guard_kv_precision, kv_bytes_per_token,  # noqa: F401
                       gemma4_kv_read_layer, build_kv_sources, prefix_reuse_start)
from .forward import Forward, Workspace  # noqa: F401

__all__ = ["KvCache", "KvCacheConfig", "KvDtype", "Forward", "Workspace", "VfkvError", "lib", "lib_path",
           "guard_kv_precision", "kv_bytes_per_token", "gemma4_kv_read_layer", "build_kv_sources", "prefix_reuse_start"]
