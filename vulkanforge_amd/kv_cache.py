"""Host mirror of the reference's ``KvCache`` (src/backend/vulkan/kv_cache.rs), over the C ABI."""
from __future__ import annotations

import ctypes as C
import enum
from dataclasses import dataclass
from typing import Optional, Sequence

from . import _ffi


class KvDtype(enum.IntEnum):
    """kv_cache.rs:42-74."""
    F32 = 0
    F16 = 1
    F8 = 2

    def element_size(self) -> int:
        return {KvDtype.F32: 4, KvDtype.F16: 2, KvDtype.F8: 1}[self]

    def label(self) -> str:
        return {KvDtype.F32: "FP32", KvDtype.F16: "FP16", KvDtype.F8: "FP8"}[self]


@dataclass
class KvCacheConfig:
    """kv_cache.rs:153-174; the dtype is explicit here instead of coming from the environment."""
    n_layers: int
    n_kv_heads: int
    head_dim: int
    max_seq_len: int
    per_layer_head_dim: Optional[Sequence[int]] = None
    per_layer_n_kv_heads: Optional[Sequence[int]] = None
    dtype: KvDtype = KvDtype.F16


def _u32_array(values):
    if values is None:
        return None, None
    arr = (C.c_uint32 * len(values))(*values)
    return arr, C.cast(arr, C.POINTER(C.c_uint32))


def kv_bytes_per_token(n_layers, n_kv_heads, head_dim, per_layer_head_dim, per_layer_n_kv_heads, elem_size) -> int:
    """kv_cache.rs:186-202."""
    _a, pa = _u32_array(per_layer_head_dim)
    _b, pb = _u32_array(per_layer_n_kv_heads)
    return int(_ffi.lib().vfkv_kv_bytes_per_token(n_layers, n_kv_heads, head_dim, pa, pb, elem_size))


def guard_kv_precision(is_gemma4_moe: bool, kv_dtype: KvDtype, force: bool = False) -> None:
    """kv_cache.rs:118-151: raises for the known-broken non-FP8 gemma-4-MoE combination."""
    _ffi.check(_ffi.lib().vfkv_guard_kv_precision(int(is_gemma4_moe), int(kv_dtype), int(force)))


KV_OWN, KV_OWN_PUBLISHES_SLIDING, KV_OWN_PUBLISHES_FULL, KV_SUBSCRIBES_SLIDING, KV_SUBSCRIBES_FULL = range(5)


def gemma4_kv_read_layer(kv_source: Optional[Sequence[int]], layer: int) -> int:
    """forward/arch/gemma4.rs:27-49: the layer whose KV slab ``layer`` reads (one KV_* value per layer)."""
    _a, pa = _u32_array(kv_source)
    return int(_ffi.lib().vfkv_kv_read_layer(pa, 0 if kv_source is None else len(kv_source), layer))


def build_kv_sources(is_sliding: Sequence[bool], first_kv_shared: int, n_layers: int) -> list:
    """gguf.rs:908-942: one KV_* value per layer from the sliding / full pattern."""
    pat = (C.c_uint8 * max(len(is_sliding), 1))(*[1 if b else 0 for b in is_sliding])
    out = (C.c_uint32 * max(n_layers, 1))()
    _ffi.lib().vfkv_build_kv_sources(pat, len(is_sliding), first_kv_shared, n_layers, out)
    return list(out)[:n_layers]


def prefix_reuse_start(cached_tokens: Sequence[int], tokens: Sequence[int]) -> int:
    """server/state.rs:49-51,199-201: common prefix of the two sequences, capped at len(tokens) - 1."""
    _a, pa = _u32_array(list(cached_tokens))
    _b, pb = _u32_array(list(tokens))
    return int(_ffi.lib().vfkv_prefix_reuse_start(pa, len(cached_tokens), pb, len(tokens)))


class KvCache:
    """Two device buffers (K and V) in pos-major layout plus the offset arithmetic.

    ``KvCache(config)`` allocates on the current HIP device (KvCache::new).  ``layout_only=True``
    builds the same object without buffers, for hosts without a GPU.
    """

    def __init__(self, config: KvCacheConfig, layout_only: bool = False, k_buffer: int = 0, v_buffer: int = 0):
        L = _ffi.lib()
        if config.per_layer_head_dim is not None and len(config.per_layer_head_dim) != config.n_layers:
            raise ValueError("per_layer_head_dim length must equal n_layers")      # kv_cache.rs:246-249
        if config.per_layer_n_kv_heads is not None and len(config.per_layer_n_kv_heads) != config.n_layers:
            raise ValueError("per_layer_n_kv_heads length must equal n_layers")    # kv_cache.rs:252-255
        self.config = config
        self.kv_dtype = KvDtype(config.dtype)
        self._hd, phd = _u32_array(config.per_layer_head_dim)
        self._kvh, pkvh = _u32_array(config.per_layer_n_kv_heads)
        cfg = _ffi.CacheConfig(config.n_layers, config.n_kv_heads, config.head_dim, config.max_seq_len, phd, pkvh,
                               int(config.dtype))
        handle = C.c_void_p()
        if layout_only or k_buffer or v_buffer:
            _ffi.check(L.vfkv_cache_create_external(C.byref(cfg), k_buffer or None, v_buffer or None, C.byref(handle)))
        else:
            _ffi.check(L.vfkv_cache_create(C.byref(cfg), C.byref(handle)))
        self._h = handle

    # -- lifetime --
    def destroy(self) -> None:
        if getattr(self, "_h", None):
            _ffi.lib().vfkv_cache_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass

    @property
    def handle(self):
        return self._h

    # -- state --
    @property
    def current_seq_len(self) -> int:
        return int(_ffi.lib().vfkv_cache_current_seq_len(self._h))

    @current_seq_len.setter
    def current_seq_len(self, n: int) -> None:
        _ffi.lib().vfkv_cache_set_current_seq_len(self._h, n)

    def reset(self) -> None:
        _ffi.lib().vfkv_cache_reset(self._h)

    def zero_fill(self, stream: int = 0) -> None:
        _ffi.check(_ffi.lib().vfkv_cache_zero_fill(self._h, stream or None))

    def zero_layer(self, layer: int, stream: int = 0) -> None:
        _ffi.check(_ffi.lib().vfkv_cache_zero_layer(self._h, layer, stream or None))

    # -- buffers --
    @property
    def k_ptr(self) -> int:
        return int(_ffi.lib().vfkv_cache_k_ptr(self._h) or 0)

    @property
    def v_ptr(self) -> int:
        return int(_ffi.lib().vfkv_cache_v_ptr(self._h) or 0)

    def bytes_per_buffer(self) -> int:
        return int(_ffi.lib().vfkv_cache_bytes_per_buffer(self._h))

    # -- layout (kv_cache.rs:412-490) --
    def head_dim_for(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_head_dim_for(self._h, layer))

    def kv_heads_for(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_kv_heads_for(self._h, layer))

    def layer_offset_elems(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_layer_offset_elems(self._h, layer))

    def pos_offset_bytes(self, layer: int, pos: int) -> int:
        return int(_ffi.lib().vfkv_cache_pos_offset_bytes(self._h, layer, pos))

    def row_bytes(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_row_bytes(self._h, layer))

    def layer_offset_bytes(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_layer_offset_bytes(self._h, layer))

    def layer_size_bytes(self, layer: int) -> int:
        return int(_ffi.lib().vfkv_cache_layer_size_bytes(self._h, layer))

    def is_fp8(self) -> bool:
        return self.kv_dtype == KvDtype.F8

    def is_fp16(self) -> bool:
        return self.kv_dtype == KvDtype.F16
