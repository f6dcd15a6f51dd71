"""Host mirror of the reference's dispatch helpers for this path (``Forward::run_*`` in
src/backend/vulkan/forward/runs.rs and the four executor steps in forward/executor/attention.rs).

Arguments are PyTorch CUDA(HIP) tensors or raw device pointers; PyTorch only supplies memory and
the stream.  Every method enqueues on ``stream`` (default: torch's current stream) and returns
without synchronising, like the reference records into an open command buffer.
"""
from __future__ import annotations

import ctypes as C
import math

from . import _ffi
from .kv_cache import KvCache, KvDtype

FA_TILE = 64  # runs.rs:766, flash_attn_split.comp:23-24


def _ptr(x) -> int:
    if x is None:
        return 0
    if isinstance(x, int):
        return x
    if not x.is_cuda:
        raise ValueError("expected a device tensor: this path has no CPU implementation")
    if not x.is_contiguous():
        raise ValueError("expected a contiguous tensor")
    return x.data_ptr()


def _stream(stream) -> int:
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


class Workspace:
    """fa_scratch_out / max / sum (forward/setup.rs:203-230)."""

    def __init__(self, n_heads: int, head_dim: int, max_seq_len: int):
        h = C.c_void_p()
        _ffi.check(_ffi.lib().vfkv_workspace_create(n_heads, head_dim, max_seq_len, C.byref(h)))
        self._h = h

    def destroy(self):
        if getattr(self, "_h", None):
            _ffi.lib().vfkv_workspace_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Forward:
    """The part of the reference's ``Forward`` that this path needs: a cache, a workspace, the head
    geometry, and the default ``attn_scale = 1/sqrt(head_dim)`` (forward/setup.rs:786)."""

    def __init__(self, kv_cache: KvCache, n_heads: int, workspace: Workspace | None = None):
        self.kv_cache = kv_cache
        self.n_heads = n_heads
        cfg = kv_cache.config
        max_hd = max(cfg.per_layer_head_dim) if cfg.per_layer_head_dim else cfg.head_dim
        self.workspace = workspace or Workspace(n_heads, max_hd, cfg.max_seq_len)
        self.attn_scale = 1.0 / math.sqrt(cfg.head_dim)

    # ---- KV append (runs.rs:2389-2478) ----
    @staticmethod
    def run_kv_store_fp8(src, dst, n_elements: int, dst_byte_offset: int, stream=None) -> None:
        _ffi.check(_ffi.lib().vfkv_store_fp8(_ptr(src), _ptr(dst), n_elements, dst_byte_offset, _stream(stream)))

    @staticmethod
    def run_kv_copy_fp16(src, dst, n_elements: int, dst_byte_offset: int, stream=None) -> None:
        _ffi.check(_ffi.lib().vfkv_copy_fp16(_ptr(src), _ptr(dst), n_elements, dst_byte_offset, _stream(stream)))

    @staticmethod
    def run_kv_fp8_to_f16(src, dst, n_elems: int, stream=None) -> None:
        """The conversion pass of run_flash_attn_cm_gemma_rs (runs.rs:1105-1137)."""
        _ffi.check(_ffi.lib().vfkv_fp8_to_f16(_ptr(src), _ptr(dst), n_elems, _stream(stream)))

    def step_kv_write(self, layer: int, position: int, k_src, v_src, stream=None) -> None:
        """executor/attention.rs:546-597 (one token)."""
        _ffi.check(_ffi.lib().vfkv_kv_write(self.kv_cache.handle, layer, position, 1, _ptr(k_src), _ptr(v_src),
                                            _stream(stream)))

    def b_step_kv_write(self, layer: int, base_pos: int, seq_len: int, batch_k, batch_v, stream=None) -> None:
        """executor/attention.rs:2134-2190 (seq_len tokens in one launch)."""
        _ffi.check(_ffi.lib().vfkv_kv_write(self.kv_cache.handle, layer, base_pos, seq_len, _ptr(batch_k),
                                            _ptr(batch_v), _stream(stream)))

    @staticmethod
    def run_rms_norm_mul_rope(qk, weight, qk_out, head_dim: int, rotary_dim: int, theta_scale: float,
                              heads_per_token: int, m: int, eps: float = 1e-6, positions=None, pos0: int = 0,
                              freq_factors=None, rope_mode: int = _ffi.ROPE_NEOX, freq_scale: float = 1.0,
                              attn_factor: float = 1.0, stream=None) -> None:
        """runs.rs:2492-2600 (``weight=None``: the plain run_rope_neox_with_pos_offset, runs.rs:647-720): per
        (token, head) row RMS-norm * weight, then RoPE with the token's position.  ``qk_out`` may be ``qk``."""
        p = _ffi.RopeParams(rope_mode, rotary_dim, theta_scale, freq_scale, attn_factor, eps)
        _ffi.check(_ffi.lib().vfkv_rms_norm_mul_rope(_ptr(qk), _ptr(weight), _ptr(qk_out), head_dim, heads_per_token, m,
                                                     _ptr(positions), pos0, _ptr(freq_factors), C.byref(p),
                                                     _stream(stream)))

    def step_k_rope_kv_write(self, layer: int, position: int, n_tokens: int, k_src, v_src, rotary_dim: int,
                             theta_scale: float, k_norm_weight=None, positions=None, freq_factors=None,
                             rope_mode: int = _ffi.ROPE_NEOX, freq_scale: float = 1.0, attn_factor: float = 1.0,
                             eps: float = 1e-6, k_out=None, stream=None) -> None:
        """step_k_norm_rope / step_k_rope followed by step_kv_write (executor/attention.rs:435-597; batch
        :2026-2190) in one launch: K is RMS-normalised * ``k_norm_weight`` (None: plain RoPE), rotated and stored in
        the cache dtype at ``position + t``; V is stored as ``step_kv_write`` stores it.  ``theta_scale`` =
        (1 / freq_base)^(2 / rotary_dim) (layer_plan.rs:532).  ``k_out`` (may be ``k_src``) receives the rotated K."""
        p = _ffi.RopeParams(rope_mode, rotary_dim, theta_scale, freq_scale, attn_factor, eps)
        _ffi.check(_ffi.lib().vfkv_k_rope_kv_write(
            self.kv_cache.handle, layer, position, n_tokens, _ptr(k_src), _ptr(v_src),
            _ptr(k_norm_weight) if k_norm_weight is not None else None,
            _ptr(positions) if positions is not None else None,
            _ptr(freq_factors) if freq_factors is not None else None, C.byref(p),
            _ptr(k_out) if k_out is not None else None, _stream(stream)))

    def step_qk_rope_kv_write(self, layer: int, position: int, n_tokens: int, q, k_src, v_src, rotary_dim: int,
                              theta_scale: float, q_norm_weight=None, k_norm_weight=None, q_out=None, positions=None,
                              freq_factors=None, rope_mode: int = _ffi.ROPE_NEOX, freq_scale: float = 1.0,
                              attn_factor: float = 1.0, eps: float = 1e-6, k_out=None, stream=None) -> None:
        """step_q_norm_rope + step_k_norm_rope + step_kv_write (executor/attention.rs:360-597) as one launch: the
        queries [n_tokens, n_heads, head_dim] are normed * ``q_norm_weight`` and rotated into ``q_out`` (default: in
        place), K and V as in ``step_k_rope_kv_write``."""
        p = _ffi.RopeParams(rope_mode, rotary_dim, theta_scale, freq_scale, attn_factor, eps)
        _ffi.check(_ffi.lib().vfkv_qk_rope_kv_write(
            self.kv_cache.handle, layer, position, n_tokens, self.n_heads, _ptr(q), _ptr(q_norm_weight),
            _ptr(q_out if q_out is not None else q), _ptr(k_src), _ptr(v_src), _ptr(k_norm_weight), _ptr(positions),
            _ptr(freq_factors), C.byref(p), _ptr(k_out), _stream(stream)))

    # ---- decode attention (runs.rs:722-822, 1463-1571) ----
    @staticmethod
    def run_flash_attn_split(q, k_layer, v_layer, kv_dtype, scratch_out, scratch_max, scratch_sum, n_heads,
                             n_kv_heads, head_dim, seq_len, scale, kv_start=0, tile=FA_TILE, softcap=0.0,
                             max_seq=0, stream=None, interleaved=False) -> int:
        """``interleaved=True`` calls vfkv_flash_attn_split_interleaved: same partial count, but partial j is
        not tile j (only the merged output is meaningful)."""
        n_tiles = (seq_len + tile - 1) // tile
        p = _ffi.SplitParams(n_heads, n_kv_heads, head_dim, seq_len, max_seq, scale, n_tiles, kv_start)
        fn = _ffi.lib().vfkv_flash_attn_split_interleaved if interleaved else _ffi.lib().vfkv_flash_attn_split
        _ffi.check(fn(_ptr(q), _ptr(k_layer), _ptr(v_layer), int(kv_dtype), _ptr(scratch_out), _ptr(scratch_max),
                      _ptr(scratch_sum), C.byref(p), tile, softcap, _stream(stream)))
        return n_tiles

    @staticmethod
    def run_flash_attn_reduce(scratch_out, scratch_max, scratch_sum, o, n_heads, head_dim, n_tiles,
                              stream=None) -> None:
        _ffi.check(_ffi.lib().vfkv_flash_attn_reduce(_ptr(scratch_out), _ptr(scratch_max), _ptr(scratch_sum),
                                                     _ptr(o), n_heads, head_dim, n_tiles, _stream(stream)))

    def run_scalar_attn(self, layer: int, position: int, q, o, kv_layer: int | None = None, kv_start: int = 0,
                        scale: float | None = None, softcap: float = 0.0, stream=None) -> None:
        """Decode router (runs.rs:722-822); scale defaults to 1/sqrt(head_dim_for(layer))."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        _ffi.check(_ffi.lib().vfkv_decode_attention(self.kv_cache.handle, layer,
                                                    layer if kv_layer is None else kv_layer, self.n_heads,
                                                    _ptr(q), _ptr(o), position, kv_start, scale, softcap,
                                                    self.workspace._h, _stream(stream)))

    step_attention = run_scalar_attn  # executor/attention.rs:599-625

    def run_scalar_attn_static(self, layer: int, position: int, q, o, kv_layer: int | None = None, kv_start: int = 0,
                               scale: float | None = None, softcap: float = 0.0, stream=None) -> None:
        """``run_scalar_attn`` without the workspace: vfkv_decode_attention_static keeps the partials in the library's
        static device array and allocates nothing (for callers under graph capture or in loops that must not allocate).
        Calls that overlap in time on one GPU race."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        _ffi.check(_ffi.lib().vfkv_decode_attention_static(self.kv_cache.handle, layer,
                                                           layer if kv_layer is None else kv_layer, self.n_heads,
                                                           _ptr(q), _ptr(o), position, kv_start, scale, softcap,
                                                           _stream(stream)))

    def step_kv_write_attention(self, layer: int, position: int, q, k_src, v_src, o, kv_start: int = 0,
                                scale: float | None = None, softcap: float = 0.0, stream=None) -> None:
        """step_kv_write + step_attention of one token (executor/attention.rs:546-625) as one call: where the
        decode worker can, it writes the new rows itself and the append launch disappears."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        _ffi.check(_ffi.lib().vfkv_kv_write_decode_attention(self.kv_cache.handle, layer, self.n_heads, _ptr(q),
                                                             _ptr(k_src), _ptr(v_src), _ptr(o), position, kv_start,
                                                             scale, softcap, self.workspace._h, _stream(stream)))

    def step_qk_rope_kv_write_attention(self, layer: int, position: int, q, k_src, v_src, o, rotary_dim: int, theta_scale: float,
                                        q_norm_weight=None, k_norm_weight=None, q_out=None, k_out=None, freq_factors=None,
                                        rope_mode: int = _ffi.ROPE_NEOX, freq_scale: float = 1.0, attn_factor: float = 1.0,
                                        eps: float = 1e-6, kv_start: int = 0, scale: float | None = None, softcap: float = 0.0,
                                        stream=None) -> None:
        """step_q_norm_rope + step_k_norm_rope + step_kv_write + step_attention of one decode token
        (executor/attention.rs:360-625) as one call: ``q`` and ``k_src`` are the rows before norm and rotation; where the
        decode worker can, it rotates them itself and no separate RoPE / append launch runs."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        p = _ffi.RopeParams(rope_mode, rotary_dim, theta_scale, freq_scale, attn_factor, eps)
        _ffi.check(_ffi.lib().vfkv_qk_rope_kv_write_decode_attention(
            self.kv_cache.handle, layer, self.n_heads, _ptr(q), _ptr(q_norm_weight), _ptr(q_out), _ptr(k_src), _ptr(v_src),
            _ptr(k_norm_weight), _ptr(freq_factors), C.byref(p), _ptr(k_out), _ptr(o), position, kv_start, scale, softcap,
            self.workspace._h, _stream(stream)))

    # ---- prefill attention (runs.rs:933-1010, executor/attention.rs:2192-2390) ----
    @staticmethod
    def run_flash_attn_batch(q, k_layer, v_layer, kv_dtype, o, n_heads, n_kv_heads, head_dim, m, q_start, n_kv,
                             scale, kv_start=0, softcap=0.0, stream=None, f16_weights=False, fp8_scores=False,
                             f16_queries=False) -> None:
        """``f16_weights=True``: vfkv_flash_attn_batch_opt with VFKV_PREFILL_F16_WEIGHTS (softmax weights rounded to f16
        in the second product: faster, output off by up to 2^-11 * max|v|)."""
        p = _ffi.BatchParams(n_heads, n_kv_heads, head_dim, m, n_kv, q_start, scale, kv_start)
        if f16_weights or fp8_scores or f16_queries:   # fp8_scores: VFKV_PREFILL_FP8_SCORES (first product on the FP8 matrix
            # instruction); f16_queries: VFKV_PREFILL_F16_QUERIES (queries rounded to f16: no remainder pass of the first product)
            opts = ((_ffi.PREFILL_F16_WEIGHTS if f16_weights else 0) | (_ffi.PREFILL_FP8_SCORES if fp8_scores else 0) |
                    (_ffi.PREFILL_F16_QUERIES if f16_queries else 0))
            _ffi.check(_ffi.lib().vfkv_flash_attn_batch_opt(_ptr(q), _ptr(k_layer), _ptr(v_layer), int(kv_dtype), _ptr(o),
                                                            C.byref(p), softcap, opts, _stream(stream)))
            return
        _ffi.check(_ffi.lib().vfkv_flash_attn_batch(_ptr(q), _ptr(k_layer), _ptr(v_layer), int(kv_dtype), _ptr(o),
                                                    C.byref(p), softcap, _stream(stream)))

    def b_step_attention(self, layer: int, base_pos: int, seq_len: int, q, o, kv_layer: int | None = None,
                         kv_start_window: int = 0, scale: float | None = None, softcap: float = 0.0,
                         stream=None, use_workspace: bool = False, f16_weights: bool = False,
                         fp8_scores: bool = False, f16_queries: bool = False) -> None:
        """``use_workspace=True``: vfkv_prefill_attention_ws (key chunks over workgroups for short chunks over long
        histories, merged through the decode workspace).  ``f16_weights=True``: vfkv_prefill_attention_opt with
        VFKV_PREFILL_F16_WEIGHTS."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        if f16_weights or fp8_scores or f16_queries:
            opts = ((_ffi.PREFILL_F16_WEIGHTS if f16_weights else 0) | (_ffi.PREFILL_FP8_SCORES if fp8_scores else 0) |
                    (_ffi.PREFILL_F16_QUERIES if f16_queries else 0))
            _ffi.check(_ffi.lib().vfkv_prefill_attention_opt(self.kv_cache.handle, layer,
                                                             layer if kv_layer is None else kv_layer, self.n_heads,
                                                             _ptr(q), _ptr(o), seq_len, base_pos, kv_start_window, scale,
                                                             softcap, opts,
                                                             self.workspace._h if use_workspace else None, _stream(stream)))
            return
        if use_workspace:
            _ffi.check(_ffi.lib().vfkv_prefill_attention_ws(self.kv_cache.handle, layer,
                                                            layer if kv_layer is None else kv_layer, self.n_heads,
                                                            _ptr(q), _ptr(o), seq_len, base_pos, kv_start_window, scale,
                                                            softcap, self.workspace._h, _stream(stream)))
            return
        _ffi.check(_ffi.lib().vfkv_prefill_attention(self.kv_cache.handle, layer,
                                                     layer if kv_layer is None else kv_layer, self.n_heads,
                                                     _ptr(q), _ptr(o), seq_len, base_pos, kv_start_window, scale,
                                                     softcap, _stream(stream)))

    # ---- gated attention output (runs.rs:2649-2681, executor/attention.rs:632-680, 2405-2444) ----
    @staticmethod
    def run_sigmoid_mul(gate, inout, ne: int, chunk: int, stride: int, gate_offset: int, stream=None) -> None:
        """inout[i] *= sigmoid(gate[(i // chunk) * stride + gate_offset + i % chunk]) for i < ne."""
        g = _ffi.Gate(_ptr(gate), chunk, stride, gate_offset)
        _ffi.check(_ffi.lib().vfkv_sigmoid_mul(C.byref(g), _ptr(inout), ne, _stream(stream)))

    def step_attn_gated_output(self, attn_out, q_buf, q_dim: int, stream=None) -> None:
        """executor/attention.rs:632-680: one token, the gate sits behind Q in ``q_buf``."""
        self.run_sigmoid_mul(q_buf, attn_out, q_dim, q_dim, q_dim, q_dim, stream)

    def b_step_attn_gated_output(self, batch_attn_out, batch_qgate, seq_len: int, head_dim: int, stream=None) -> None:
        """executor/attention.rs:2405-2444: per (token, head) the gate follows the head's Q in ``batch_qgate``."""
        self.run_sigmoid_mul(batch_qgate, batch_attn_out, seq_len * self.n_heads * head_dim, head_dim, 2 * head_dim, head_dim,
                             stream)

    def step_attention_gated(self, layer: int, position: int, q, o, gate, chunk: int, stride: int, gate_offset: int,
                             k_src=None, v_src=None, kv_layer: int | None = None, kv_start: int = 0,
                             scale: float | None = None, softcap: float = 0.0, stream=None) -> None:
        """(step_kv_write +) step_attention + step_attn_gated_output as one call: the merge applies the gate."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        g = _ffi.Gate(_ptr(gate), chunk, stride, gate_offset)
        _ffi.check(_ffi.lib().vfkv_decode_attention_gated(
            self.kv_cache.handle, layer, layer if kv_layer is None else kv_layer, self.n_heads, _ptr(q), _ptr(k_src),
            _ptr(v_src), _ptr(o), position, kv_start, scale, softcap, C.byref(g), self.workspace._h, _stream(stream)))

    def b_step_attention_gated(self, layer: int, base_pos: int, seq_len: int, q, o, gate, chunk: int, stride: int,
                               gate_offset: int, kv_layer: int | None = None, kv_start_window: int = 0,
                               scale: float | None = None, softcap: float = 0.0, stream=None) -> None:
        """b_step_attention + b_step_attn_gated_output."""
        if scale is None:
            hd = self.kv_cache.head_dim_for(layer)
            scale = self.attn_scale if hd == self.kv_cache.config.head_dim else 1.0 / math.sqrt(hd)
        g = _ffi.Gate(_ptr(gate), chunk, stride, gate_offset)
        _ffi.check(_ffi.lib().vfkv_prefill_attention_gated(
            self.kv_cache.handle, layer, layer if kv_layer is None else kv_layer, self.n_heads, _ptr(q), _ptr(o), seq_len,
            base_pos, kv_start_window, scale, softcap, C.byref(g), _stream(stream)))


__all__ = ["Forward", "Workspace", "KvDtype", "FA_TILE"]
