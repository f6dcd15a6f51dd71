// FFI declarations of libvfkv for the reference's Rust host (to live at src/backend/hip/ffi.rs there): one declaration per
// symbol of include/vfkv.h, same argument order.  Not compiled in this repository (no Rust toolchain in the build image);
// tests/test_abi_cpu.py checks the function names and argument counts against the header.
#![allow(non_camel_case_types, dead_code)]
use std::os::raw::{c_char, c_int, c_void};
#[repr(C)] pub struct VfkvCacheConfig {          // KvCacheConfig, kv_cache.rs:153-174
    pub n_layers: u32, pub n_kv_heads: u32, pub head_dim: u32, pub max_seq_len: u32,
    pub per_layer_head_dim: *const u32, pub per_layer_n_kv_heads: *const u32,
    pub dtype: u32,                               // 0 = F32, 1 = F16, 2 = F8E4M3 (KvDtype, kv_cache.rs:42-56)
}
#[repr(C)] pub struct VfkvSplitParams {           // FlashAttnSplitPushConstants, pipeline.rs:553-569
    pub n_heads: u32, pub n_kv_heads: u32, pub head_dim: u32, pub seq_len: u32,
    pub max_seq: u32, pub scale: f32, pub n_tiles: u32, pub kv_start: u32,
}
#[repr(C)] pub struct VfkvBatchParams {           // FlashAttnBatchPushConstants, pipeline.rs:592-611
    pub n_heads: u32, pub n_kv_heads: u32, pub head_dim: u32, pub m: u32,
    pub n_kv: u32, pub q_start: u32, pub scale: f32, pub kv_start: u32,
}
#[repr(C)] pub struct VfkvRopeParams {            // the fields of RopePushConstants the callers vary, runs.rs:2547-2580
    pub rope_mode: u32, pub rotary_dim: u32, pub theta_scale: f32, pub freq_scale: f32,
    pub attn_factor: f32, pub eps: f32,
}
#[repr(C)] pub struct VfkvGate {                  // SigmoidMulPushConstants (runs.rs:2667) plus the gate buffer
    pub gate: *const f32, pub chunk: u32, pub stride: u32, pub gate_offset: u32,
}
pub enum VfkvCache {} pub enum VfkvWorkspace {}
extern "C" {
    pub fn vfkv_last_error() -> *const c_char;
    pub fn vfkv_last_note() -> *const c_char;
    pub fn vfkv_status_string(status: c_int) -> *const c_char;
    pub fn vfkv_abi_version() -> u32;
    pub fn vfkv_device_count() -> c_int;
    pub fn vfkv_cache_create(cfg: *const VfkvCacheConfig, out: *mut *mut VfkvCache) -> c_int;
    pub fn vfkv_cache_create_external(cfg: *const VfkvCacheConfig, k_buffer: *mut c_void, v_buffer: *mut c_void,
                                      out: *mut *mut VfkvCache) -> c_int;
    pub fn vfkv_cache_kv_alignment_note(c: *const VfkvCache) -> *const c_char;
    pub fn vfkv_cache_destroy(c: *mut VfkvCache);
    pub fn vfkv_cache_zero_fill(c: *mut VfkvCache, stream: *mut c_void) -> c_int;
    pub fn vfkv_cache_zero_layer(c: *mut VfkvCache, layer: u32, stream: *mut c_void) -> c_int;
    pub fn vfkv_cache_current_seq_len(c: *const VfkvCache) -> u32;
    pub fn vfkv_cache_set_current_seq_len(c: *mut VfkvCache, n: u32);
    pub fn vfkv_cache_reset(c: *mut VfkvCache);
    pub fn vfkv_cache_dtype(c: *const VfkvCache) -> u32;
    pub fn vfkv_cache_bytes_per_buffer(c: *const VfkvCache) -> u64;
    pub fn vfkv_cache_head_dim_for(c: *const VfkvCache, layer: u32) -> u32;
    pub fn vfkv_cache_kv_heads_for(c: *const VfkvCache, layer: u32) -> u32;
    pub fn vfkv_cache_layer_offset_elems(c: *const VfkvCache, layer: u32) -> u64;
    pub fn vfkv_kv_bytes_per_token(n_layers: u32, n_kv_heads: u32, head_dim: u32, per_layer_head_dim: *const u32,
                                   per_layer_n_kv_heads: *const u32, elem_size: u64) -> u64;
    pub fn vfkv_guard_kv_precision(is_gemma4_moe: c_int, dtype: u32, force: c_int) -> c_int;
    pub fn vfkv_kv_start_batch(base_pos: u32, seq_len: u32, window: u32) -> u32;
    pub fn vfkv_decode_tile_for(span: u32, n_heads: u32, n_kv_heads: u32, head_dim: u32, kv_dtype: u32) -> u32;
    pub fn vfkv_cache_k_ptr(c: *const VfkvCache) -> *mut c_void;
    pub fn vfkv_cache_v_ptr(c: *const VfkvCache) -> *mut c_void;
    pub fn vfkv_cache_pos_offset_bytes(c: *const VfkvCache, layer: u32, pos: u32) -> u64;
    pub fn vfkv_cache_layer_offset_bytes(c: *const VfkvCache, layer: u32) -> u64;
    pub fn vfkv_cache_layer_size_bytes(c: *const VfkvCache, layer: u32) -> u64;
    pub fn vfkv_cache_row_bytes(c: *const VfkvCache, layer: u32) -> u64;
    pub fn vfkv_kv_start_decode(position: u32, sliding_window: u32) -> u32;
    pub fn vfkv_build_kv_sources(is_sliding: *const u8, n_pattern: u32, first_kv_shared: u32, n_layers: u32,
                                 kv_source_out: *mut u32);
    pub fn vfkv_kv_read_layer(kv_source: *const u32, n_layers: u32, layer: u32) -> u32;
    pub fn vfkv_prefix_reuse_start(cached_tokens: *const u32, n_cached: u32, tokens: *const u32, n_tokens: u32) -> u32;
    pub fn vfkv_store_fp8(src: *const f32, dst: *mut c_void, n_elements: u32, dst_byte_offset: u64,
                          stream: *mut c_void) -> c_int;                    // run_kv_store_fp8, runs.rs:2437
    pub fn vfkv_copy_fp16(src: *const f32, dst: *mut c_void, n_elements: u32, dst_byte_offset: u64,
                          stream: *mut c_void) -> c_int;                    // run_kv_copy_fp16, runs.rs:2389
    pub fn vfkv_fp8_to_f16(src: *const c_void, dst_f16: *mut c_void, n_elems: u64,
                           stream: *mut c_void) -> c_int;                   // runs.rs:1105-1137
    pub fn vfkv_kv_write(c: *mut VfkvCache, layer: u32, pos: u32, n_tokens: u32,
                         k_src: *const f32, v_src: *const f32, stream: *mut c_void) -> c_int; // step_kv_write
    pub fn vfkv_rms_norm_mul_rope(qk: *const f32, weight: *const f32, qk_out: *mut f32, head_dim: u32,
                                  heads_per_token: u32, m: u32, positions: *const i32, pos0: u32,
                                  freq_factors: *const f32, p: *const VfkvRopeParams,
                                  stream: *mut c_void) -> c_int;      // run_rms_norm_mul_rope, runs.rs:2492
    pub fn vfkv_k_rope_kv_write(c: *mut VfkvCache, layer: u32, pos: u32, n_tokens: u32, k_src: *const f32,
                                v_src: *const f32, k_norm_weight: *const f32, positions: *const i32,
                                freq_factors: *const f32, p: *const VfkvRopeParams, k_out: *mut f32,
                                stream: *mut c_void) -> c_int;        // KNormRope / KRope + KvWrite
    pub fn vfkv_qk_rope_kv_write(c: *mut VfkvCache, layer: u32, pos: u32, n_tokens: u32, n_heads: u32, q: *const f32,
                                 q_norm_weight: *const f32, q_out: *mut f32, k_src: *const f32, v_src: *const f32,
                                 k_norm_weight: *const f32, positions: *const i32, freq_factors: *const f32,
                                 p: *const VfkvRopeParams, k_out: *mut f32, stream: *mut c_void) -> c_int;
    pub fn vfkv_flash_attn_split(q: *const f32, k_layer: *const c_void, v_layer: *const c_void, kv_dtype: u32,
                                 so: *mut f32, sm: *mut f32, ss: *mut f32, p: *const VfkvSplitParams,
                                 tile: u32, softcap: f32, stream: *mut c_void) -> c_int;
    pub fn vfkv_flash_attn_split_interleaved(q: *const f32, k_layer: *const c_void, v_layer: *const c_void, kv_dtype: u32,
                                 so: *mut f32, sm: *mut f32, ss: *mut f32, p: *const VfkvSplitParams,
                                 tile: u32, softcap: f32, stream: *mut c_void) -> c_int;   // partial j is not tile j
    pub fn vfkv_flash_attn_reduce(so: *const f32, sm: *const f32, ss: *const f32, o: *mut f32,
                                  n_heads: u32, head_dim: u32, n_tiles: u32, stream: *mut c_void) -> c_int;
    pub fn vfkv_workspace_create(n_heads: u32, head_dim: u32, max_seq_len: u32, out: *mut *mut VfkvWorkspace) -> c_int;
    pub fn vfkv_workspace_destroy(w: *mut VfkvWorkspace);
    pub fn vfkv_decode_attention(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32,
                                 q: *const f32, o: *mut f32, position: u32, kv_start: u32, scale: f32,
                                 softcap: f32, ws: *mut VfkvWorkspace, stream: *mut c_void) -> c_int; // run_scalar_attn
    pub fn vfkv_decode_attention_static(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32,
                                        q: *const f32, o: *mut f32, position: u32, kv_start: u32, scale: f32,
                                        softcap: f32, stream: *mut c_void) -> c_int; // no workspace, no allocation
    pub fn vfkv_prefill_attention(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32, q: *const f32,
                                  o: *mut f32, m: u32, base_pos: u32, window: u32, scale: f32, softcap: f32,
                                  stream: *mut c_void) -> c_int;               // b_step_attention
    pub fn vfkv_qk_rope_kv_write_decode_attention(c: *mut VfkvCache, layer: u32, n_heads: u32, q: *const f32, q_norm_weight: *const f32,
                                                  q_out: *mut f32, k_src: *const f32, v_src: *const f32, k_norm_weight: *const f32,
                                                  freq_factors: *const f32, p: *const VfkvRopeParams, k_out: *mut f32, o: *mut f32,
                                                  position: u32, kv_start: u32, scale: f32, softcap: f32, ws: *mut VfkvWorkspace,
                                                  stream: *mut c_void) -> c_int;
    pub fn vfkv_kv_write_decode_attention(c: *mut VfkvCache, layer: u32, n_heads: u32, q: *const f32,
                                          k_src: *const f32, v_src: *const f32, o: *mut f32, position: u32,
                                          kv_start: u32, scale: f32, softcap: f32, ws: *mut VfkvWorkspace,
                                          stream: *mut c_void) -> c_int;      // step_kv_write + step_attention
    pub fn vfkv_prefill_attention_ws(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32, q: *const f32,
                                     o: *mut f32, m: u32, base_pos: u32, window: u32, scale: f32, softcap: f32,
                                     ws: *mut VfkvWorkspace, stream: *mut c_void) -> c_int;
    pub fn vfkv_flash_attn_batch_opt(q: *const f32, k_layer: *const c_void, v_layer: *const c_void, kv_dtype: u32,
                                     o: *mut f32, p: *const VfkvBatchParams, softcap: f32, options: u32,
                                     stream: *mut c_void) -> c_int;            // options: VFKV_PREFILL_F16_WEIGHTS = 1, _FP8_SCORES = 2, _F16_QUERIES = 4
    pub fn vfkv_prefill_attention_opt(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32, q: *const f32,
                                      o: *mut f32, m: u32, base_pos: u32, window: u32, scale: f32, softcap: f32,
                                      options: u32, ws: *mut VfkvWorkspace, stream: *mut c_void) -> c_int;
    pub fn vfkv_sigmoid_mul(gate: *const VfkvGate, data: *mut f32, ne: u32, stream: *mut c_void) -> c_int;
    pub fn vfkv_decode_attention_gated(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32, q: *const f32,
                                       k_src: *const f32, v_src: *const f32, o: *mut f32, position: u32, kv_start: u32,
                                       scale: f32, softcap: f32, gate: *const VfkvGate, ws: *mut VfkvWorkspace,
                                       stream: *mut c_void) -> c_int;
    pub fn vfkv_prefill_attention_gated(c: *mut VfkvCache, layer: u32, kv_layer: u32, n_heads: u32, q: *const f32,
                                        o: *mut f32, m: u32, base_pos: u32, window: u32, scale: f32, softcap: f32,
                                        gate: *const VfkvGate, stream: *mut c_void) -> c_int;
    pub fn vfkv_flash_attn_batch(q: *const f32, k_layer: *const c_void, v_layer: *const c_void, kv_dtype: u32,
                                 o: *mut f32, p: *const VfkvBatchParams, softcap: f32, stream: *mut c_void) -> c_int;
}
