/*
 * vfkv.h -- C ABI of the MI355X (gfx950) KV-cache / attention hot path.
 *
 * Every entry point replaces one piece of the reference's Vulkan dispatch layer; the reference
 * location is cited next to it (paths relative to the reference tree).  Conventions:
 *
 *   - All data pointers are HIP device pointers owned by the caller, except the two cache
 *     buffers owned by a `vfkv_cache` created with vfkv_cache_create().
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Functions only
 *     enqueue work on it (the analogue of "record into the open command buffer") and never
 *     synchronise; ordering between calls is stream order, which replaces the reference's
 *     in-command-buffer barriers (executor/attention.rs:583-595, runs.rs:1539-1541).
 *   - Return value: VFKV_OK (0) or a negative vfkv_status.  Nothing panics or aborts across the
 *     ABI; vfkv_last_error() returns a thread-local description of the last failure.
 *   - Thread-compatible: distinct caches / workspaces / streams may be used from distinct
 *     threads; one workspace must not be used by two in-flight calls at once.
 *   - There is no CPU fallback: without a HIP device every compute entry point fails with
 *     VFKV_ERR_HIP / VFKV_ERR_NO_DEVICE.  Layout arithmetic works without a device.
 *   - Two environment variables are read, once per process, and nothing else is tunable at run time:
 *       VFKV_DECODE_TILE=<multiple of 64>   keys per workgroup in vfkv_decode_attention, instead of the library's own
 *                                            choice (the reference's split-chunk size, runs.rs:766);
 *       VFKV_DECODE_WORKER=valu              serve every decode shape with the vector-ALU worker instead of the
 *                                            matrix-core worker (for comparisons).
 */
#ifndef VFKV_H
#define VFKV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* The library is built with hidden symbol visibility; the declarations of this header are its whole exported surface. */
#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility push(default)
#endif

#define VFKV_ABI_VERSION 1u

typedef void* vfkv_stream; /* hipStream_t */

typedef enum vfkv_status {
    VFKV_OK = 0,
    VFKV_ERR_INVALID_ARG = -1, /* NULL pointer, zero dimension, n_heads % n_kv_heads != 0, ... */
    VFKV_ERR_OVERFLOW = -2,    /* size arithmetic does not fit (kv_cache.rs:270-291) */
    VFKV_ERR_ALIGNMENT = -3,   /* dst_byte_offset % 4 != 0 (runs.rs:2400-2404, 2448-2453) */
    VFKV_ERR_UNSUPPORTED = -4, /* shape outside what the kernels cover (e.g. head_dim > 512) */
    VFKV_ERR_HIP = -5,         /* a HIP runtime call failed; see vfkv_last_error() */
    VFKV_ERR_NO_DEVICE = -6,
    VFKV_ERR_WORKSPACE = -7    /* workspace too small for the requested launch */
} vfkv_status;

/* KvDtype, kv_cache.rs:42-74 (element_size 4 / 2 / 1). */
typedef enum vfkv_dtype { VFKV_F32 = 0, VFKV_F16 = 1, VFKV_F8E4M3 = 2 } vfkv_dtype;

const char* vfkv_status_string(int status);
const char* vfkv_last_error(void);
/* Advisory left by the last attention call of this thread ("" when there is none; never an error and never mixed into
 * vfkv_last_error): set when the shape fell to the generic fallback kernels (head_dim other than 64, 128, 256, 512 or a
 * multiple of 16 between 64 and 256 -- over F32 caches decode has no tiled kernel for 512 --, pointers not 16-byte aligned,
 * or a layer slab of 2 GiB or more), which are 50-100x slower than the tiled kernels. */
const char* vfkv_last_note(void);
uint32_t vfkv_abi_version(void);
/* Number of visible HIP devices (0 when there is none or the runtime cannot initialise). */
int vfkv_device_count(void);

/* ------------------------------------------------------------------------------------------ */
/* KV cache object -- replaces `KvCache` (kv_cache.rs:204-500).                                */
/* Pos-major layout K[layer][pos][kv_head][d] (kv_cache.rs:3-12), two buffers K and V.         */
/* ------------------------------------------------------------------------------------------ */

/* KvCacheConfig, kv_cache.rs:153-174.  The per-layer tables may be NULL (uniform layout); when
 * given they hold n_layers entries and select the cumulative-offset layout (kv_cache.rs:256-283). */
typedef struct vfkv_cache_config {
    uint32_t n_layers;
    uint32_t n_kv_heads;
    uint32_t head_dim;
    uint32_t max_seq_len;
    const uint32_t* per_layer_head_dim;
    const uint32_t* per_layer_n_kv_heads;
    uint32_t dtype; /* vfkv_dtype; the reference reads it from the environment (kv_cache.rs:85-101) */
} vfkv_cache_config;

typedef struct vfkv_cache vfkv_cache;

/* KvCache::new (kv_cache.rs:224-339): checked size arithmetic, then two device allocations.  The V
 * buffer starts 256 bytes into its allocation (vfkv_cache_v_ptr returns the shifted pointer): K and V
 * of a row are requested together, and with equally aligned buffers one 128-byte column of every row
 * is served measurably slower. */
int vfkv_cache_create(const vfkv_cache_config* cfg, vfkv_cache** out);
/* Same layout object over caller-owned buffers (either may be NULL for layout-only use, e.g. on a
 * host without a GPU).  No allocation happens and destroy() leaves the buffers alone.  For speed give
 * the two buffers different alignment modulo 512 bytes (e.g. v_buffer = allocation + 256): results are
 * identical either way, but equally aligned buffers cost the attention kernels up to 8 %;
 * vfkv_cache_kv_alignment_note() tells. */
int vfkv_cache_create_external(const vfkv_cache_config* cfg, void* k_buffer, void* v_buffer,
                               vfkv_cache** out);
/* "" when the two buffers of the cache differ in address bits 7-8 (or one is NULL), else a one-line advisory that says
 * what to change.  No counterpart in the reference (its allocator places the buffers, kv_cache.rs:293-339). */
const char* vfkv_cache_kv_alignment_note(const vfkv_cache* c);
/* KvCache::destroy (kv_cache.rs:496-499). */
void vfkv_cache_destroy(vfkv_cache* c);
/* KvCache::zero_fill (kv_cache.rs:357-380) / zero_layer (kv_cache.rs:389-407).  Both enqueue fill
 * kernels (no memset nodes), so they may be captured into a HIP graph like the compute calls. */
int vfkv_cache_zero_fill(vfkv_cache* c, vfkv_stream stream);
int vfkv_cache_zero_layer(vfkv_cache* c, uint32_t layer, vfkv_stream stream);
/* current_seq_len field and KvCache::reset (kv_cache.rs:492-494). */
uint32_t vfkv_cache_current_seq_len(const vfkv_cache* c);
void vfkv_cache_set_current_seq_len(vfkv_cache* c, uint32_t n);
void vfkv_cache_reset(vfkv_cache* c);

void* vfkv_cache_k_ptr(const vfkv_cache* c);
void* vfkv_cache_v_ptr(const vfkv_cache* c);
uint32_t vfkv_cache_dtype(const vfkv_cache* c);
uint64_t vfkv_cache_bytes_per_buffer(const vfkv_cache* c);                       /* kv_cache.rs:383 */
uint32_t vfkv_cache_head_dim_for(const vfkv_cache* c, uint32_t layer);           /* kv_cache.rs:412 */
uint32_t vfkv_cache_kv_heads_for(const vfkv_cache* c, uint32_t layer);           /* kv_cache.rs:422 */
uint64_t vfkv_cache_layer_offset_elems(const vfkv_cache* c, uint32_t layer);     /* kv_cache.rs:431 */
uint64_t vfkv_cache_pos_offset_bytes(const vfkv_cache* c, uint32_t layer, uint32_t pos); /* :446 */
uint64_t vfkv_cache_row_bytes(const vfkv_cache* c, uint32_t layer);              /* kv_cache.rs:456 */
uint64_t vfkv_cache_layer_offset_bytes(const vfkv_cache* c, uint32_t layer);     /* kv_cache.rs:466 */
uint64_t vfkv_cache_layer_size_bytes(const vfkv_cache* c, uint32_t layer);       /* kv_cache.rs:485 */
/* kv_bytes_per_token (kv_cache.rs:186-202), saturating. */
uint64_t vfkv_kv_bytes_per_token(uint32_t n_layers, uint32_t n_kv_heads, uint32_t head_dim,
                                 const uint32_t* per_layer_head_dim,
                                 const uint32_t* per_layer_n_kv_heads, uint64_t elem_size);
/* guard_kv_precision_inner (kv_cache.rs:127-151): 0 when the combination is allowed. */
int vfkv_guard_kv_precision(int is_gemma4_moe, uint32_t dtype, int force);
/* gemma4_kv_start (forward/arch/gemma4.rs:59-73): max(0, position + 1 - sliding_window). */
uint32_t vfkv_kv_start_decode(uint32_t position, uint32_t sliding_window);
/* b_step_attention (executor/attention.rs:2215-2219): window of the LAST query of the batch. */
uint32_t vfkv_kv_start_batch(uint32_t base_pos, uint32_t seq_len, uint32_t window);
/* Gemma4KvSource (gguf.rs:879-895): how a layer relates to the cross-layer KV share. */
#define VFKV_KV_OWN 0u
#define VFKV_KV_OWN_PUBLISHES_SLIDING 1u
#define VFKV_KV_OWN_PUBLISHES_FULL 2u
#define VFKV_KV_SUBSCRIBES_SLIDING 3u
#define VFKV_KV_SUBSCRIBES_FULL 4u
/* gemma4_kv_read_layer (forward/arch/gemma4.rs:27-49): the layer whose slab `layer` reads, i.e. the
 * `kv_layer` argument of the attention entry points.  `kv_source` holds one VFKV_KV_* value per
 * layer (NULL: no sharing).  Owners read themselves, subscribers the FIRST layer that publishes
 * their kind, and themselves when nobody does.  `layer >= n_layers` returns `layer`. */
uint32_t vfkv_kv_read_layer(const uint32_t* kv_source, uint32_t n_layers, uint32_t layer);
/* build_kv_sources (gguf.rs:908-942): fills kv_source_out[n_layers] from the model's sliding /
 * full pattern (is_sliding[i] != 0: sliding layer; layers beyond n_pattern count as sliding).
 * Layers before `first_kv_shared` own their rows, the LAST sliding and the LAST full layer among
 * them publish; every later layer subscribes to its kind. */
void vfkv_build_kv_sources(const uint8_t* is_sliding, uint32_t n_pattern, uint32_t first_kv_shared,
                           uint32_t n_layers, uint32_t* kv_source_out);
/* The start position of a request that reuses the resident rows of the previous one
 * (ServerSession::generate_reuse, server/state.rs:199-201, longest_common_prefix :49-51): the
 * length of the common prefix of the two token sequences, capped at n_tokens - 1 so that at
 * least one token is prefilled.  The caller then keeps rows [0, k) (k > 0:
 * vfkv_cache_set_current_seq_len(c, k); k == 0: vfkv_cache_reset(c)) and prefills from base_pos k. */
uint32_t vfkv_prefix_reuse_start(const uint32_t* cached_tokens, uint32_t n_cached,
                                 const uint32_t* tokens, uint32_t n_tokens);

/* ------------------------------------------------------------------------------------------ */
/* KV append and expansion kernels.                                                           */
/* ------------------------------------------------------------------------------------------ */

/* Forward::run_kv_store_fp8 (forward/runs.rs:2437-2478) + kv_store_fp8.comp:42-67.
 * dst[dst_byte_offset + i] = e4m3(src[i]) for i < n_elements, saturating round-to-nearest-even
 * E4M3FN (fp8_ext.rs:126-186); the tail of the last 32-bit word is zero-filled. */
int vfkv_store_fp8(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset,
                   vfkv_stream stream);
/* Forward::run_kv_copy_fp16 (forward/runs.rs:2389-2430) + kv_copy_fp16.comp:39-51. */
int vfkv_copy_fp16(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset,
                   vfkv_stream stream);
/* The kv_fp8_to_f16 pass of run_flash_attn_cm_gemma_rs (forward/runs.rs:1105-1137) +
 * kv_fp8_to_f16.comp:28-33: dst_f16[i] = f16(e4m3_decode(src[i])), i < n_elems. */
int vfkv_fp8_to_f16(const void* src, void* dst_f16, uint64_t n_elems, vfkv_stream stream);

/* step_kv_write (executor/attention.rs:546-597) and b_step_kv_write (:2134-2190): append
 * `n_tokens` rows of K and of V (f32, [n_tokens, kv_heads_for(layer) * head_dim_for(layer)]) at
 * position `pos` of `layer`, in the cache's dtype.  K and V go out in one launch.  For an F32
 * cache this is the reference's plain buffer copy. */
int vfkv_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens,
                  const float* k_src, const float* v_src, vfkv_stream stream);

/* RoPE parameters as the reference's callers fill RopePushConstants (forward/runs.rs:2547-2580,
 * 680-700): freq_scale = attn_factor = 1, ext_factor = 0 (the YaRN ramp of rope_funcs.glsl:17-37 is
 * not built), no sections. */
#define VFKV_ROPE_NORM 0u /* GGML_ROPE_TYPE_NORMAL: pairs (2p, 2p + 1)              (rope_funcs.glsl:39-76)  */
#define VFKV_ROPE_NEOX 2u /* GGML_ROPE_TYPE_NEOX:   pairs (p, p + rotary_dim / 2)   (rope_funcs.glsl:78-112) */
typedef struct {
    uint32_t rope_mode;   /* VFKV_ROPE_NORM / VFKV_ROPE_NEOX (config.rope_variant, runs.rs:2532-2535) */
    uint32_t rotary_dim;  /* n_dims: even, <= head_dim; elements beyond it pass through */
    float theta_scale;    /* (1 / freq_base)^(2 / rotary_dim)  (forward/layer_plan.rs:532) */
    float freq_scale;     /* 1.0 in the reference's callers */
    float attn_factor;    /* 1.0 in the reference's callers */
    float eps;            /* rms_norm epsilon (cfg.rms_norm_eps); used only with a norm weight */
} vfkv_rope_params;

/* Forward::run_rms_norm_mul_rope (forward/runs.rs:2492-2600; rms_norm.comp:36-129 in its fused
 * form) and, with `weight` NULL, Forward::run_rope_neox_with_pos_offset (runs.rs:647-720;
 * rope_neox.comp / rope_norm.comp): `qk` is [m, heads_per_token, head_dim] f32; each (token, head)
 * row is RMS-normalised, multiplied by weight[head_dim] and rotated with the token's position
 * (positions[t], or pos0 + t when positions is NULL).  `qk_out` may alias `qk` (the production
 * callers rotate in place).  This is the Q side (step_q_norm_rope / step_q_rope,
 * executor/attention.rs:360-432,490-512); for K use vfkv_k_rope_kv_write, which also appends. */
int vfkv_rms_norm_mul_rope(const float* qk, const float* weight, float* qk_out, uint32_t head_dim,
                           uint32_t heads_per_token, uint32_t m, const int32_t* positions,
                           uint32_t pos0, const float* freq_factors, const vfkv_rope_params* p,
                           vfkv_stream stream);

/* `KNormRope` or `KRope` followed by `KvWrite` (forward/layer_plan.rs:119-137) in one launch:
 * step_k_norm_rope / step_k_rope (executor/attention.rs:435-530; batch :2026-2133) =
 * run_rms_norm_mul_rope (forward/runs.rs:2492-2600, rms_norm.comp:36-129 fused with
 * rope_funcs.glsl:39-112) or run_rope_neox_with_pos_offset (runs.rs:647-720), then step_kv_write
 * (attention.rs:546-597).  K rows [n_tokens, kv_heads * head_dim] f32 are RMS-normalised per head
 * and multiplied by `k_norm_weight[head_dim]` (NULL: no norm, the plain `KRope`), rotated with
 * theta = positions[t] * theta_scale^p / freq_factors[p] (positions NULL: pos + t, the values the
 * reference writes to rope_pos_buf; freq_factors NULL: 1, has_ff = 0), and stored at position
 * pos + t of `layer` in the cache dtype; V rows are stored as vfkv_kv_write stores them.  `k_out`
 * (may be k_src, may be NULL) receives the rotated K as f32, which is what the reference leaves in
 * k_buf. */
int vfkv_k_rope_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens,
                         const float* k_src, const float* v_src, const float* k_norm_weight,
                         const int32_t* positions, const float* freq_factors,
                         const vfkv_rope_params* p, float* k_out, vfkv_stream stream);

/* The same launch with the query rows added: `QNormRope` / `QRope` + `KNormRope` / `KRope` + `KvWrite`
 * of one layer (forward/layer_plan.rs:119-137; step_q_norm_rope, step_k_norm_rope, step_kv_write,
 * executor/attention.rs:360-597) as ONE launch.  `q` is [n_tokens, n_heads, head_dim] f32 and is
 * RMS-normalised * q_norm_weight (NULL: no norm) and rotated with the same angles into `q_out`
 * (may alias `q`); K, V and the remaining arguments are those of vfkv_k_rope_kv_write. */
int vfkv_qk_rope_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens,
                          uint32_t n_heads, const float* q, const float* q_norm_weight, float* q_out,
                          const float* k_src, const float* v_src, const float* k_norm_weight,
                          const int32_t* positions, const float* freq_factors,
                          const vfkv_rope_params* p, float* k_out, vfkv_stream stream);

/* ------------------------------------------------------------------------------------------ */
/* Decode attention: split-K worker + log-sum-exp merge.                                      */
/* ------------------------------------------------------------------------------------------ */

/* FlashAttnSplitPushConstants, pipeline.rs:553-569 (32 bytes, same field order). */
typedef struct vfkv_split_params {
    uint32_t n_heads;
    uint32_t n_kv_heads;
    uint32_t head_dim;
    uint32_t seq_len;
    uint32_t max_seq; /* unused by the kernels, kept for layout compatibility */
    float scale;
    uint32_t n_tiles; /* ceil(seq_len / tile) */
    uint32_t kv_start;
} vfkv_split_params;

/* Forward::run_flash_attn_split_reduce, worker half (forward/runs.rs:1463-1537) +
 * flash_attn_split.comp:82-162.  `k_layer` / `v_layer` point at the start of the layer's slab
 * (buffer + layer_offset_bytes(kv_layer), runs.rs:1507-1508).  Tile j covers keys
 * [j*tile, (j+1)*tile); partials go to scratch_out[(h*n_tiles + j)*head_dim + d] and
 * scratch_max / scratch_sum[h*n_tiles + j].  The reference fixes tile = 64
 * (flash_attn_split.comp:23-24); here it is a parameter (multiple of 16, <= 65536).
 * `softcap` > 0 applies s <- softcap * tanh(s / softcap) after scaling (an extension: the
 * reference has no attention soft-cap); 0 disables it. */
int vfkv_flash_attn_split(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                          float* scratch_out, float* scratch_max, float* scratch_sum,
                          const vfkv_split_params* p, uint32_t tile, float softcap,
                          vfkv_stream stream);

/* Same arguments and the same number of partials as vfkv_flash_attn_split, for callers that only ever
 * hand the partials to vfkv_flash_attn_reduce: partial j is then not tile j.  Where the matrix-core
 * worker serves the shape, the rows are dealt to the n_tiles workgroups in interleaved runs (what
 * vfkv_decode_attention launches); elsewhere this is vfkv_flash_attn_split.  The merged output is the
 * same either way (forward/runs.rs:1463-1571 as a whole; no single counterpart in the reference). */
int vfkv_flash_attn_split_interleaved(const float* q, const void* k_layer, const void* v_layer,
                                      uint32_t kv_dtype, float* scratch_out, float* scratch_max,
                                      float* scratch_sum, const vfkv_split_params* p, uint32_t tile,
                                      float softcap, vfkv_stream stream);

/* Forward::run_flash_attn_split_reduce, reducer half (forward/runs.rs:1543-1571) +
 * flash_attn_reduce.comp:35-81 (FlashAttnReducePushConstants, pipeline.rs:573-580). */
int vfkv_flash_attn_reduce(const float* scratch_out, const float* scratch_max,
                           const float* scratch_sum, float* o, uint32_t n_heads, uint32_t head_dim,
                           uint32_t n_tiles, vfkv_stream stream);

/* Scratch for vfkv_decode_attention -- replaces fa_scratch_out/max/sum (forward/setup.rs:203-230),
 * sized for ceil(max_seq_len / 64) tiles of n_heads * head_dim floats.  vfkv_prefill_attention_ws
 * borrows the same buffers.  Calls that share a workspace must be ordered on one stream. */
typedef struct vfkv_workspace vfkv_workspace;
int vfkv_workspace_create(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len,
                          vfkv_workspace** out);
void vfkv_workspace_destroy(vfkv_workspace* w);

/* Tile length (keys per workgroup) vfkv_decode_attention uses for `span` visible keys.  No
 * counterpart in the reference, which hard-codes 64 (runs.rs:766); exposed so that callers who
 * drive vfkv_flash_attn_split / _reduce themselves can reproduce the same launch.  The
 * environment variable VFKV_DECODE_TILE (a multiple of 64) overrides the choice. */
uint32_t vfkv_decode_tile_for(uint32_t span, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                              uint32_t kv_dtype);

/* Forward::run_scalar_attn (forward/runs.rs:722-822) == step_attention's body
 * (executor/attention.rs:599-625): one decode query per head over keys [kv_start, position].
 * `kv_layer` is the layer whose slab is read (Gemma-4 KV share, gemma4.rs:27-49; equals `layer`
 * otherwise), `layer` selects head_dim_for / kv_heads_for.  `scale` and `kv_start` are supplied
 * by the caller (runs.rs:734-760).  Chooses the tile length itself so that the launch fills the
 * GPU, skips tiles below kv_start, and merges the partials on the same stream.  Short contexts
 * go through the same kernels (the reference routes seq_len <= 64 to a single-workgroup shader,
 * runs.rs:766-821; the result is the same attention). */
int vfkv_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                          const float* q, float* o, uint32_t position, uint32_t kv_start, float scale,
                          float softcap, vfkv_workspace* ws, vfkv_stream stream);

/* vfkv_decode_attention for callers that cannot allocate device memory or carry a workspace object:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose scratch buffers are allocated once in forward/setup.rs:203-230).
 * The partials live in a device array that is part of the loaded library (VFKV_STATIC_SCRATCH_BYTES
 * per GPU, held until the process ends); the call makes no hipMalloc / hipFree and returns
 * VFKV_ERR_WORKSPACE when n_heads * partials * (head_dim + 2) floats exceed that size (32 / 8 / 128 at
 * any context needs 0.5 MiB; few KV heads at head_dim 512 need the most).  Same kernels, same tile
 * choice and bit-identical output as vfkv_decode_attention.  Every call on one GPU shares that GPU's
 * array: calls that overlap in time on one GPU (two streams, two threads) race; order them on one
 * stream.  Nothing in the array needs clearing between calls (every partial a merge reads is written
 * by the launch before it).  The array's address is looked up on the first call on each device,
 * which should therefore happen outside stream capture. */
#define VFKV_STATIC_SCRATCH_BYTES (5u << 20)
int vfkv_decode_attention_static(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                                 const float* q, float* o, uint32_t position, uint32_t kv_start,
                                 float scale, float softcap, vfkv_stream stream);

/* step_kv_write followed by step_attention for the same layer and token, as the executor issues them
 * back to back (executor/attention.rs:546-625): appends the token's K and V rows (f32,
 * kv_heads_for(layer) * head_dim_for(layer) elements each) at `position`, then attends over keys
 * [kv_start, position].  Where the decode worker can, the workgroups that own `position` write the
 * rows themselves before reading them, which saves the append launch; otherwise this is exactly
 * vfkv_kv_write + vfkv_decode_attention.  The cache bytes and the output are the same either way. */
int vfkv_kv_write_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t n_heads, const float* q,
                                   const float* k_src, const float* v_src, float* o, uint32_t position,
                                   uint32_t kv_start, float scale, float softcap, vfkv_workspace* ws,
                                   vfkv_stream stream);

/* The whole attention block of a decode layer as the executor issues it back to back (executor/attention.rs:360-625):
 * step_q_norm_rope / step_q_rope, step_k_norm_rope / step_k_rope, step_kv_write and step_attention of one token.
 * `q` [n_heads, head_dim] and `k_src` [kv_heads * head_dim] are the rows BEFORE norm and rotation; they are
 * RMS-normalised per head times q_norm_weight / k_norm_weight (NULL: no norm) and rotated for `position` exactly as
 * vfkv_qk_rope_kv_write does (same arithmetic: the cache bytes and k_out are bit-identical to that call), K and V are
 * appended at `position`, and the rotated queries attend over keys [kv_start, position].  Where the decode worker can,
 * all of this is ONE launch plus the merge: every workgroup rotates its query heads while its first K rows are in
 * flight, and the wavefront that reads the new row rotates, converts and stores it itself; otherwise the call is
 * vfkv_qk_rope_kv_write + vfkv_decode_attention.  `q_out` (may be NULL; must not overlap `q`) receives the rotated
 * queries, `k_out` (may be NULL, may be k_src) the rotated K row as f32 (what the reference leaves in q_buf / k_buf). */
int vfkv_qk_rope_kv_write_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t n_heads, const float* q,
                                           const float* q_norm_weight, float* q_out, const float* k_src,
                                           const float* v_src, const float* k_norm_weight,
                                           const float* freq_factors, const vfkv_rope_params* p, float* k_out,
                                           float* o, uint32_t position, uint32_t kv_start, float scale,
                                           float softcap, vfkv_workspace* ws, vfkv_stream stream);

/* ------------------------------------------------------------------------------------------ */
/* Chunked-prefill causal attention over the cache.                                           */
/* ------------------------------------------------------------------------------------------ */

/* FlashAttnBatchPushConstants, pipeline.rs:592-611 (32 bytes, same field order). */
typedef struct vfkv_batch_params {
    uint32_t n_heads;
    uint32_t n_kv_heads;
    uint32_t head_dim;
    uint32_t m;       /* queries in this batch */
    uint32_t n_kv;    /* populated KV positions (= q_start + m) */
    uint32_t q_start; /* KV position of the first query */
    float scale;
    uint32_t kv_start; /* one lower bound for the whole batch */
} vfkv_batch_params;

/* Forward::run_flash_attn_batch (forward/runs.rs:933-1010) + flash_attn_batch.comp:105-208.
 * q and o are [m, n_heads, head_dim] row-major f32; query i sees keys
 * [kv_start, min(q_start + i + 1, n_kv)). */
int vfkv_flash_attn_batch(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                          float* o, const vfkv_batch_params* p, float softcap, vfkv_stream stream);

/* b_step_attention's fallback route (executor/attention.rs:2192-2219, 2383-2390): batch attention
 * of `m` queries starting at `base_pos` over the cache, kv_start derived from `window`
 * (0 = full history) exactly as the reference does. */
int vfkv_prefill_attention(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                           const float* q, float* o, uint32_t m, uint32_t base_pos, uint32_t window,
                           float scale, float softcap, vfkv_stream stream);

/* vfkv_prefill_attention with a workspace (the one of the decode path).  Short chunks over long
 * histories -- the suffix of a request that keeps the resident rows of its prefix, server/state.rs:
 * 199-224 -- leave most compute units without a workgroup; with a workspace the keys are also cut
 * into chunks over workgroups and the decode merge (vfkv_flash_attn_reduce's kernel) combines the
 * partials.  Same results within f32 rounding; falls back to the plain call whenever that is not
 * worth it or the workspace is too small (it needs m * n_heads * chunks * head_dim floats). */
int vfkv_prefill_attention_ws(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                              const float* q, float* o, uint32_t m, uint32_t base_pos, uint32_t window,
                              float scale, float softcap, vfkv_workspace* ws, vfkv_stream stream);

/* Options of the two calls below (no counterpart in the reference, whose scalar shader has one precision). */
#define VFKV_PREFILL_F16_WEIGHTS 1u /* The softmax weights enter the P.V product rounded to f16 (11 significant bits)
                                     * instead of as an f16 value + remainder pair: a third fewer matrix instructions
                                     * (512 x 4 608 queries x keys, 32 / 8 / 128, FP8: 70.7 -> 60.3 us per layer).  Each
                                     * weight is off by up to 2^-11 relative, the output by up to 2^-11 * max|v| (4.5e-5
                                     * measured on N(0,1) inputs; 1.3e-2 with +-40 outliers in V, which is outside this
                                     * path's 5e-3 bound -- hence an option and not the default).  Honoured for FP8 / F16
                                     * caches at head_dim 128 with GQA groups of 2-8 heads (FP8) or 3-4 (F16); ignored
                                     * elsewhere. */

#define VFKV_PREFILL_FP8_SCORES 2u  /* The first product K.Q^T runs on the FP8 matrix instruction: the cache rows enter as
                                     * stored (no widening to f16), the queries as three E4M3 terms (12 significant bits:
                                     * exact for f16-representable q).  The instruction sums its 128 products with about 15
                                     * bits, so a score is off by about 1e-5 of the sum of its |k.q| products.  Honoured for
                                     * FP8 caches at head_dim 128 with GQA groups of 2-4 heads; ignored elsewhere. */

#define VFKV_PREFILL_F16_QUERIES 4u /* The queries enter the first product rounded to f16 (11 significant bits); without it, queries
                                     * that f16 cannot represent are multiplied as f16 value + remainder, which repeats the
                                     * first product.  A score is off by up to 2^-12 of the sum of its |k.q| products times
                                     * scale (outputs off by 1e-3 at most over 160 k values with queries of standard
                                     * deviation 2 and N(0,1) rows at head_dim 128).  What a caller gets who casts
                                     * its queries to f16 precision first, without that pass: 512 x 4 608, 32 / 8 / 128, f32
                                     * queries: FP8 72.4 -> 64.8 us per layer, F16 102 -> 76 us.  Honoured by the f16
                                     * matrix-core kernels (FP8 / F16 caches, head_dim 64 / 128 / 256 / 512); ignored elsewhere. */

/* vfkv_flash_attn_batch with options (VFKV_PREFILL_* bits). */
int vfkv_flash_attn_batch_opt(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                              float* o, const vfkv_batch_params* p, float softcap, uint32_t options,
                              vfkv_stream stream);

/* vfkv_prefill_attention with options; `ws` (may be NULL) as in vfkv_prefill_attention_ws. */
int vfkv_prefill_attention_opt(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                               const float* q, float* o, uint32_t m, uint32_t base_pos, uint32_t window,
                               float scale, float softcap, uint32_t options, vfkv_workspace* ws,
                               vfkv_stream stream);

/* ------------------------------------------------------------------------------------------ */
/* Gated attention output (Qwen3.6 full-attention layers).                                    */
/* ------------------------------------------------------------------------------------------ */
/* Where the gate of output element i lives (SigmoidMulPushConstants, forward/runs.rs:2667;
 * vk_shaders/sigmoid_mul.comp:30-48): gate[(i / chunk) * stride + gate_offset + i % chunk],
 * i = flat index into the output.  Decode passes (q_dim, q_dim, q_dim) with gate = q_buf
 * (executor/attention.rs:655-664), the batch path (head_dim, 2 * head_dim, head_dim) with
 * gate = batch_qgate (executor/attention.rs:2433-2441). */
typedef struct vfkv_gate {
    const float* gate;
    uint32_t chunk;       /* > 0 */
    uint32_t stride;
    uint32_t gate_offset;
} vfkv_gate;

/* Forward::run_sigmoid_mul (forward/runs.rs:2649-2681) + sigmoid_mul.comp:40-53:
 * data[i] *= 1 / (1 + exp(-gate[...])) for i < ne, in place. */
int vfkv_sigmoid_mul(const vfkv_gate* gate, float* data, uint32_t ne, vfkv_stream stream);

/* step_attention followed by step_attn_gated_output (executor/attention.rs:599-680), and with
 * k_src / v_src != NULL also the step_kv_write before them (layer == kv_layer then, as in
 * vfkv_kv_write_decode_attention): `o` leaves already multiplied by sigmoid(gate).  The merge
 * kernel applies the gate in its own store, so no third launch runs (spans that fit one tile
 * take a separate vfkv_sigmoid_mul launch).  Results are bit-identical to the separate calls.
 * `gate->gate` must not overlap `o`. */
int vfkv_decode_attention_gated(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                                const float* q, const float* k_src, const float* v_src, float* o,
                                uint32_t position, uint32_t kv_start, float scale, float softcap,
                                const vfkv_gate* gate, vfkv_workspace* ws, vfkv_stream stream);

/* b_step_attention followed by b_step_attn_gated_output (executor/attention.rs:2192-2219,
 * 2405-2444): vfkv_prefill_attention with the gate on the m * n_heads * head_dim outputs.  The
 * FP8 / F16 matrix-core kernel applies the gate in its own store when gate->chunk is a multiple of
 * head_dim, chunk / stride / gate_offset are multiples of 4 and gate->gate is 16-byte aligned (the
 * reference's [Q | G] per (token, head) layout qualifies); otherwise a vfkv_sigmoid_mul launch
 * follows on the same stream.  Results are bit-identical to the separate calls either way.
 * `gate->gate` must not overlap `o`. */
int vfkv_prefill_attention_gated(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads,
                                 const float* q, float* o, uint32_t m, uint32_t base_pos, uint32_t window,
                                 float scale, float softcap, const vfkv_gate* gate, vfkv_stream stream);

#if defined(__GNUC__) || defined(__clang__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* VFKV_H */
