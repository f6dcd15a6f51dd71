// Internal launch interface between the C ABI (api.cpp) and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vfkv {

// ---- kv_append.hip ----
hipError_t launch_kv_append(uint32_t dtype, const float* k_src, const float* v_src, void* k_dst, void* v_dst,
                            uint32_t n_elements, int n_tensors, hipStream_t stream);
hipError_t launch_fp8_to_f16(const void* src, void* dst, uint64_t n, hipStream_t stream);
hipError_t launch_zero_bytes(void* dst, uint64_t n, hipStream_t stream);

// K RMS-norm * weight + RoPE + append of K and V rows in one launch (rope_append.hip).
struct RopeAppendLaunch {
    const float* q_src = nullptr;         // optional Q rows [n_tokens][n_q_heads][head_dim]: normed * q_weight, rotated -> q_out
    const float* q_weight = nullptr;
    float* q_out = nullptr;
    uint32_t n_q_heads = 0;
    const float* k_src = nullptr;         // [n_tokens][n_kv_heads][head_dim]
    const float* v_src = nullptr;         // same shape; NULL = K only
    const float* weight = nullptr;        // [head_dim]; NULL = no RMS-norm
    const int32_t* positions = nullptr;   // [n_tokens]; NULL = pos0 + token
    const float* freq_factors = nullptr;  // [rotary_dim / 2]; NULL = 1
    float* k_out = nullptr;               // rotated K as f32 (may alias k_src); NULL = not wanted
    void* k_dst = nullptr;                // cache row of the first token (layer offset + pos0 * row_bytes applied);
                                          // NULL = no cache store: norm + RoPE into k_out only (v_src must be NULL too)
    void* v_dst = nullptr;
    uint32_t dtype = 0, n_tokens = 0, n_kv_heads = 0, head_dim = 0, rotary_dim = 0;
    uint32_t mode = 2;                    // 0 = NORM (adjacent pairs), 2 = NEOX (split halves)
    uint32_t pos0 = 0;
    uint64_t row_bytes = 0;
    float theta_scale = 1.f, freq_scale = 1.f, attn_factor = 1.f, eps = 0.f;
};
hipError_t launch_rope_append(const RopeAppendLaunch& L, hipStream_t stream);

// ---- attn_decode.hip ----
// Q-norm / RoPE and K-norm / RoPE of the decode token, folded into the decode worker (attn_decode_il.h).
struct RopeFold {
    const float* q_weight = nullptr;       // [head_dim] or NULL
    const float* k_weight = nullptr;       // [head_dim] or NULL
    const float* freq_factors = nullptr;   // [rotary_dim / 2] or NULL
    float* q_out = nullptr;                // rotated queries [n_heads][head_dim] (must not overlap q), or NULL
    float* k_out = nullptr;                // rotated K row [n_kv_heads][head_dim] as f32, or NULL
    uint32_t rotary_dim = 0, mode = 2;
    float theta_scale = 1.f, freq_scale = 1.f, attn_factor = 1.f, eps = 0.f;
};
struct SplitLaunch {
    const float* q = nullptr;        // [n_heads, head_dim] f32
    const void* k = nullptr;         // layer slab, [pos][kv_head][d] in `dtype`
    const void* v = nullptr;
    float* scratch_out = nullptr;    // [(h * n_tiles + j) * head_dim + d]
    float* scratch_max = nullptr;    // [h * n_tiles + j]
    float* scratch_sum = nullptr;
    uint32_t dtype = 0, n_heads = 0, n_kv_heads = 0, head_dim = 0;
    uint32_t seq_len = 0, kv_start = 0;
    uint32_t tile = 0;         // keys per tile
    uint32_t tile_first = 0;   // absolute index of the first tile launched
    uint32_t n_tiles = 0;      // tiles launched == row length of the scratch arrays
    float scale = 0.f, softcap = 0.f;
    // optional fused append of one token (f32 rows of n_kv_heads * head_dim elements) at row append_pos of the slab
    const float* k_new = nullptr;
    const float* v_new = nullptr;
    uint32_t append_pos = 0;
    // optional, launches of a single tile: final output [n_heads, head_dim]; the worker normalises itself and writes
    // no partials (only when split_writes_output() is true)
    float* o_direct = nullptr;
    // partial j need not be tile j: the matrix-core worker then deals the rows of the launched tiles to its
    // workgroups in interleaved runs (other workers ignore the flag); the merge is the same either way
    bool interleave = false;
    // optional (interleaved launches that split_folds_rope() accepts): q and k_new are the rows BEFORE norm and rotation; the
    // worker RMS-normalises (weights may be NULL) and rotates them for position append_pos itself
    const struct RopeFold* rope = nullptr;
};
// Returns hipErrorInvalidValue when no kernel covers the shape (or when k_new / v_new are given although
// split_appends() is false: then the caller appends the row with launch_kv_append and leaves them NULL).
// *generic_used (optional) is set when the shape fell to the one-wavefront-per-(head, tile) fallback kernel.
hipError_t launch_split(const SplitLaunch& a, hipStream_t stream, bool* generic_used = nullptr);
bool split_appends(const SplitLaunch& a);
bool split_writes_output(const SplitLaunch& a);
// Gate of the attention output (vk_shaders/sigmoid_mul.comp:30-53): element i of the output is multiplied by
// sigmoid(gate[(i / chunk) * stride + gate_offset + i % chunk]).  gate == NULL: no gate.
struct GateArgs {
    const float* gate = nullptr;
    uint32_t chunk = 1, stride = 1, gate_offset = 0;
};
// `gate` (optional) is applied in the merge's own store where the kernel chosen for the shape can do so; otherwise
// (and only then) *gate_applied is false and the caller follows up with launch_sigmoid_mul.
hipError_t launch_reduce(const float* scratch_out, const float* scratch_max, const float* scratch_sum, float* o,
                         uint32_t n_heads, uint32_t head_dim, uint32_t n_tiles, hipStream_t stream,
                         const GateArgs* gate = nullptr, bool* gate_applied = nullptr);
// ---- gated_output.hip ----
hipError_t launch_sigmoid_mul(float* data, uint32_t ne, const GateArgs& gate, hipStream_t stream);
// True when launch_split would run the interleaved worker of attn_decode_il.h for L (it deals the runs to n_tiles
// workgroups per KV head whatever L.tile says, so the caller may choose n_tiles freely), and when that worker would also
// fold L.rope (which needs k_new / v_new as well).
bool split_interleaves(const SplitLaunch& a);
// True when launch_split will take pairs of neighbouring 64-wide FP8 KV heads as rows of 128 bytes (long spans, groups of up
// to four heads, no folded RoPE): the launch then has half as many KV heads to give workgroups to.
bool split_pairs_heads(const SplitLaunch& a);
bool split_folds_rope(const SplitLaunch& a);
// Width of the matrix-core worker that serves this head width with its tail masked off (FP8 / F16 rows of 80 / 96 / 112 ->
// 128, 160 / 192 / 224 -> 256); 0 for every other shape.
uint32_t split_padded_dim(uint32_t dtype, uint32_t head_dim);
// Rows per run of the matrix-core worker for this shape (0: the shape is not the matrix-core worker's).
uint32_t split_run_rows(uint32_t dtype, uint32_t head_dim);
// Run streams per workgroup when the launch deals the runs of the span to its workgroups, not tiles (else 0), and how many
// query heads of a GQA group one workgroup serves.
uint32_t split_run_streams(const SplitLaunch& a, uint32_t* heads_per_wg);
// Smallest tile granule (keys) the split kernel for this shape works in; 0 if unsupported.
uint32_t split_tile_granule(uint32_t dtype, uint32_t head_dim);

// ---- attn_prefill.hip ----
struct BatchLaunch {
    const float* q;   // [m, n_heads, head_dim] f32
    const void* k;
    const void* v;
    float* o;         // [m, n_heads, head_dim] f32
    uint32_t dtype, n_heads, n_kv_heads, head_dim;
    uint32_t m, n_kv, q_start, kv_start;
    float scale, softcap;
    // optional scratch for partials of key chunks (short query chunks over long histories): [rows][chunks][head_dim] floats and
    // two [rows][chunks] arrays, rows = m * n_heads; NULL: every workgroup walks all keys of its queries
    float* scratch_out = nullptr;
    float* scratch_max = nullptr;
    float* scratch_sum = nullptr;
    uint64_t scratch_out_floats = 0, scratch_ml_floats = 0;
    // optional gated output: o *= sigmoid(gate[...]), in the attention kernel's or the merge's own store where the shape
    // allows it and as a follow-up launch otherwise
    const GateArgs* gate = nullptr;
    // FP8 / F16 caches on the f16 matrix-core kernel: the softmax weights enter the second product rounded to f16 (one
    // product instead of value + remainder): about 15 % faster, every weight off by up to 2^-11 relative, so the output by up
    // to 2^-11 * max|v|.  Built for head_dim 128 with the GQA group in one wavefront pair (FP8) or one wavefront (F16); other
    // shapes and kernels ignore it and keep both products.
    bool f16_weights = false;
    // FP8 caches at head_dim 128, GQA groups of 2-4 heads: the first product K Q^T runs on the FP8 matrix instruction, K rows as
    // stored and Q as three E4M3 terms (12 significant bits); no widening of K.  Other shapes ignore it.
    bool fp8_scores = false;
    // f16 matrix-core kernels: the queries enter the first product as f16(q) only (no remainder pass for queries that f16
    // cannot represent): scores off by up to 2^-12 of the sum of their |k q| products
    bool f16_queries = false;
};
// *generic_used (optional) is set when the shape fell to the one-wavefront-per-(query, head) fallback kernel.
hipError_t launch_batch(const BatchLaunch& a, hipStream_t stream, bool* generic_used = nullptr);

}  // namespace vfkv
