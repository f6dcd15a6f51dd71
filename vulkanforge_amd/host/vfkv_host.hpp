// C++ host side above the C ABI: the reference's `KvCache` (src/backend/vulkan/kv_cache.rs) and the
// part of `Forward` that owns this path (the run_* dispatch helpers of forward/runs.rs and the four
// executor steps of forward/executor/attention.rs), with the reference's names, argument meaning and
// error behaviour.  Fallible construction throws vfkv::Error (the reference returns Err from
// KvCache::new, kv_cache.rs:224-228); the run_* helpers throw where the reference would panic on a
// failed dispatch (forward/mod.rs:127-128).  Everything forwards to libvfkv through extern "C"; a Rust
// host would bind the same symbols.
#pragma once
#include <cmath>
#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/vfkv.h"

namespace vfkv {

struct Error : std::runtime_error {
    int status;
    Error(int st, const std::string& what) : std::runtime_error(what), status(st) {}
};

inline void check(int status) {
    if (status != VFKV_OK) throw Error(status, std::string(vfkv_status_string(status)) + ": " + vfkv_last_error());
}

// KvDtype, kv_cache.rs:42-74
enum class KvDtype : uint32_t { F32 = VFKV_F32, F16 = VFKV_F16, F8 = VFKV_F8E4M3 };
inline uint64_t element_size(KvDtype d) { return d == KvDtype::F32 ? 4 : d == KvDtype::F16 ? 2 : 1; }
inline const char* label(KvDtype d) { return d == KvDtype::F32 ? "FP32" : d == KvDtype::F16 ? "FP16" : "FP8"; }

// KvCacheConfig, kv_cache.rs:153-174 (+ the dtype, which the reference reads from the environment)
struct KvCacheConfig {
    uint32_t n_layers = 0, n_kv_heads = 0, head_dim = 0, max_seq_len = 0;
    std::optional<std::vector<uint32_t>> per_layer_head_dim;
    std::optional<std::vector<uint32_t>> per_layer_n_kv_heads;
    KvDtype dtype = KvDtype::F16;
};

// kv_bytes_per_token, kv_cache.rs:186-202
inline uint64_t kv_bytes_per_token(uint32_t n_layers, uint32_t n_kv_heads, uint32_t head_dim,
                                   const std::vector<uint32_t>* per_layer_head_dim,
                                   const std::vector<uint32_t>* per_layer_n_kv_heads, uint64_t elem_size) {
    return vfkv_kv_bytes_per_token(n_layers, n_kv_heads, head_dim, per_layer_head_dim ? per_layer_head_dim->data() : nullptr,
                                   per_layer_n_kv_heads ? per_layer_n_kv_heads->data() : nullptr, elem_size);
}
// guard_kv_precision, kv_cache.rs:118-151
inline void guard_kv_precision(bool is_gemma4_moe, KvDtype dtype, bool force = false) {
    check(vfkv_guard_kv_precision(is_gemma4_moe, (uint32_t)dtype, force));
}
// gemma4_kv_start, forward/arch/gemma4.rs:59-73
inline uint32_t gemma4_kv_start(uint32_t position, uint32_t sliding_window) { return vfkv_kv_start_decode(position, sliding_window); }
// gemma4_kv_read_layer, forward/arch/gemma4.rs:27-49 (one VFKV_KV_* value per layer)
inline uint32_t gemma4_kv_read_layer(const std::vector<uint32_t>& kv_source, uint32_t layer) {
    return vfkv_kv_read_layer(kv_source.data(), (uint32_t)kv_source.size(), layer);
}
// build_kv_sources, gguf.rs:908-942
inline std::vector<uint32_t> build_kv_sources(const std::vector<uint8_t>& is_sliding, uint32_t first_kv_shared, uint32_t n_layers) {
    std::vector<uint32_t> out(n_layers);
    vfkv_build_kv_sources(is_sliding.data(), (uint32_t)is_sliding.size(), first_kv_shared, n_layers, out.data());
    return out;
}
// start position of a request that keeps the common prefix of the resident rows, server/state.rs:199-201
inline uint32_t prefix_reuse_start(const std::vector<uint32_t>& cached, const std::vector<uint32_t>& tokens) {
    return vfkv_prefix_reuse_start(cached.data(), (uint32_t)cached.size(), tokens.data(), (uint32_t)tokens.size());
}

class KvCache {
public:
    KvCacheConfig config;
    KvDtype kv_dtype;

    // KvCache::new (kv_cache.rs:224-339).  layout_only builds the offset arithmetic without buffers.
    explicit KvCache(KvCacheConfig cfg, bool layout_only = false) : config(std::move(cfg)), kv_dtype(config.dtype) {
        if (config.per_layer_head_dim && config.per_layer_head_dim->size() != config.n_layers)
            throw Error(VFKV_ERR_INVALID_ARG, "per_layer_head_dim length must equal n_layers");
        if (config.per_layer_n_kv_heads && config.per_layer_n_kv_heads->size() != config.n_layers)
            throw Error(VFKV_ERR_INVALID_ARG, "per_layer_n_kv_heads length must equal n_layers");
        vfkv_cache_config c{config.n_layers, config.n_kv_heads, config.head_dim, config.max_seq_len,
                            config.per_layer_head_dim ? config.per_layer_head_dim->data() : nullptr,
                            config.per_layer_n_kv_heads ? config.per_layer_n_kv_heads->data() : nullptr,
                            (uint32_t)config.dtype};
        check(layout_only ? vfkv_cache_create_external(&c, nullptr, nullptr, &h_) : vfkv_cache_create(&c, &h_));
    }
    KvCache(const KvCache&) = delete;
    KvCache& operator=(const KvCache&) = delete;
    KvCache(KvCache&& o) noexcept : config(std::move(o.config)), kv_dtype(o.kv_dtype), h_(o.h_) { o.h_ = nullptr; }
    ~KvCache() { destroy(); }
    void destroy() { if (h_) { vfkv_cache_destroy(h_); h_ = nullptr; } }   // kv_cache.rs:496-499

    vfkv_cache* handle() const { return h_; }
    void* k_buffer() const { return vfkv_cache_k_ptr(h_); }
    void* v_buffer() const { return vfkv_cache_v_ptr(h_); }
    uint32_t current_seq_len() const { return vfkv_cache_current_seq_len(h_); }
    void set_current_seq_len(uint32_t n) { vfkv_cache_set_current_seq_len(h_, n); }
    void reset() { vfkv_cache_reset(h_); }                                        // kv_cache.rs:492
    void zero_fill(vfkv_stream s = nullptr) { check(vfkv_cache_zero_fill(h_, s)); }            // :357
    void zero_layer(uint32_t layer, vfkv_stream s = nullptr) { check(vfkv_cache_zero_layer(h_, layer, s)); }  // :389
    uint64_t bytes_per_buffer() const { return vfkv_cache_bytes_per_buffer(h_); }
    uint32_t head_dim_for(uint32_t layer) const { return vfkv_cache_head_dim_for(h_, layer); }
    uint32_t kv_heads_for(uint32_t layer) const { return vfkv_cache_kv_heads_for(h_, layer); }
    uint64_t layer_offset_elems(uint32_t layer) const { return vfkv_cache_layer_offset_elems(h_, layer); }
    uint64_t pos_offset_bytes(uint32_t layer, uint32_t pos) const { return vfkv_cache_pos_offset_bytes(h_, layer, pos); }
    uint64_t row_bytes(uint32_t layer) const { return vfkv_cache_row_bytes(h_, layer); }
    uint64_t layer_offset_bytes(uint32_t layer) const { return vfkv_cache_layer_offset_bytes(h_, layer); }
    uint64_t layer_size_bytes(uint32_t layer) const { return vfkv_cache_layer_size_bytes(h_, layer); }
    bool is_fp8() const { return kv_dtype == KvDtype::F8; }
    bool is_fp16() const { return kv_dtype == KvDtype::F16; }

private:
    vfkv_cache* h_ = nullptr;
};

// The slice of `Forward` this path needs: the cache, the split-K scratch (setup.rs:203-230), the
// head count and attn_scale = 1/sqrt(head_dim) (setup.rs:786).  `stream` plays the role of the open
// command buffer: calls enqueue in order and never synchronise.
class Forward {
public:
    KvCache kv_cache;
    uint32_t n_heads;
    float attn_scale;
    vfkv_stream stream = nullptr;

    Forward(KvCache cache, uint32_t heads) : kv_cache(std::move(cache)), n_heads(heads) {
        uint32_t max_hd = kv_cache.config.head_dim;
        if (kv_cache.config.per_layer_head_dim)
            for (uint32_t d : *kv_cache.config.per_layer_head_dim) max_hd = d > max_hd ? d : max_hd;
        check(vfkv_workspace_create(n_heads, max_hd, kv_cache.config.max_seq_len, &ws_));
        attn_scale = 1.0f / std::sqrt((float)kv_cache.config.head_dim);
    }
    Forward(const Forward&) = delete;
    ~Forward() { if (ws_) vfkv_workspace_destroy(ws_); }

    // runs.rs:2437-2478 / 2389-2430 / 1105-1137
    void run_kv_store_fp8(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset) {
        check(vfkv_store_fp8(src, dst, n_elements, dst_byte_offset, stream));
    }
    void run_kv_copy_fp16(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset) {
        check(vfkv_copy_fp16(src, dst, n_elements, dst_byte_offset, stream));
    }
    void run_kv_fp8_to_f16(const void* src, void* dst_f16, uint64_t n_elems) { check(vfkv_fp8_to_f16(src, dst_f16, n_elems, stream)); }

    // executor/attention.rs:546-597 and :2134-2190
    void step_kv_write(uint32_t layer, uint32_t position, const float* k_src, const float* v_src) {
        check(vfkv_kv_write(kv_cache.handle(), layer, position, 1, k_src, v_src, stream));
    }
    void b_step_kv_write(uint32_t layer, uint32_t base_pos, uint32_t seq_len, const float* batch_k, const float* batch_v) {
        check(vfkv_kv_write(kv_cache.handle(), layer, base_pos, seq_len, batch_k, batch_v, stream));
    }

    // step_k_norm_rope / step_k_rope + step_kv_write (attention.rs:435-597, batch :2026-2190) in one launch;
    // k_norm_weight == nullptr is the plain KRope
    void step_k_rope_kv_write(uint32_t layer, uint32_t position, uint32_t n_tokens, const float* k_src, const float* v_src,
                              const float* k_norm_weight, const vfkv_rope_params& rope, const int32_t* positions = nullptr,
                              const float* freq_factors = nullptr, float* k_out = nullptr) {
        check(vfkv_k_rope_kv_write(kv_cache.handle(), layer, position, n_tokens, k_src, v_src, k_norm_weight, positions,
                                   freq_factors, &rope, k_out, stream));
    }

    // step_q_norm_rope + step_k_norm_rope + step_kv_write (attention.rs:360-597) in one launch; q is rotated in place
    void step_qk_rope_kv_write(uint32_t layer, uint32_t position, uint32_t n_tokens, float* q, const float* q_norm_weight,
                               const float* k_src, const float* v_src, const float* k_norm_weight, const vfkv_rope_params& rope,
                               const int32_t* positions = nullptr, const float* freq_factors = nullptr, float* k_out = nullptr) {
        check(vfkv_qk_rope_kv_write(kv_cache.handle(), layer, position, n_tokens, n_heads, q, q_norm_weight, q, k_src, v_src,
                                    k_norm_weight, positions, freq_factors, &rope, k_out, stream));
    }

    // runs.rs:1463-1571
    void run_flash_attn_split_reduce(uint32_t layer, uint32_t position, uint32_t kv_layer, uint32_t kv_start, const float* q,
                                     float* attn_out, float softcap = 0.f) {
        check(vfkv_decode_attention(kv_cache.handle(), layer, kv_layer, n_heads, q, attn_out, position, kv_start,
                                    scale_for(layer), softcap, ws_, stream));
    }
    // runs.rs:722-822 (the caller supplies kv_layer / kv_start as gemma4_kv_read_layer / gemma4_kv_start would)
    void run_scalar_attn(uint32_t layer, uint32_t position, const float* q, float* attn_out, uint32_t kv_layer, uint32_t kv_start,
                         float softcap = 0.f) {
        run_flash_attn_split_reduce(layer, position, kv_layer, kv_start, q, attn_out, softcap);
    }
    void step_attention(uint32_t layer, uint32_t position, const float* q, float* attn_out) {   // attention.rs:599-625
        run_scalar_attn(layer, position, q, attn_out, layer, 0);
    }
    // run_scalar_attn for callers that must not allocate or pass a workspace: the partials live in the library's own
    // static device array (one per GPU; calls that overlap in time on one GPU race)
    void run_scalar_attn_static(uint32_t layer, uint32_t position, const float* q, float* attn_out, uint32_t kv_layer,
                                uint32_t kv_start, float softcap = 0.f) {
        check(vfkv_decode_attention_static(kv_cache.handle(), layer, kv_layer, n_heads, q, attn_out, position, kv_start,
                                           scale_for(layer), softcap, stream));
    }
    // step_kv_write + step_attention of one token (attention.rs:546-625) in one call; the decode worker writes the
    // new rows itself where it can
    void step_kv_write_attention(uint32_t layer, uint32_t position, const float* q, const float* k_src, const float* v_src,
                                 float* attn_out, uint32_t kv_start = 0, float softcap = 0.f) {
        check(vfkv_kv_write_decode_attention(kv_cache.handle(), layer, n_heads, q, k_src, v_src, attn_out, position, kv_start,
                                             scale_for(layer), softcap, ws_, stream));
    }
    // step_q_norm_rope + step_k_norm_rope + step_kv_write + step_attention of one decode token (attention.rs:360-625) in one
    // call: q and k_src are the rows before norm and rotation; q_out / k_out receive what the reference leaves in q_buf / k_buf
    void step_qk_rope_kv_write_attention(uint32_t layer, uint32_t position, const float* q, const float* q_norm_weight,
                                         float* q_out, const float* k_src, const float* v_src, const float* k_norm_weight,
                                         const vfkv_rope_params& rope, float* attn_out, uint32_t kv_start = 0, float softcap = 0.f,
                                         const float* freq_factors = nullptr, float* k_out = nullptr) {
        check(vfkv_qk_rope_kv_write_decode_attention(kv_cache.handle(), layer, n_heads, q, q_norm_weight, q_out, k_src, v_src,
                                                     k_norm_weight, freq_factors, &rope, k_out, attn_out, position, kv_start,
                                                     scale_for(layer), softcap, ws_, stream));
    }
    // runs.rs:933-1010
    void run_flash_attn_batch(uint32_t layer, const float* q_buf, float* o_buf, uint32_t m, uint32_t q_start, uint32_t n_kv,
                              uint32_t kv_layer, uint32_t kv_start, float softcap = 0.f) {
        vfkv_batch_params p{n_heads, kv_cache.kv_heads_for(layer), kv_cache.head_dim_for(layer), m, n_kv, q_start,
                            scale_for(layer), kv_start};
        const uint64_t off = kv_cache.layer_offset_bytes(kv_layer);
        check(vfkv_flash_attn_batch(q_buf, (const char*)kv_cache.k_buffer() + off, (const char*)kv_cache.v_buffer() + off,
                                    (uint32_t)kv_cache.kv_dtype, o_buf, &p, softcap, stream));
    }
    // attention.rs:2192-2219 + the run_flash_attn_batch route (:2383-2390)
    void b_step_attention(uint32_t layer, uint32_t base_pos, uint32_t seq_len, const float* q, float* o, uint32_t kv_layer,
                          uint32_t kv_start_window, float softcap = 0.f) {
        check(vfkv_prefill_attention(kv_cache.handle(), layer, kv_layer, n_heads, q, o, seq_len, base_pos, kv_start_window,
                                     scale_for(layer), softcap, stream));
    }
    // the same with the call's precision options (VFKV_PREFILL_F16_WEIGHTS | VFKV_PREFILL_FP8_SCORES | VFKV_PREFILL_F16_QUERIES):
    // faster, weights to 11 bits / scores through the FP8 matrix instruction / queries to 11 bits; bounds in include/vfkv.h
    void b_step_attention_opt(uint32_t layer, uint32_t base_pos, uint32_t seq_len, const float* q, float* o, uint32_t kv_layer,
                              uint32_t kv_start_window, uint32_t options, float softcap = 0.f) {
        check(vfkv_prefill_attention_opt(kv_cache.handle(), layer, kv_layer, n_heads, q, o, seq_len, base_pos, kv_start_window,
                                         scale_for(layer), softcap, options, nullptr, stream));
    }
    // the same with the decode workspace: short chunks over long histories cut the keys into chunks over workgroups
    void b_step_attention_ws(uint32_t layer, uint32_t base_pos, uint32_t seq_len, const float* q, float* o, uint32_t kv_layer,
                             uint32_t kv_start_window, float softcap = 0.f) {
        check(vfkv_prefill_attention_ws(kv_cache.handle(), layer, kv_layer, n_heads, q, o, seq_len, base_pos, kv_start_window,
                                        scale_for(layer), softcap, ws_, stream));
    }
    // runs.rs:2649-2681
    void run_sigmoid_mul(const float* gate, float* inout, uint32_t ne, uint32_t chunk, uint32_t stride, uint32_t gate_offset) {
        const vfkv_gate g{gate, chunk, stride, gate_offset};
        check(vfkv_sigmoid_mul(&g, inout, ne, stream));
    }
    // attention.rs:632-680 (one token: the gate sits behind Q in q_buf) and :2405-2444 (per (token, head) slices [Q | G])
    void step_attn_gated_output(float* attn_out, const float* q_buf, uint32_t q_dim) { run_sigmoid_mul(q_buf, attn_out, q_dim, q_dim, q_dim, q_dim); }
    void b_step_attn_gated_output(float* batch_attn_out, const float* batch_qgate, uint32_t seq_len, uint32_t head_dim) {
        run_sigmoid_mul(batch_qgate, batch_attn_out, seq_len * n_heads * head_dim, head_dim, 2 * head_dim, head_dim);
    }
    // (step_kv_write +) step_attention + step_attn_gated_output as one call; k_src / v_src may be NULL
    void step_attention_gated(uint32_t layer, uint32_t kv_layer, uint32_t position, const float* q, const float* k_src,
                              const float* v_src, float* attn_out, const vfkv_gate& gate, uint32_t kv_start = 0, float softcap = 0.f) {
        check(vfkv_decode_attention_gated(kv_cache.handle(), layer, kv_layer, n_heads, q, k_src, v_src, attn_out, position, kv_start,
                                          scale_for(layer), softcap, &gate, ws_, stream));
    }
    void b_step_attention_gated(uint32_t layer, uint32_t base_pos, uint32_t seq_len, const float* q, float* o, uint32_t kv_layer,
                                uint32_t kv_start_window, const vfkv_gate& gate, float softcap = 0.f) {
        check(vfkv_prefill_attention_gated(kv_cache.handle(), layer, kv_layer, n_heads, q, o, seq_len, base_pos, kv_start_window,
                                           scale_for(layer), softcap, &gate, stream));
    }

    float scale_for(uint32_t layer) const {   // runs.rs:746-760 without the Gemma-4 special case (pass scale = 1 explicitly)
        const uint32_t hd = kv_cache.head_dim_for(layer);
        return hd == kv_cache.config.head_dim ? attn_scale : 1.0f / std::sqrt((float)hd);
    }

private:
    vfkv_workspace* ws_ = nullptr;
};

}  // namespace vfkv
