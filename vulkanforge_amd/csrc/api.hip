// extern "C" boundary of libvfkv: the cache object (KvCache, kv_cache.rs:204-500), the scratch
// workspace (forward/setup.rs:203-230) and one entry point per reference dispatch helper
// (forward/runs.rs).  Host code only; the kernels live in the other translation units.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/vfkv.h"
#include "device_utils.h"
#include "kernels.h"

namespace {

thread_local char g_err[512] = "";
// Advisory of the last attention call on this thread (vfkv_last_note): never an error, never touches g_err.
thread_local char g_note[256] = "";

void note_generic(const char* who, uint32_t dtype, uint32_t head_dim) {
    snprintf(g_note, sizeof(g_note), "%s: this shape (kv dtype %u, head_dim %u, or unaligned pointers / a layer slab of 2 GiB or more) "
             "ran on the generic fallback kernel, 50-100x slower than the tiled kernels", who, dtype, head_dim);
}

int fail(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(e == hipErrorNoDevice ? VFKV_ERR_NO_DEVICE : VFKV_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define VFKV_HIP(call)                                  \
    do {                                                \
        hipError_t e_ = (call);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #call); \
    } while (0)

inline bool mul_ovf(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_mul_overflow(a, b, r); }
inline bool add_ovf(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_add_overflow(a, b, r); }
inline uint64_t esize(uint32_t dtype) { return vfkv::elem_size(dtype); }
inline hipStream_t S(vfkv_stream s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace

struct vfkv_cache {
    uint32_t n_layers, n_kv_heads, head_dim, max_seq_len, dtype;
    std::vector<uint32_t> per_layer_head_dim;     // empty = uniform
    std::vector<uint32_t> per_layer_n_kv_heads;   // empty = uniform
    std::vector<uint64_t> layer_byte_offsets;     // n_layers + 1 entries when heterogeneous, else empty
    uint64_t bytes;                               // per buffer
    void* k;
    void* v;
    void* v_alloc;                                // what hipMalloc returned for V when the cache owns its buffers
    bool owns;
    uint32_t current_seq_len;
};

struct vfkv_workspace {
    uint32_t n_heads, head_dim, max_tiles;
    float* scratch_out;
    float* scratch_max;
    float* scratch_sum;
    float* q_rot;          // n_heads * head_dim floats: rotated queries of vfkv_qk_rope_kv_write_decode_attention when the caller
                           // does not want them and the shape takes the separate RoPE launch
};

// Decode partials of vfkv_decode_attention_static: device memory that exists from the moment the library is loaded, so
// the call needs no allocation.  Every GPU holds its own copy at its own address; host code never uses the array's
// name as an address, only what hipGetSymbolAddress returned for the current device (static_scratch() below).
static __device__ __align__(256) unsigned char scratch[VFKV_STATIC_SCRATCH_BYTES];

namespace {

// KvCache::new size arithmetic (kv_cache.rs:224-291).
int build_layout(const vfkv_cache_config* cfg, vfkv_cache* c) {
    if (!cfg) return fail(VFKV_ERR_INVALID_ARG, "cache config is NULL");
    if (cfg->dtype > VFKV_F8E4M3) return fail(VFKV_ERR_INVALID_ARG, "unknown kv dtype %u", cfg->dtype);
    if (cfg->n_layers == 0) return fail(VFKV_ERR_INVALID_ARG, "n_layers must be > 0");
    c->n_layers = cfg->n_layers;
    c->n_kv_heads = cfg->n_kv_heads;
    c->head_dim = cfg->head_dim;
    c->max_seq_len = cfg->max_seq_len;
    c->dtype = cfg->dtype;
    c->current_seq_len = 0;
    const uint64_t es = esize(cfg->dtype);
    const bool hetero = cfg->per_layer_head_dim || cfg->per_layer_n_kv_heads;
    if (hetero) {
        if (cfg->per_layer_head_dim) c->per_layer_head_dim.assign(cfg->per_layer_head_dim, cfg->per_layer_head_dim + cfg->n_layers);
        if (cfg->per_layer_n_kv_heads) c->per_layer_n_kv_heads.assign(cfg->per_layer_n_kv_heads, cfg->per_layer_n_kv_heads + cfg->n_layers);
        c->layer_byte_offsets.reserve((size_t)cfg->n_layers + 1);
        uint64_t acc = 0;
        c->layer_byte_offsets.push_back(0);
        for (uint32_t i = 0; i < cfg->n_layers; ++i) {
            const uint64_t hd = cfg->per_layer_head_dim ? cfg->per_layer_head_dim[i] : cfg->head_dim;
            const uint64_t kvh = cfg->per_layer_n_kv_heads ? cfg->per_layer_n_kv_heads[i] : cfg->n_kv_heads;
            uint64_t b;
            if (mul_ovf(cfg->max_seq_len, kvh, &b) || mul_ovf(b, hd, &b) || mul_ovf(b, es, &b))
                return fail(VFKV_ERR_OVERFLOW, "kv-cache per-layer size overflow");
            if (add_ovf(acc, b, &acc)) return fail(VFKV_ERR_OVERFLOW, "kv-cache total size overflow");
            c->layer_byte_offsets.push_back(acc);
        }
        c->bytes = acc;
    } else {
        uint64_t t;
        if (mul_ovf(cfg->n_layers, cfg->n_kv_heads, &t) || mul_ovf(t, cfg->max_seq_len, &t) ||
            mul_ovf(t, cfg->head_dim, &t) || mul_ovf(t, es, &t))
            return fail(VFKV_ERR_OVERFLOW, "kv-cache size overflow");
        c->bytes = t;
    }
    return VFKV_OK;
}

inline uint32_t hd_for(const vfkv_cache* c, uint32_t layer) {
    return c->per_layer_head_dim.empty() ? c->head_dim : c->per_layer_head_dim[layer];
}
inline uint32_t kvh_for(const vfkv_cache* c, uint32_t layer) {
    return c->per_layer_n_kv_heads.empty() ? c->n_kv_heads : c->per_layer_n_kv_heads[layer];
}
inline uint64_t layer_off(const vfkv_cache* c, uint32_t layer) {
    if (!c->layer_byte_offsets.empty()) return c->layer_byte_offsets[layer];
    return (uint64_t)layer * c->n_kv_heads * c->max_seq_len * c->head_dim * esize(c->dtype);
}
inline uint64_t row_b(const vfkv_cache* c, uint32_t layer) {
    return (uint64_t)kvh_for(c, layer) * hd_for(c, layer) * esize(c->dtype);
}

// The kernels fold the softmax scale into the exponent (max(x) * scale), which needs a positive finite scale.
int check_scale(float scale, const char* who) {
    if (!(scale > 0.f) || !(scale < __builtin_inff()))
        return fail(VFKV_ERR_INVALID_ARG, "%s: scale must be positive and finite (got %g)", who, (double)scale);
    return VFKV_OK;
}

// A layer that reads another layer's slab (cross-layer KV share) must agree with it on the row geometry: the slab is
// addressed with the reading layer's head_dim and n_kv_heads.
int check_kv_layer(const vfkv_cache* c, uint32_t layer, uint32_t kv_layer, const char* who) {
    if (kv_layer != layer && (hd_for(c, layer) != hd_for(c, kv_layer) || kvh_for(c, layer) != kvh_for(c, kv_layer)))
        return fail(VFKV_ERR_INVALID_ARG, "%s: layer %u (%u kv heads x %u) cannot read the slab of kv_layer %u (%u kv heads x %u)", who,
                    layer, kvh_for(c, layer), hd_for(c, layer), kv_layer, kvh_for(c, kv_layer), hd_for(c, kv_layer));
    return VFKV_OK;
}

int check_attn_dims(uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim) {
    if (n_heads == 0 || n_kv_heads == 0 || head_dim == 0)
        return fail(VFKV_ERR_INVALID_ARG, "n_heads, n_kv_heads and head_dim must be > 0");
    if (n_heads % n_kv_heads != 0)
        return fail(VFKV_ERR_INVALID_ARG, "n_heads (%u) is not a multiple of n_kv_heads (%u)", n_heads, n_kv_heads);
    if (head_dim > 512) return fail(VFKV_ERR_UNSUPPORTED, "head_dim %u > 512 (flash_attn_split.comp:127-132)", head_dim);
    return VFKV_OK;
}

}  // namespace

extern "C" {

const char* vfkv_status_string(int status) {
    switch (status) {
        case VFKV_OK: return "ok";
        case VFKV_ERR_INVALID_ARG: return "invalid argument";
        case VFKV_ERR_OVERFLOW: return "size overflow";
        case VFKV_ERR_ALIGNMENT: return "misaligned offset";
        case VFKV_ERR_UNSUPPORTED: return "unsupported shape";
        case VFKV_ERR_HIP: return "HIP runtime error";
        case VFKV_ERR_NO_DEVICE: return "no HIP device";
        case VFKV_ERR_WORKSPACE: return "workspace too small";
        default: return "unknown status";
    }
}

const char* vfkv_last_error(void) { return g_err; }
uint32_t vfkv_abi_version(void) { return VFKV_ABI_VERSION; }

int vfkv_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

// ---- cache ---------------------------------------------------------------------------------------
int vfkv_cache_create_external(const vfkv_cache_config* cfg, void* k_buffer, void* v_buffer, vfkv_cache** out) {
    if (!out) return fail(VFKV_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    vfkv_cache* c = new (std::nothrow) vfkv_cache();
    if (!c) return fail(VFKV_ERR_HIP, "host allocation failed");
    const int rc = build_layout(cfg, c);
    if (rc != VFKV_OK) { delete c; return rc; }
    c->k = k_buffer;
    c->v = v_buffer;
    c->v_alloc = nullptr;
    c->owns = false;
    *out = c;
    return VFKV_OK;
}

// Not an error, but worth telling the caller: K and V buffers whose addresses agree in bits 7-8 cost the attention
// kernels up to 8 % (see vfkv_cache_create).
const char* vfkv_cache_kv_alignment_note(const vfkv_cache* c) {
    if (c && c->k && c->v && ((((uintptr_t)c->k) ^ ((uintptr_t)c->v)) & 0x180u) == 0u)
        return "k_buffer and v_buffer have the same alignment modulo 512 bytes; offsetting v_buffer by 256 bytes inside its "
               "allocation makes decode attention up to 8 % faster";
    return "";
}

const char* vfkv_last_note(void) { return g_note; }

int vfkv_cache_create(const vfkv_cache_config* cfg, vfkv_cache** out) {
    if (!out) return fail(VFKV_ERR_INVALID_ARG, "out is NULL");
    vfkv_cache* c = nullptr;
    const int rc = vfkv_cache_create_external(cfg, nullptr, nullptr, &c);
    if (rc != VFKV_OK) return rc;
    *out = nullptr;
    if (c->bytes == 0) { delete c; return fail(VFKV_ERR_INVALID_ARG, "kv-cache size is zero"); }
    // K and V of one cache row are requested together by every attention kernel.  When the two addresses
    // agree in bits 7-8 (two allocations of the same alignment, same offset inside the row) the requests of one
    // 128-byte column of the row collide in the memory system and that column's reads run ~17 % slower; V
    // therefore starts 256 bytes into its allocation.
    constexpr size_t v_skew = 256;
    hipError_t e = hipMalloc(&c->k, c->bytes);
    if (e == hipSuccess) {
        e = hipMalloc(&c->v_alloc, c->bytes + v_skew);
        if (e != hipSuccess) { (void)hipFree(c->k); c->k = nullptr; }
    }
    if (e != hipSuccess) { delete c; return hip_fail(e, "hipMalloc(kv cache)"); }
    c->v = (char*)c->v_alloc + v_skew;
    c->owns = true;
    *out = c;
    return VFKV_OK;
}

void vfkv_cache_destroy(vfkv_cache* c) {
    if (!c) return;
    if (c->owns) {
        if (c->k) (void)hipFree(c->k);
        if (c->v_alloc) (void)hipFree(c->v_alloc);
    }
    delete c;
}

int vfkv_cache_zero_fill(vfkv_cache* c, vfkv_stream stream) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "cache has no buffers");
    VFKV_HIP(vfkv::launch_zero_bytes(c->k, c->bytes, S(stream)));
    VFKV_HIP(vfkv::launch_zero_bytes(c->v, c->bytes, S(stream)));
    return VFKV_OK;
}

int vfkv_cache_zero_layer(vfkv_cache* c, uint32_t layer, vfkv_stream stream) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "cache has no buffers");
    if (layer >= c->n_layers) return fail(VFKV_ERR_INVALID_ARG, "layer %u out of range", layer);
    const uint64_t off = layer_off(c, layer);
    const uint64_t size = (uint64_t)c->max_seq_len * row_b(c, layer);
    if (size == 0) return VFKV_OK;
    VFKV_HIP(vfkv::launch_zero_bytes((char*)c->k + off, size, S(stream)));
    VFKV_HIP(vfkv::launch_zero_bytes((char*)c->v + off, size, S(stream)));
    return VFKV_OK;
}

uint32_t vfkv_cache_current_seq_len(const vfkv_cache* c) { return c ? c->current_seq_len : 0u; }
void vfkv_cache_set_current_seq_len(vfkv_cache* c, uint32_t n) { if (c) c->current_seq_len = n; }
void vfkv_cache_reset(vfkv_cache* c) { if (c) c->current_seq_len = 0; }
void* vfkv_cache_k_ptr(const vfkv_cache* c) { return c ? c->k : nullptr; }
void* vfkv_cache_v_ptr(const vfkv_cache* c) { return c ? c->v : nullptr; }
uint32_t vfkv_cache_dtype(const vfkv_cache* c) { return c ? c->dtype : 0u; }
uint64_t vfkv_cache_bytes_per_buffer(const vfkv_cache* c) { return c ? c->bytes : 0u; }
uint32_t vfkv_cache_head_dim_for(const vfkv_cache* c, uint32_t layer) { return (c && layer < c->n_layers) ? hd_for(c, layer) : 0u; }
uint32_t vfkv_cache_kv_heads_for(const vfkv_cache* c, uint32_t layer) { return (c && layer < c->n_layers) ? kvh_for(c, layer) : 0u; }
uint64_t vfkv_cache_layer_offset_bytes(const vfkv_cache* c, uint32_t layer) { return (c && layer < c->n_layers) ? layer_off(c, layer) : 0u; }
uint64_t vfkv_cache_layer_offset_elems(const vfkv_cache* c, uint32_t layer) {
    return (c && layer < c->n_layers) ? layer_off(c, layer) / esize(c->dtype) : 0u;
}
uint64_t vfkv_cache_row_bytes(const vfkv_cache* c, uint32_t layer) { return (c && layer < c->n_layers) ? row_b(c, layer) : 0u; }
uint64_t vfkv_cache_pos_offset_bytes(const vfkv_cache* c, uint32_t layer, uint32_t pos) {
    return (c && layer < c->n_layers) ? layer_off(c, layer) + (uint64_t)pos * row_b(c, layer) : 0u;
}
uint64_t vfkv_cache_layer_size_bytes(const vfkv_cache* c, uint32_t layer) {
    return (c && layer < c->n_layers) ? (uint64_t)c->max_seq_len * row_b(c, layer) : 0u;
}

uint64_t vfkv_kv_bytes_per_token(uint32_t n_layers, uint32_t n_kv_heads, uint32_t head_dim,
                                 const uint32_t* per_layer_head_dim, const uint32_t* per_layer_n_kv_heads,
                                 uint64_t elem_size) {
    uint64_t elems = 0;
    for (uint32_t i = 0; i < n_layers; ++i) {
        const uint64_t hd = per_layer_head_dim ? per_layer_head_dim[i] : head_dim;
        const uint64_t kvh = per_layer_n_kv_heads ? per_layer_n_kv_heads[i] : n_kv_heads;
        uint64_t p;
        if (mul_ovf(kvh, hd, &p)) p = UINT64_MAX;
        if (add_ovf(elems, p, &elems)) elems = UINT64_MAX;
    }
    uint64_t r;
    if (mul_ovf(elems, elem_size, &r) || mul_ovf(r, 2u, &r)) return UINT64_MAX;
    return r;
}

int vfkv_guard_kv_precision(int is_gemma4_moe, uint32_t dtype, int force) {
    if (!is_gemma4_moe || dtype == VFKV_F8E4M3) return VFKV_OK;
    if (force) {
        fprintf(stderr, "vfkv: warning: gemma-4-MoE with %s KV is known-broken in the reference; proceeding (forced)\n",
                dtype == VFKV_F16 ? "FP16" : "FP32");
        return VFKV_OK;
    }
    return fail(VFKV_ERR_UNSUPPORTED,
                "gemma-4-MoE requires an FP8 (E4M3) KV cache; %s KV is known-broken for this model",
                dtype == VFKV_F16 ? "FP16" : "FP32");
}

uint32_t vfkv_kv_start_decode(uint32_t position, uint32_t sliding_window) {
    const uint64_t seq = (uint64_t)position + 1u;
    return seq > sliding_window ? (uint32_t)(seq - sliding_window) : 0u;
}

uint32_t vfkv_kv_start_batch(uint32_t base_pos, uint32_t seq_len, uint32_t window) {
    if (window == 0u) return 0u;
    const uint64_t end = (uint64_t)base_pos + seq_len;
    return end > window ? (uint32_t)(end - window) : 0u;
}

uint32_t vfkv_kv_read_layer(const uint32_t* kv_source, uint32_t n_layers, uint32_t layer) {
    if (!kv_source || layer >= n_layers) return layer;
    uint32_t want;
    switch (kv_source[layer]) {
        case VFKV_KV_SUBSCRIBES_SLIDING: want = VFKV_KV_OWN_PUBLISHES_SLIDING; break;
        case VFKV_KV_SUBSCRIBES_FULL: want = VFKV_KV_OWN_PUBLISHES_FULL; break;
        default: return layer;
    }
    for (uint32_t i = 0; i < n_layers; ++i)
        if (kv_source[i] == want) return i;
    return layer;
}

void vfkv_build_kv_sources(const uint8_t* is_sliding, uint32_t n_pattern, uint32_t first_kv_shared, uint32_t n_layers,
                           uint32_t* kv_source_out) {
    if (!kv_source_out) return;
    auto sliding = [&](uint32_t i) { return !is_sliding || i >= n_pattern || is_sliding[i] != 0; };
    int64_t last_sliding = -1, last_full = -1;
    for (uint32_t i = 0; i < first_kv_shared; ++i) (sliding(i) ? last_sliding : last_full) = i;
    for (uint32_t i = 0; i < n_layers; ++i) {
        if (i >= first_kv_shared) kv_source_out[i] = sliding(i) ? VFKV_KV_SUBSCRIBES_SLIDING : VFKV_KV_SUBSCRIBES_FULL;
        else if ((int64_t)i == last_sliding) kv_source_out[i] = VFKV_KV_OWN_PUBLISHES_SLIDING;
        else if ((int64_t)i == last_full) kv_source_out[i] = VFKV_KV_OWN_PUBLISHES_FULL;
        else kv_source_out[i] = VFKV_KV_OWN;
    }
}

uint32_t vfkv_prefix_reuse_start(const uint32_t* cached_tokens, uint32_t n_cached, const uint32_t* tokens,
                                 uint32_t n_tokens) {
    if (!cached_tokens || !tokens || n_tokens == 0u) return 0u;
    uint32_t k = 0;
    while (k < n_cached && k < n_tokens && cached_tokens[k] == tokens[k]) ++k;
    return k < n_tokens - 1u ? k : n_tokens - 1u;
}

// ---- append / expansion ----------------------------------------------------------------------------
static int append_one(uint32_t dtype, const float* src, void* dst, uint32_t n, uint64_t off, vfkv_stream stream,
                      const char* what) {
    if (n == 0) return VFKV_OK;
    if (!src || !dst) return fail(VFKV_ERR_INVALID_ARG, "%s: NULL buffer", what);
    if (off % 4u != 0u) return fail(VFKV_ERR_ALIGNMENT, "%s: dst_byte_offset must be uint-aligned (got %llu)", what, (unsigned long long)off);
    if ((((uintptr_t)dst) & 3u) != 0u || (((uintptr_t)src) & 3u) != 0u)
        return fail(VFKV_ERR_ALIGNMENT, "%s: buffers must be 4-byte aligned", what);
    char* d = (char*)dst + off;
    VFKV_HIP(vfkv::launch_kv_append(dtype, src, src, d, d, n, 1, S(stream)));
    return VFKV_OK;
}

int vfkv_store_fp8(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset, vfkv_stream stream) {
    return append_one(vfkv::kF8, src, dst, n_elements, dst_byte_offset, stream, "kv_store_fp8");
}

int vfkv_copy_fp16(const float* src, void* dst, uint32_t n_elements, uint64_t dst_byte_offset, vfkv_stream stream) {
    return append_one(vfkv::kF16, src, dst, n_elements, dst_byte_offset, stream, "kv_copy_fp16");
}

int vfkv_fp8_to_f16(const void* src, void* dst_f16, uint64_t n_elems, vfkv_stream stream) {
    if (n_elems == 0) return VFKV_OK;
    if (!src || !dst_f16) return fail(VFKV_ERR_INVALID_ARG, "kv_fp8_to_f16: NULL buffer");
    if ((((uintptr_t)dst_f16) & 1u) != 0u) return fail(VFKV_ERR_ALIGNMENT, "kv_fp8_to_f16: dst must be 2-byte aligned");
    VFKV_HIP(vfkv::launch_fp8_to_f16(src, dst_f16, n_elems, S(stream)));
    return VFKV_OK;
}

int vfkv_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens, const float* k_src,
                  const float* v_src, vfkv_stream stream) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "kv_write: cache has no buffers");
    if (layer >= c->n_layers) return fail(VFKV_ERR_INVALID_ARG, "kv_write: layer %u out of range", layer);
    if (n_tokens == 0) return VFKV_OK;
    if (!k_src || !v_src) return fail(VFKV_ERR_INVALID_ARG, "kv_write: NULL source");
    if ((uint64_t)pos + n_tokens > c->max_seq_len)
        return fail(VFKV_ERR_INVALID_ARG, "kv_write: positions [%u, %llu) exceed max_seq_len %u", pos,
                    (unsigned long long)pos + n_tokens, c->max_seq_len);
    const uint64_t kv_dim = (uint64_t)kvh_for(c, layer) * hd_for(c, layer);
    const uint64_t n = kv_dim * n_tokens;
    if (n > UINT32_MAX) return fail(VFKV_ERR_OVERFLOW, "kv_write: %llu elements exceed the u32 element count", (unsigned long long)n);
    const uint64_t off = layer_off(c, layer) + (uint64_t)pos * row_b(c, layer);
    if (off % 4u != 0u) return fail(VFKV_ERR_ALIGNMENT, "kv_write: dst_byte_offset must be uint-aligned (got %llu)", (unsigned long long)off);
    VFKV_HIP(vfkv::launch_kv_append(c->dtype, k_src, v_src, (char*)c->k + off, (char*)c->v + off, (uint32_t)n, 2, S(stream)));
    return VFKV_OK;
}

static int rope_kv_write_impl(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens, const float* q, uint32_t n_heads,
                              const float* q_norm_weight, float* q_out, const float* k_src, const float* v_src,
                              const float* k_norm_weight, const int32_t* positions, const float* freq_factors,
                              const vfkv_rope_params* p, float* k_out, vfkv_stream stream) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: cache has no buffers");
    if (!p) return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: params is NULL");
    if (layer >= c->n_layers) return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: layer %u out of range", layer);
    if (n_tokens == 0) return VFKV_OK;
    if (!k_src || !v_src) return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: NULL source");
    if ((uint64_t)pos + n_tokens > c->max_seq_len)
        return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: positions [%u, %llu) exceed max_seq_len %u", pos,
                    (unsigned long long)pos + n_tokens, c->max_seq_len);
    const uint32_t hd = hd_for(c, layer), kvh = kvh_for(c, layer);
    if (p->rope_mode != VFKV_ROPE_NORM && p->rope_mode != VFKV_ROPE_NEOX)
        return fail(VFKV_ERR_UNSUPPORTED, "k_rope_kv_write: rope_mode %u (0 = NORM and 2 = NEOX are built)", p->rope_mode);
    if (p->rotary_dim % 2u != 0u || p->rotary_dim > hd)
        return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: rotary_dim %u must be even and <= head_dim %u", p->rotary_dim, hd);
    if (hd > 512u || hd % 4u != 0u)
        return fail(VFKV_ERR_UNSUPPORTED, "k_rope_kv_write: head_dim %u (multiples of 4 up to 512 are built)", hd);
    if (!(p->freq_scale > 0.f)) return fail(VFKV_ERR_INVALID_ARG, "k_rope_kv_write: freq_scale must be > 0");
    const uint64_t off = layer_off(c, layer) + (uint64_t)pos * row_b(c, layer);
    vfkv::RopeAppendLaunch L;
    L.k_src = k_src; L.v_src = v_src; L.weight = k_norm_weight; L.positions = positions; L.freq_factors = freq_factors;
    L.q_src = q; L.q_weight = q_norm_weight; L.q_out = q_out; L.n_q_heads = q ? n_heads : 0u;
    L.k_out = k_out; L.k_dst = (char*)c->k + off; L.v_dst = (char*)c->v + off;
    L.dtype = c->dtype; L.n_tokens = n_tokens; L.n_kv_heads = kvh; L.head_dim = hd; L.rotary_dim = p->rotary_dim;
    L.mode = p->rope_mode; L.pos0 = pos; L.row_bytes = row_b(c, layer);
    L.theta_scale = p->theta_scale; L.freq_scale = p->freq_scale; L.attn_factor = p->attn_factor; L.eps = p->eps;
    VFKV_HIP(vfkv::launch_rope_append(L, S(stream)));
    return VFKV_OK;
}

int vfkv_k_rope_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens, const float* k_src,
                         const float* v_src, const float* k_norm_weight, const int32_t* positions,
                         const float* freq_factors, const vfkv_rope_params* p, float* k_out, vfkv_stream stream) {
    return rope_kv_write_impl(c, layer, pos, n_tokens, nullptr, 0, nullptr, nullptr, k_src, v_src, k_norm_weight, positions,
                              freq_factors, p, k_out, stream);
}

int vfkv_qk_rope_kv_write(vfkv_cache* c, uint32_t layer, uint32_t pos, uint32_t n_tokens, uint32_t n_heads, const float* q,
                          const float* q_norm_weight, float* q_out, const float* k_src, const float* v_src,
                          const float* k_norm_weight, const int32_t* positions, const float* freq_factors,
                          const vfkv_rope_params* p, float* k_out, vfkv_stream stream) {
    if (n_tokens != 0 && (!q || !q_out)) return fail(VFKV_ERR_INVALID_ARG, "qk_rope_kv_write: NULL query buffer");
    if (n_heads == 0) return fail(VFKV_ERR_INVALID_ARG, "qk_rope_kv_write: n_heads must be > 0");
    return rope_kv_write_impl(c, layer, pos, n_tokens, q, n_heads, q_norm_weight, q_out, k_src, v_src, k_norm_weight, positions,
                              freq_factors, p, k_out, stream);
}

int vfkv_rms_norm_mul_rope(const float* qk, const float* weight, float* qk_out, uint32_t head_dim,
                           uint32_t heads_per_token, uint32_t m, const int32_t* positions, uint32_t pos0,
                           const float* freq_factors, const vfkv_rope_params* p, vfkv_stream stream) {
    if (!p) return fail(VFKV_ERR_INVALID_ARG, "rms_norm_mul_rope: params is NULL");
    if (m == 0 || heads_per_token == 0) return VFKV_OK;
    if (!qk || !qk_out) return fail(VFKV_ERR_INVALID_ARG, "rms_norm_mul_rope: NULL buffer");
    if (p->rope_mode != VFKV_ROPE_NORM && p->rope_mode != VFKV_ROPE_NEOX)
        return fail(VFKV_ERR_UNSUPPORTED, "rms_norm_mul_rope: rope_mode %u (0 = NORM and 2 = NEOX are built)", p->rope_mode);
    if (p->rotary_dim % 2u != 0u || p->rotary_dim > head_dim)
        return fail(VFKV_ERR_INVALID_ARG, "rms_norm_mul_rope: rotary_dim %u must be even and <= head_dim %u", p->rotary_dim, head_dim);
    if (head_dim == 0u || head_dim > 512u || head_dim % 4u != 0u)
        return fail(VFKV_ERR_UNSUPPORTED, "rms_norm_mul_rope: head_dim %u (multiples of 4 up to 512 are built)", head_dim);
    if (!(p->freq_scale > 0.f)) return fail(VFKV_ERR_INVALID_ARG, "rms_norm_mul_rope: freq_scale must be > 0");
    if (heads_per_token > 65535u * 4u) return fail(VFKV_ERR_UNSUPPORTED, "rms_norm_mul_rope: %u heads per token", heads_per_token);
    vfkv::RopeAppendLaunch L;
    L.k_src = qk; L.weight = weight; L.positions = positions; L.freq_factors = freq_factors; L.k_out = qk_out;
    L.dtype = vfkv::kF32; L.n_tokens = m; L.n_kv_heads = heads_per_token; L.head_dim = head_dim; L.rotary_dim = p->rotary_dim;
    L.mode = p->rope_mode; L.pos0 = pos0;
    L.theta_scale = p->theta_scale; L.freq_scale = p->freq_scale; L.attn_factor = p->attn_factor; L.eps = p->eps;
    VFKV_HIP(vfkv::launch_rope_append(L, S(stream)));
    return VFKV_OK;
}

// ---- decode attention ----------------------------------------------------------------------------------
static int flash_attn_split_impl(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                                 float* scratch_out, float* scratch_max, float* scratch_sum, const vfkv_split_params* p,
                                 uint32_t tile, float softcap, bool interleave, vfkv_stream stream) {
    if (!p) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: params is NULL");
    if (!q || !k_layer || !v_layer || !scratch_out || !scratch_max || !scratch_sum)
        return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: NULL buffer");
    if (kv_dtype > VFKV_F8E4M3) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: unknown kv dtype %u", kv_dtype);
    int rc = check_attn_dims(p->n_heads, p->n_kv_heads, p->head_dim);
    if (rc != VFKV_OK) return rc;
    if (p->seq_len == 0) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: seq_len must be > 0");
    if (tile == 0 || tile % 16u != 0u || tile > 65536u)
        return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: tile must be a multiple of 16 in [16, 65536] (got %u)", tile);
    const uint32_t need = (p->seq_len + tile - 1u) / tile;
    if (p->n_tiles != need)
        return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: n_tiles (%u) != ceil(seq_len / tile) (%u)", p->n_tiles, need);
    if (!(softcap >= 0.f)) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_split: softcap must be >= 0");
    rc = check_scale(p->scale, "flash_attn_split");
    if (rc != VFKV_OK) return rc;
    vfkv::SplitLaunch L;
    L.q = q; L.k = k_layer; L.v = v_layer;
    L.scratch_out = scratch_out; L.scratch_max = scratch_max; L.scratch_sum = scratch_sum;
    L.dtype = kv_dtype; L.n_heads = p->n_heads; L.n_kv_heads = p->n_kv_heads; L.head_dim = p->head_dim;
    L.seq_len = p->seq_len; L.kv_start = p->kv_start; L.tile = tile; L.tile_first = 0; L.n_tiles = p->n_tiles;
    L.scale = p->scale; L.softcap = softcap; L.interleave = interleave;
    bool generic = false;
    g_note[0] = '\0';
    VFKV_HIP(vfkv::launch_split(L, S(stream), &generic));
    if (generic) note_generic("flash_attn_split", kv_dtype, p->head_dim);
    return VFKV_OK;
}

int vfkv_flash_attn_split(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                          float* scratch_out, float* scratch_max, float* scratch_sum, const vfkv_split_params* p,
                          uint32_t tile, float softcap, vfkv_stream stream) {
    return flash_attn_split_impl(q, k_layer, v_layer, kv_dtype, scratch_out, scratch_max, scratch_sum, p, tile, softcap,
                                 false, stream);
}

int vfkv_flash_attn_split_interleaved(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype,
                                      float* scratch_out, float* scratch_max, float* scratch_sum,
                                      const vfkv_split_params* p, uint32_t tile, float softcap, vfkv_stream stream) {
    return flash_attn_split_impl(q, k_layer, v_layer, kv_dtype, scratch_out, scratch_max, scratch_sum, p, tile, softcap,
                                 true, stream);
}

int vfkv_flash_attn_reduce(const float* scratch_out, const float* scratch_max, const float* scratch_sum, float* o,
                           uint32_t n_heads, uint32_t head_dim, uint32_t n_tiles, vfkv_stream stream) {
    if (!scratch_out || !scratch_max || !scratch_sum || !o) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_reduce: NULL buffer");
    if (n_heads == 0 || head_dim == 0 || n_tiles == 0)
        return fail(VFKV_ERR_INVALID_ARG, "flash_attn_reduce: n_heads, head_dim and n_tiles must be > 0");
    if (head_dim > 512) return fail(VFKV_ERR_UNSUPPORTED, "flash_attn_reduce: head_dim %u > 512", head_dim);
    VFKV_HIP(vfkv::launch_reduce(scratch_out, scratch_max, scratch_sum, o, n_heads, head_dim, n_tiles, S(stream)));
    return VFKV_OK;
}

int vfkv_workspace_create(uint32_t n_heads, uint32_t head_dim, uint32_t max_seq_len, vfkv_workspace** out) {
    if (!out) return fail(VFKV_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (n_heads == 0 || head_dim == 0 || max_seq_len == 0)
        return fail(VFKV_ERR_INVALID_ARG, "workspace: n_heads, head_dim and max_seq_len must be > 0");
    vfkv_workspace* w = new (std::nothrow) vfkv_workspace();
    if (!w) return fail(VFKV_ERR_HIP, "host allocation failed");
    w->n_heads = n_heads;
    w->head_dim = head_dim;
    w->max_tiles = (max_seq_len + 63u) / 64u;   // setup.rs:208-230
    uint64_t n_out;
    if (mul_ovf((uint64_t)n_heads * w->max_tiles, head_dim, &n_out) || n_out > (UINT64_MAX / 8)) {
        delete w;
        return fail(VFKV_ERR_OVERFLOW, "workspace size overflow");
    }
    const uint64_t n_ml = (uint64_t)n_heads * w->max_tiles;
    // one allocation: [out | max | sum], each 256-byte aligned
    const uint64_t out_b = (n_out * 4u + 255u) & ~255ull, ml_b = (n_ml * 4u + 255u) & ~255ull;
    void* base = nullptr;
    const uint64_t q_b = ((uint64_t)n_heads * head_dim * 4u + 255u) & ~255ull;
    hipError_t e = hipMalloc(&base, out_b + 2u * ml_b + q_b);
    if (e != hipSuccess) { delete w; return hip_fail(e, "hipMalloc(workspace)"); }
    w->scratch_out = (float*)base;
    w->scratch_max = (float*)((char*)base + out_b);
    w->scratch_sum = (float*)((char*)base + out_b + ml_b);
    w->q_rot = (float*)((char*)base + out_b + 2u * ml_b);
    *out = w;
    return VFKV_OK;
}

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* ptr[kMaxDevices] = {};
    int dev = -1;
    VFKV_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(VFKV_ERR_UNSUPPORTED, "decode_attention_static: device index %d", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void* p = nullptr;
        VFKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(VFKV_ERR_HIP, "decode_attention_static: hipGetSymbolAddress returned NULL");
        ptr[dev] = p;
    }
    *out = ptr[dev];
    return VFKV_OK;
}

void vfkv_workspace_destroy(vfkv_workspace* w) {
    if (!w) return;
    if (w->scratch_out) (void)hipFree(w->scratch_out);
    delete w;
}

// Compute units of the current device, asked once (256 on MI355X; the same figure when no device answers, so that the
// layout-only helpers keep working on a host without a GPU).
static uint32_t device_cus() {
    static const uint32_t n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            return 256u;
        return (uint32_t)cus;
    }();
    return n;
}

// Tile length for the convenience path: enough workgroups to cover the CUs once (matrix-core worker) or twice, tiles a
// multiple of 64 keys (so they never exceed the workspace's ceil(max_seq / 64) rows).
// VFKV_DECODE_TILE: keys per workgroup forced by the environment (0: the library chooses)
static uint32_t forced_tile() {
    static const uint32_t forced = [] {
        const char* e = getenv("VFKV_DECODE_TILE");
        const uint32_t v = e ? (uint32_t)strtoul(e, nullptr, 10) : 0u;
        return (v >= 64u && v % 64u == 0u) ? v : 0u;
    }();
    return forced;
}

static uint32_t choose_tile(uint32_t span, uint32_t n_kv_heads, uint32_t groups, uint32_t target_wgs) {
    if (forced_tile() != 0u) return forced_tile();
    uint32_t tiles = (target_wgs + n_kv_heads * groups - 1u) / (n_kv_heads * groups);
    if (tiles == 0u) tiles = 1u;
    uint32_t tile = (span + tiles - 1u) / tiles;
    tile = ((tile + 63u) / 64u) * 64u;
    if (tile < 64u) tile = 64u;
    return tile;
}

uint32_t vfkv_decode_tile_for(uint32_t span, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t kv_dtype) {
    if (span == 0u || n_kv_heads == 0u || n_heads == 0u || n_heads % n_kv_heads != 0u) return 0u;
    const uint32_t g = n_heads / n_kv_heads;
    // The matrix-core worker (1- and 2-byte caches, head_dim 64 / 128) runs best with one workgroup per CU and
    // serves up to 8 heads of a group per workgroup; the vector-ALU worker wants two and serves up to 4.
    const bool mfma = (kv_dtype == VFKV_F8E4M3 || kv_dtype == VFKV_F16) &&
                      (head_dim == 64u || head_dim == 128u || head_dim == 256u || head_dim == 512u ||
                       vfkv::split_padded_dim(kv_dtype, head_dim) != 0u);
    if (mfma) {
        // short spans: one tile, so the worker writes the output itself and no merge launch follows.  The tile's runs of 32
        // keys are walked by the workgroup's four run streams (two at head_dim 512) one after the other, and a further round
        // costs more than the merge launch saves: up to two rounds (one at head_dim 512: 8 / 1 / 512 F16 over 256 keys took
        // 22.7 us in one tile against 13.6 us in four).
        static const bool forced = getenv("VFKV_DECODE_TILE") != nullptr;
        if (span <= (head_dim == 512u ? 64u : 256u) && !forced) return 256u;
        return choose_tile(span, n_kv_heads, (g + 7u) / 8u, device_cus());
    }
    // F32 caches on the f32 matrix instruction: one workgroup per CU as well, up to 16 heads of a group per workgroup
    static const bool valu_forced = [] { const char* e = getenv("VFKV_DECODE_WORKER"); return e && e[0] == 'v'; }();
    if (kv_dtype == VFKV_F32 && !valu_forced &&
        (head_dim == 64u || head_dim == 128u || head_dim == 256u || vfkv::split_padded_dim(kv_dtype, head_dim) != 0u)) {
        static const bool forced = getenv("VFKV_DECODE_TILE") != nullptr;
        if (span <= 256u && !forced) return 256u;
        return choose_tile(span, n_kv_heads, (g + 15u) / 16u, device_cus());
    }
    const uint32_t groups = (g % 4u == 0u) ? g / 4u : (g % 2u == 0u) ? g / 2u : g;
    return choose_tile(span, n_kv_heads, groups, 2u * device_cus());
}

static int decode_attention_impl(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                                 uint32_t position, uint32_t kv_start, float scale, float softcap, vfkv_workspace* ws,
                                 const float* k_new, const float* v_new, vfkv_stream stream, const char* who,
                                 const vfkv::GateArgs* gate = nullptr, bool static_ws = false, const vfkv::RopeFold* rope = nullptr,
                                 const vfkv_rope_params* rope_params = nullptr) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "%s: cache has no buffers", who);
    if (!ws && !static_ws) return fail(VFKV_ERR_INVALID_ARG, "%s: workspace is NULL", who);
    if (!q || !o) return fail(VFKV_ERR_INVALID_ARG, "%s: NULL buffer", who);
    if (layer >= c->n_layers || kv_layer >= c->n_layers)
        return fail(VFKV_ERR_INVALID_ARG, "%s: layer %u / kv_layer %u out of range", who, layer, kv_layer);
    if (position >= c->max_seq_len)
        return fail(VFKV_ERR_INVALID_ARG, "%s: position %u >= max_seq_len %u", who, position, c->max_seq_len);
    if (!(softcap >= 0.f)) return fail(VFKV_ERR_INVALID_ARG, "%s: softcap must be >= 0", who);
    const uint32_t hd = hd_for(c, layer), kvh = kvh_for(c, layer);
    int rc = check_attn_dims(n_heads, kvh, hd);
    if (rc != VFKV_OK) return rc;
    if ((rc = check_scale(scale, who)) != VFKV_OK) return rc;
    if ((rc = check_kv_layer(c, layer, kv_layer, who)) != VFKV_OK) return rc;
    const uint32_t seq_len = position + 1u;
    if (kv_start >= seq_len) return fail(VFKV_ERR_INVALID_ARG, "%s: kv_start %u leaves no visible key (seq_len %u)", who, kv_start, seq_len);
    if (ws && (n_heads > ws->n_heads || hd > ws->head_dim))
        return fail(VFKV_ERR_WORKSPACE, "%s: workspace built for %u heads x %u dims, need %u x %u", who,
                    ws->n_heads, ws->head_dim, n_heads, hd);
    uint32_t tile = vfkv_decode_tile_for(seq_len - kv_start, n_heads, kvh, hd, c->dtype);
    uint32_t first = kv_start / tile;
    uint32_t n_tiles = (seq_len + tile - 1u) / tile - first;
    const uint64_t off = layer_off(c, kv_layer);
    vfkv::SplitLaunch L;
    L.q = q; L.k = (char*)c->k + off; L.v = (char*)c->v + off;
    L.dtype = c->dtype; L.n_heads = n_heads; L.n_kv_heads = kvh; L.head_dim = hd;
    L.seq_len = seq_len; L.kv_start = kv_start; L.tile = tile; L.tile_first = first; L.n_tiles = n_tiles;
    L.scale = scale; L.softcap = softcap;
    // the partials stay inside the workspace, so they need not correspond to tiles
    L.interleave = true;
    // (the choice of worker below depends on whether the token's rotation will be folded into it)
    if (rope) {
        vfkv::SplitLaunch T = L;
        T.k_new = k_new; T.v_new = v_new; T.append_pos = position; T.rope = rope;
        L.rope = vfkv::split_folds_rope(T) ? rope : nullptr;
    }
    // The interleaved worker deals the runs of the span to its workgroups whatever the tile length says: the workgroup count
    // is chosen directly (one per CU, none without a run), and the launch covers the rows from the 64-row boundary at or
    // below kv_start.
    uint32_t heads_per_wg = 8u;
    const uint32_t streams = n_tiles > 1u && forced_tile() == 0u ? vfkv::split_run_streams(L, &heads_per_wg) : 0u;
    if (streams != 0u) {
        const uint32_t run_rows = vfkv::split_run_rows(c->dtype, hd), nz = (n_heads / kvh + heads_per_wg - 1u) / heads_per_wg;
        const uint32_t runs = (seq_len - kv_start / 64u * 64u + run_rows - 1u) / run_rows;
        const uint32_t kvh_wg = vfkv::split_pairs_heads(L) ? kvh / 2u : kvh;      // KV heads (or pairs of them) that get workgroups
        uint32_t wgs = device_cus() / (kvh_wg * nz);
        if (wgs > (runs + streams - 1u) / streams) wgs = (runs + streams - 1u) / streams;   // none without a run
        if (wgs > (seq_len + 63u) / 64u) wgs = (seq_len + 63u) / 64u;   // what a workspace sized for this length holds (head_dim 512: two streams per workgroup)
        if (!static_ws && wgs > ws->max_tiles) wgs = ws->max_tiles;
        if (wgs < 1u) wgs = 1u;
        tile = 64u; first = kv_start / 64u; n_tiles = wgs;
        L.tile = tile; L.tile_first = first; L.n_tiles = n_tiles;
    }
    vfkv_workspace fixed;
    if (static_ws) {
        // the partials of this launch laid out in the static array: [out | max | sum], each part 256-byte aligned
        const uint64_t n_ml = (uint64_t)n_heads * n_tiles;
        const uint64_t out_b = (n_ml * hd * 4u + 255u) & ~255ull, ml_b = (n_ml * 4u + 255u) & ~255ull;
        if (out_b + 2u * ml_b > (uint64_t)VFKV_STATIC_SCRATCH_BYTES)
            return fail(VFKV_ERR_WORKSPACE, "%s: %u heads x %u partials x %u dims need %llu bytes of scratch, the static buffer holds %llu "
                        "(use vfkv_decode_attention with a workspace)", who, n_heads, n_tiles, hd,
                        (unsigned long long)(out_b + 2u * ml_b), (unsigned long long)VFKV_STATIC_SCRATCH_BYTES);
        void* base = nullptr;
        rc = static_scratch(&base);
        if (rc != VFKV_OK) return rc;
        fixed.n_heads = n_heads; fixed.head_dim = hd; fixed.max_tiles = n_tiles;
        fixed.scratch_out = (float*)base;
        fixed.scratch_max = (float*)((char*)base + out_b);
        fixed.scratch_sum = (float*)((char*)base + out_b + ml_b);
        fixed.q_rot = nullptr;
        ws = &fixed;
    }
    if (n_tiles > ws->max_tiles) return fail(VFKV_ERR_WORKSPACE, "%s: %u tiles > workspace capacity %u", who, n_tiles, ws->max_tiles);
    L.scratch_out = ws->scratch_out; L.scratch_max = ws->scratch_max; L.scratch_sum = ws->scratch_sum;
    // Q / K norm + RoPE of the token: inside the worker where it can (then q and k_new are the rows before rotation), else
    // as the launch of its own that vfkv_qk_rope_kv_write makes (which also appends)
    if (rope) {
        L.k_new = k_new; L.v_new = v_new; L.append_pos = position; L.rope = rope;
        if (!vfkv::split_folds_rope(L)) {
            float* const q_rot = rope->q_out ? rope->q_out : ws->q_rot;
            if (!q_rot) return fail(VFKV_ERR_WORKSPACE, "%s: no room for the rotated queries (give q_out)", who);
            rc = rope_kv_write_impl(c, layer, position, 1, q, n_heads, rope->q_weight, q_rot, k_new, v_new, rope->k_weight, nullptr,
                                    rope->freq_factors, rope_params, rope->k_out, stream);
            if (rc != VFKV_OK) return rc;
            L.q = q_rot; L.rope = nullptr; L.k_new = nullptr; L.v_new = nullptr; k_new = nullptr;
        }
    }
    if (k_new) {
        L.k_new = k_new; L.v_new = v_new; L.append_pos = position;
        if (!vfkv::split_appends(L)) {          // this shape's worker cannot write the row itself: append in its own launch
            L.k_new = nullptr; L.v_new = nullptr;
            rc = vfkv_kv_write(c, layer, position, 1, k_new, v_new, stream);
            if (rc != VFKV_OK) return rc;
        }
    }
    bool generic = false;
    g_note[0] = '\0';
    if (vfkv::split_writes_output(L) && ((uintptr_t)o & 15u) == 0u) {   // one tile sees every key: the worker normalises and writes o itself
        L.o_direct = o;
        VFKV_HIP(vfkv::launch_split(L, S(stream)));
        if (gate) VFKV_HIP(vfkv::launch_sigmoid_mul(o, n_heads * hd, *gate, S(stream)));
        return VFKV_OK;
    }
    VFKV_HIP(vfkv::launch_split(L, S(stream), &generic));
    if (generic) note_generic(who, c->dtype, hd);
    bool gate_applied = false;
    VFKV_HIP(vfkv::launch_reduce(ws->scratch_out, ws->scratch_max, ws->scratch_sum, o, n_heads, hd, n_tiles, S(stream), gate,
                                 &gate_applied));
    if (gate && !gate_applied) VFKV_HIP(vfkv::launch_sigmoid_mul(o, n_heads * hd, *gate, S(stream)));
    return VFKV_OK;
}

int vfkv_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                          uint32_t position, uint32_t kv_start, float scale, float softcap, vfkv_workspace* ws,
                          vfkv_stream stream) {
    return decode_attention_impl(c, layer, kv_layer, n_heads, q, o, position, kv_start, scale, softcap, ws, nullptr, nullptr,
                                 stream, "decode_attention");
}

int vfkv_decode_attention_static(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                                 uint32_t position, uint32_t kv_start, float scale, float softcap, vfkv_stream stream) {
    return decode_attention_impl(c, layer, kv_layer, n_heads, q, o, position, kv_start, scale, softcap, nullptr, nullptr, nullptr,
                                 stream, "decode_attention_static", nullptr, true);
}

int vfkv_kv_write_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t n_heads, const float* q, const float* k_src,
                                   const float* v_src, float* o, uint32_t position, uint32_t kv_start, float scale,
                                   float softcap, vfkv_workspace* ws, vfkv_stream stream) {
    if (!k_src || !v_src) return fail(VFKV_ERR_INVALID_ARG, "kv_write_decode_attention: NULL source row");
    if (c && layer < c->n_layers && (layer_off(c, layer) + (uint64_t)position * row_b(c, layer)) % 4u != 0u)
        return fail(VFKV_ERR_ALIGNMENT, "kv_write_decode_attention: dst_byte_offset must be uint-aligned");
    return decode_attention_impl(c, layer, layer, n_heads, q, o, position, kv_start, scale, softcap, ws, k_src, v_src, stream,
                                 "kv_write_decode_attention");
}

int vfkv_qk_rope_kv_write_decode_attention(vfkv_cache* c, uint32_t layer, uint32_t n_heads, const float* q,
                                           const float* q_norm_weight, float* q_out, const float* k_src, const float* v_src,
                                           const float* k_norm_weight, const float* freq_factors, const vfkv_rope_params* p,
                                           float* k_out, float* o, uint32_t position, uint32_t kv_start, float scale, float softcap,
                                           vfkv_workspace* ws, vfkv_stream stream) {
    const char* who = "qk_rope_kv_write_decode_attention";
    if (!p) return fail(VFKV_ERR_INVALID_ARG, "%s: params is NULL", who);
    if (!k_src || !v_src) return fail(VFKV_ERR_INVALID_ARG, "%s: NULL source row", who);
    if (!c || layer >= c->n_layers) return fail(VFKV_ERR_INVALID_ARG, "%s: layer out of range", who);
    const uint32_t hd = hd_for(c, layer);
    if (p->rope_mode != VFKV_ROPE_NORM && p->rope_mode != VFKV_ROPE_NEOX)
        return fail(VFKV_ERR_UNSUPPORTED, "%s: rope_mode %u (0 = NORM and 2 = NEOX are built)", who, p->rope_mode);
    if (p->rotary_dim % 2u != 0u || p->rotary_dim > hd)
        return fail(VFKV_ERR_INVALID_ARG, "%s: rotary_dim %u must be even and <= head_dim %u", who, p->rotary_dim, hd);
    if (!(p->freq_scale > 0.f)) return fail(VFKV_ERR_INVALID_ARG, "%s: freq_scale must be > 0", who);
    if ((layer_off(c, layer) + (uint64_t)position * row_b(c, layer)) % 4u != 0u)
        return fail(VFKV_ERR_ALIGNMENT, "%s: dst_byte_offset must be uint-aligned", who);
    if (q_out != nullptr && q != nullptr) {
        const uintptr_t a0 = (uintptr_t)q, a1 = a0 + (uintptr_t)n_heads * hd * 4u, b0 = (uintptr_t)q_out, b1 = b0 + (uintptr_t)n_heads * hd * 4u;
        if (a0 < b1 && b0 < a1) return fail(VFKV_ERR_INVALID_ARG, "%s: q_out must not overlap q (every workgroup reads q while one writes q_out)", who);
    }
    vfkv::RopeFold rf;
    rf.q_weight = q_norm_weight; rf.k_weight = k_norm_weight; rf.freq_factors = freq_factors; rf.q_out = q_out; rf.k_out = k_out;
    rf.rotary_dim = p->rotary_dim; rf.mode = p->rope_mode; rf.theta_scale = p->theta_scale; rf.freq_scale = p->freq_scale;
    rf.attn_factor = p->attn_factor; rf.eps = p->eps;
    return decode_attention_impl(c, layer, layer, n_heads, q, o, position, kv_start, scale, softcap, ws, k_src, v_src, stream, who,
                                 nullptr, false, &rf, p);
}

// ---- prefill attention -------------------------------------------------------------------------------
static int flash_attn_batch_impl(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype, float* o,
                                 const vfkv_batch_params* p, float softcap, vfkv_workspace* ws, vfkv_stream stream,
                                 const vfkv::GateArgs* gate = nullptr, uint32_t options = 0u) {
    if ((options & ~(VFKV_PREFILL_F16_WEIGHTS | VFKV_PREFILL_FP8_SCORES | VFKV_PREFILL_F16_QUERIES)) != 0u) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: unknown option bits 0x%x", options);
    if (!p) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: params is NULL");
    if (!q || !k_layer || !v_layer || !o) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: NULL buffer");
    if (kv_dtype > VFKV_F8E4M3) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: unknown kv dtype %u", kv_dtype);
    int rc = check_attn_dims(p->n_heads, p->n_kv_heads, p->head_dim);
    if (rc != VFKV_OK) return rc;
    if (p->m == 0) return VFKV_OK;
    if (p->n_kv == 0) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: n_kv must be > 0");
    if (!(softcap >= 0.f)) return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: softcap must be >= 0");
    if ((rc = check_scale(p->scale, "flash_attn_batch")) != VFKV_OK) return rc;
    const uint64_t first_len = (uint64_t)p->q_start + 1u;
    const uint64_t vis0 = first_len < p->n_kv ? first_len : p->n_kv;
    if (p->kv_start >= vis0)
        return fail(VFKV_ERR_INVALID_ARG, "flash_attn_batch: kv_start %u leaves query 0 without a visible key", p->kv_start);
    if (gate && (uint64_t)p->m * p->n_heads * p->head_dim > 0xFFFFFFFFull)
        return fail(VFKV_ERR_OVERFLOW, "prefill_attention_gated: %llu output elements",
                    (unsigned long long)p->m * p->n_heads * p->head_dim);
    vfkv::BatchLaunch L;
    L.gate = gate;
    L.q = q; L.k = k_layer; L.v = v_layer; L.o = o;
    L.dtype = kv_dtype; L.n_heads = p->n_heads; L.n_kv_heads = p->n_kv_heads; L.head_dim = p->head_dim;
    L.m = p->m; L.n_kv = p->n_kv; L.q_start = p->q_start; L.kv_start = p->kv_start;
    L.scale = p->scale; L.softcap = softcap;
    L.f16_weights = (options & VFKV_PREFILL_F16_WEIGHTS) != 0u;
    L.fp8_scores = (options & VFKV_PREFILL_FP8_SCORES) != 0u;
    L.f16_queries = (options & VFKV_PREFILL_F16_QUERIES) != 0u;
    if (ws) {
        L.scratch_out = ws->scratch_out; L.scratch_max = ws->scratch_max; L.scratch_sum = ws->scratch_sum;
        L.scratch_ml_floats = (uint64_t)ws->n_heads * ws->max_tiles;
        L.scratch_out_floats = L.scratch_ml_floats * ws->head_dim;
    }
    bool generic = false;
    g_note[0] = '\0';
    VFKV_HIP(vfkv::launch_batch(L, S(stream), &generic));
    if (generic) note_generic("flash_attn_batch", kv_dtype, p->head_dim);
    return VFKV_OK;
}

int vfkv_flash_attn_batch(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype, float* o,
                          const vfkv_batch_params* p, float softcap, vfkv_stream stream) {
    return flash_attn_batch_impl(q, k_layer, v_layer, kv_dtype, o, p, softcap, nullptr, stream);
}

int vfkv_flash_attn_batch_opt(const float* q, const void* k_layer, const void* v_layer, uint32_t kv_dtype, float* o,
                              const vfkv_batch_params* p, float softcap, uint32_t options, vfkv_stream stream) {
    return flash_attn_batch_impl(q, k_layer, v_layer, kv_dtype, o, p, softcap, nullptr, stream, nullptr, options);
}

static int prefill_attention_impl(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                                  uint32_t m, uint32_t base_pos, uint32_t window, float scale, float softcap,
                                  vfkv_workspace* ws, vfkv_stream stream, const vfkv::GateArgs* gate = nullptr,
                                  uint32_t options = 0u) {
    if (!c || !c->k || !c->v) return fail(VFKV_ERR_INVALID_ARG, "prefill_attention: cache has no buffers");
    if (layer >= c->n_layers || kv_layer >= c->n_layers)
        return fail(VFKV_ERR_INVALID_ARG, "prefill_attention: layer %u / kv_layer %u out of range", layer, kv_layer);
    if ((uint64_t)base_pos + m > c->max_seq_len)
        return fail(VFKV_ERR_INVALID_ARG, "prefill_attention: positions [%u, %llu) exceed max_seq_len %u", base_pos,
                    (unsigned long long)base_pos + m, c->max_seq_len);
    const int rc_kv = check_kv_layer(c, layer, kv_layer, "prefill_attention");
    if (rc_kv != VFKV_OK) return rc_kv;
    vfkv_batch_params p;
    p.n_heads = n_heads;
    p.n_kv_heads = kvh_for(c, layer);
    p.head_dim = hd_for(c, layer);
    p.m = m;
    p.n_kv = base_pos + m;
    p.q_start = base_pos;
    p.scale = scale;
    p.kv_start = vfkv_kv_start_batch(base_pos, m, window);
    const uint64_t off = layer_off(c, kv_layer);
    return flash_attn_batch_impl(q, (char*)c->k + off, (char*)c->v + off, c->dtype, o, &p, softcap, ws, stream, gate, options);
}

int vfkv_prefill_attention(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                           uint32_t m, uint32_t base_pos, uint32_t window, float scale, float softcap,
                           vfkv_stream stream) {
    return prefill_attention_impl(c, layer, kv_layer, n_heads, q, o, m, base_pos, window, scale, softcap, nullptr, stream);
}

int vfkv_prefill_attention_ws(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                              uint32_t m, uint32_t base_pos, uint32_t window, float scale, float softcap,
                              vfkv_workspace* ws, vfkv_stream stream) {
    if (!ws) return fail(VFKV_ERR_INVALID_ARG, "prefill_attention_ws: workspace is NULL");
    return prefill_attention_impl(c, layer, kv_layer, n_heads, q, o, m, base_pos, window, scale, softcap, ws, stream);
}

int vfkv_prefill_attention_opt(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                               uint32_t m, uint32_t base_pos, uint32_t window, float scale, float softcap, uint32_t options,
                               vfkv_workspace* ws, vfkv_stream stream) {
    return prefill_attention_impl(c, layer, kv_layer, n_heads, q, o, m, base_pos, window, scale, softcap, ws, stream, nullptr, options);
}

// ---- gated output --------------------------------------------------------------------------------------
static int check_gate(const vfkv_gate* gate, const char* who, vfkv::GateArgs* out) {
    if (!gate || !gate->gate) return fail(VFKV_ERR_INVALID_ARG, "%s: gate is NULL", who);
    if (gate->chunk == 0u) return fail(VFKV_ERR_INVALID_ARG, "%s: gate chunk must be > 0", who);
    if ((((uintptr_t)gate->gate) & 3u) != 0u) return fail(VFKV_ERR_ALIGNMENT, "%s: gate must be 4-byte aligned", who);
    out->gate = gate->gate; out->chunk = gate->chunk; out->stride = gate->stride; out->gate_offset = gate->gate_offset;
    return VFKV_OK;
}

int vfkv_sigmoid_mul(const vfkv_gate* gate, float* data, uint32_t ne, vfkv_stream stream) {
    if (ne == 0u) return VFKV_OK;
    vfkv::GateArgs g;
    const int rc = check_gate(gate, "sigmoid_mul", &g);
    if (rc != VFKV_OK) return rc;
    if (!data) return fail(VFKV_ERR_INVALID_ARG, "sigmoid_mul: NULL buffer");
    if ((((uintptr_t)data) & 3u) != 0u) return fail(VFKV_ERR_ALIGNMENT, "sigmoid_mul: data must be 4-byte aligned");
    VFKV_HIP(vfkv::launch_sigmoid_mul(data, ne, g, S(stream)));
    return VFKV_OK;
}

int vfkv_decode_attention_gated(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q,
                                const float* k_src, const float* v_src, float* o, uint32_t position, uint32_t kv_start,
                                float scale, float softcap, const vfkv_gate* gate, vfkv_workspace* ws, vfkv_stream stream) {
    vfkv::GateArgs g;
    const int rc = check_gate(gate, "decode_attention_gated", &g);
    if (rc != VFKV_OK) return rc;
    if ((k_src == nullptr) != (v_src == nullptr))
        return fail(VFKV_ERR_INVALID_ARG, "decode_attention_gated: k_src and v_src must both be given or both be NULL");
    if (k_src) {
        if (layer != kv_layer) return fail(VFKV_ERR_INVALID_ARG, "decode_attention_gated: a layer that appends reads its own slab (layer %u, kv_layer %u)", layer, kv_layer);
        if (c && layer < c->n_layers && (layer_off(c, layer) + (uint64_t)position * row_b(c, layer)) % 4u != 0u)
            return fail(VFKV_ERR_ALIGNMENT, "decode_attention_gated: dst_byte_offset must be uint-aligned");
    }
    return decode_attention_impl(c, layer, kv_layer, n_heads, q, o, position, kv_start, scale, softcap, ws, k_src, v_src, stream,
                                 "decode_attention_gated", &g);
}

int vfkv_prefill_attention_gated(vfkv_cache* c, uint32_t layer, uint32_t kv_layer, uint32_t n_heads, const float* q, float* o,
                                 uint32_t m, uint32_t base_pos, uint32_t window, float scale, float softcap,
                                 const vfkv_gate* gate, vfkv_stream stream) {
    vfkv::GateArgs g;
    int rc = check_gate(gate, "prefill_attention_gated", &g);
    if (rc != VFKV_OK) return rc;
    return prefill_attention_impl(c, layer, kv_layer, n_heads, q, o, m, base_pos, window, scale, softcap, nullptr, stream, &g);
}

}  // extern "C"
