/*
 * vfkv_oracle.c -- CPU restatement of the reference's KV-cache / attention hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this
 * file; it exists so the HIP kernels can be checked against an independent CPU
 * implementation of the reference's semantics, and so a CPU baseline can be timed.
 *
 * Every function cites the reference source (paths relative to the reference tree) whose
 * behaviour it restates.  How each function is pinned (which known-answer vectors, closed
 * forms or library routines it is checked against) is listed next to it; the checks
 * themselves live in tests/test_oracle_*.py.
 *
 *   function                      restates                                         pinned by
 *   ---------------------------------------------------------------------------------------------
 *   vfo_e4m3_to_f32               src/backend/vulkan/fp8_ext.rs:104-122            reference unit-test vectors (fp8_ext.rs:217-263),
 *                                                                                 torch.float8_e4m3fn decode of all 256 codes
 *   vfo_f32_to_e4m3               src/backend/vulkan/fp8_ext.rs:126-211            reference vectors, torch.float8_e4m3fn casts (|x|<=448),
 *                                                                                 exhaustive code round trip, tie-to-even midpoints,
 *                                                                                 independent ldexp/rint formulation over 2^16 bit patterns
 *   vfo_f32_to_f16 / f16_to_f32   vk_shaders/kv_copy_fp16.comp:46-50 (packHalf)    numpy.float16 over all 2^16 halves and 2^20 random f32
 *   vfo_kv_store_fp8              vk_shaders/kv_store_fp8.comp:42-67               composition of vfo_f32_to_e4m3 + byte order check
 *   vfo_kv_copy_fp16              vk_shaders/kv_copy_fp16.comp:39-51               numpy.float16 view of the written bytes
 *   vfo_kv_fp8_to_f16             vk_shaders/kv_fp8_to_f16.comp:28-33              torch.float8_e4m3fn -> float16 cast of all codes
 *   vfo_layout_*                  src/backend/vulkan/kv_cache.rs:224-291,431-490   reference unit-test figures (kv_cache.rs:518-587)
 *   vfo_attn_decode_ref           tests/correctness.rs:2567-2617                   seq=1 => V[0]; constant-K => mean(V); scipy softmax @ V in
 *                                                                                 f64; reference closed-form generator cases
 *   vfo_attn_split / _reduce      vk_shaders/flash_attn_split.comp:82-162,         == vfo_attn_decode_ref for every tile size (tile
 *                                 vk_shaders/flash_attn_reduce.comp:35-81          invariance, tests/flash_attn_tiled_ref.rs:279-295)
 *   vfo_attn_batch_ref            tests/correctness.rs:3016-3071                   scipy softmax per query; M=1 == decode; causal isolation
 *   vfo_attn_batch_shader         vk_shaders/flash_attn_batch.comp:105-208         == vfo_attn_batch_ref within 1e-4..5e-3 on the reference's cases
 *   vfo_rms_norm_rope             vk_shaders/rms_norm.comp:36-129 (fusion path),   NEOX: the reference's generator case and f32 CPU formula at
 *                                 vk_shaders/rope_funcs.glsl:17-112                positions 0 / 100 / 4096 with its thresholds
 *                                                                                 (tests/correctness.rs:799-884); both modes: numpy complex-
 *                                                                                 rotation formulation, pair-norm invariance, pos=0 identity,
 *                                                                                 additivity of positions; norm: numpy x/sqrt(mean(x^2)+eps)*w
 *                                                                                 (the CPU formula of tests/correctness.rs:665-700).
 *                                                                                 NORM mode (adjacent pairs), partial rotary_dim and frequency
 *                                                                                 factors have no reference test: parity unpinned by the
 *                                                                                 reference, pinned by the formulations above only.
 *   vfo_sigmoid_mul               vk_shaders/sigmoid_mul.comp:40-53                scipy.special.expit in f64 rounded once; g = 0 halves the value,
 *                                                                                 g = +-100 keeps / zeroes it; the index map against a
 *                                                                                 pure-Python loop for the decode form (chunk = stride = offset
 *                                                                                 = q_dim, executor/attention.rs:655-664) and the interleaved
 *                                                                                 per-head form (head_dim, 2 * head_dim, head_dim, :2433-2441).
 *                                                                                 The reference holds no test of this shader: parity unpinned
 *                                                                                 by the reference, pinned by the above only.
 *
 * Extensions that the reference does not implement (so no reference test can pin them):
 *   - `kv_start > 0` on every attention routine follows the shader text
 *     (flash_attn_split.comp:97-113, flash_attn_batch.comp:145-150); pinned by the identity
 *     attention(kv_start=s) == attention over the slab shifted by s rows.
 *   - the attention logit soft-cap  s <- cap * tanh(s / cap)  (applied after *scale, before
 *     max/exp; cap == 0 disables it): parity unpinned by the reference (it has no such
 *     parameter); pinned here only by the closed form against scipy.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define VFO_DTYPE_F32 0u
#define VFO_DTYPE_F16 1u
#define VFO_DTYPE_F8 2u

/* ------------------------------------------------------------------------------------------
 * E4M3FN  (fp8_ext.rs:104-211)
 * ---------------------------------------------------------------------------------------- */

/* fp8_ext.rs:104-122 -- one NaN code per sign (E=15,M=7), no infinities, subnormals M/8*2^-6. */
float vfo_e4m3_to_f32(uint8_t bits) {
    const uint32_t sign = (bits >> 7) & 1u;
    const uint32_t e = (bits >> 3) & 0xFu;
    const uint32_t m = bits & 0x7u;
    const float sf = sign ? -1.0f : 1.0f;
    if (e == 0xFu && m == 0x7u) return sf * NAN;
    if (e == 0u) return sf * ((float)m / 8.0f) * ldexpf(1.0f, -6);
    return sf * (1.0f + (float)m / 8.0f) * ldexpf(1.0f, (int)e - 7);
}

/* fp8_ext.rs:188-211 -- keep the top 3 bits of a 23(+1)-bit significand after shifting right by
 * 20+extra, round to nearest, ties to even.  May return 8 (carry into the exponent). */
static uint32_t round_sig_to_3(uint32_t sig, uint32_t extra) {
    const uint32_t sh = 20u + extra;
    if (sh >= 32u) return 0u;
    const uint32_t kept = sig >> sh;
    const uint32_t half = (sig >> (sh - 1u)) & 1u;
    const uint32_t below = sig & ((1u << (sh - 1u)) - 1u);
    if (half && (below != 0u || (kept & 1u))) return kept + 1u;
    return kept;
}

/* fp8_ext.rs:126-186 -- saturating (|x| >= 448 and +-Inf -> 0x7E|sign), NaN -> 0x7F, RNE,
 * subnormal-aware, underflow to signed zero. */
uint8_t vfo_f32_to_e4m3(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7Fu; /* NaN: sign dropped */
    const uint8_t s = (uint8_t)((u >> 31) << 7);
    const uint32_t au = u & 0x7FFFFFFFu;
    if (au == 0u) return s;
    float ax;
    memcpy(&ax, &au, 4);
    if (ax >= 448.0f) return (uint8_t)(s | 0x7Eu);
    const int e32 = (int)((au >> 23) & 0xFFu);
    const uint32_t man = au & 0x007FFFFFu;
    const int e = e32 - 127 + 7;
    if (e >= 1 && e <= 15) {
        const uint32_t m3 = round_sig_to_3(man, 0u);
        if (m3 == 8u) {
            if (e + 1 == 16) return (uint8_t)(s | 0x7Eu);
            return (uint8_t)(s | (uint8_t)((e + 1) << 3));
        }
        return (uint8_t)(s | (uint8_t)(e << 3) | (uint8_t)m3);
    }
    if (e <= 0) {
        const uint32_t shift = (uint32_t)(1 - e);
        if (shift > 23u) return s;
        const uint32_t m3 = round_sig_to_3(0x00800000u | man, shift);
        if (m3 == 8u) return (uint8_t)(s | 0x08u);
        return (uint8_t)(s | (uint8_t)m3);
    }
    return (uint8_t)(s | 0x7Eu);
}

void vfo_f32_to_e4m3_array(const float* src, uint8_t* dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = vfo_f32_to_e4m3(src[i]);
}
void vfo_e4m3_to_f32_array(const uint8_t* src, float* dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = vfo_e4m3_to_f32(src[i]);
}

/* ------------------------------------------------------------------------------------------
 * IEEE binary16  (packHalf2x16 / unpackHalf2x16, kv_copy_fp16.comp:46-50;
 * CPU-side convention is round-to-nearest-even: tests/coopmat_fa_gemma.rs:74,212)
 * ---------------------------------------------------------------------------------------- */
uint16_t vfo_f32_to_f16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    const uint16_t s = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t au = u & 0x7FFFFFFFu;
    if (au > 0x7F800000u) return (uint16_t)(s | 0x7E00u | ((au >> 13) & 0x03FFu)); /* NaN */
    if (au >= 0x47800000u) return (uint16_t)(s | 0x7C00u); /* >= 65536 or Inf */
    const int e = (int)(au >> 23) - 127;
    uint32_t sig = (au & 0x007FFFFFu) | 0x00800000u;
    uint32_t sh, base;
    if (e >= -14) {          /* normal half */
        sh = 13u;
        base = (uint32_t)(e + 15 - 1) << 10; /* implicit bit adds one more to the exponent field */
    } else {                 /* subnormal half */
        if (e < -25) return s;
        sh = (uint32_t)(13 + (-14 - e));
        base = 0u;
    }
    uint32_t kept = sig >> sh;
    const uint32_t half = (sig >> (sh - 1u)) & 1u;
    const uint32_t below = sig & ((1u << (sh - 1u)) - 1u);
    if (half && (below != 0u || (kept & 1u))) kept += 1u;
    uint32_t h = base + kept;              /* carries ripple into the exponent on their own */
    if (h >= 0x7C00u) h = 0x7C00u;
    return (uint16_t)(s | (uint16_t)h);
}

float vfo_f16_to_f32(uint16_t h) {
    const uint32_t s = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t m = h & 0x3FFu;
    uint32_t u;
    if (e == 0x1Fu) {
        u = s | 0x7F800000u | (m << 13);
    } else if (e == 0u) {
        const float v = ldexpf((float)m, -24);
        memcpy(&u, &v, 4);
        u |= s;
    } else {
        u = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void vfo_f32_to_f16_array(const float* src, uint16_t* dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = vfo_f32_to_f16(src[i]);
}
void vfo_f16_to_f32_array(const uint16_t* src, float* dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = vfo_f16_to_f32(src[i]);
}

/* ------------------------------------------------------------------------------------------
 * KV append / expansion  (kv_store_fp8.comp:42-67, kv_copy_fp16.comp:39-51,
 * kv_fp8_to_f16.comp:28-33).  The GPU writes whole 32-bit words, so a ragged tail is
 * zero-padded to the word; byte 0 / low half is the lowest-indexed element.
 * ---------------------------------------------------------------------------------------- */
int vfo_kv_store_fp8(const float* src, uint8_t* dst_base, uint32_t n, uint64_t dst_byte_off) {
    if (dst_byte_off % 4u) return -1; /* runs.rs:2448-2453 */
    uint8_t* dst = dst_base + dst_byte_off;
    const uint32_t n_words = (n + 3u) / 4u;
    for (uint32_t w = 0; w < n_words; ++w) {
        for (uint32_t j = 0; j < 4u; ++j) {
            const uint32_t i = 4u * w + j;
            dst[i] = (i < n) ? vfo_f32_to_e4m3(src[i]) : 0u; /* floate4m3_t(0.0) == 0x00 */
        }
    }
    return 0;
}

int vfo_kv_copy_fp16(const float* src, uint8_t* dst_base, uint32_t n, uint64_t dst_byte_off) {
    if (dst_byte_off % 4u) return -1; /* runs.rs:2400-2404 */
    uint8_t* dst = dst_base + dst_byte_off;
    const uint32_t n_words = (n + 1u) / 2u;
    for (uint32_t w = 0; w < n_words; ++w) {
        for (uint32_t j = 0; j < 2u; ++j) {
            const uint32_t i = 2u * w + j;
            const uint16_t h = (i < n) ? vfo_f32_to_f16(src[i]) : 0u;
            dst[2u * i] = (uint8_t)(h & 0xFFu);
            dst[2u * i + 1u] = (uint8_t)(h >> 8);
        }
    }
    return 0;
}

void vfo_kv_fp8_to_f16(const uint8_t* src, uint16_t* dst, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = vfo_f32_to_f16(vfo_e4m3_to_f32(src[i]));
}

/* ------------------------------------------------------------------------------------------
 * Cache layout arithmetic  (kv_cache.rs:224-291 allocation, :431-490 offsets, :186-202)
 * per_layer_* may be NULL (uniform).  Returns 0, or -1 on 64-bit overflow.
 * offsets_out (n_layers+1 entries) receives the cumulative byte-offset table.
 * ---------------------------------------------------------------------------------------- */
static int mul_ovf(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_mul_overflow(a, b, r); }
static int add_ovf(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_add_overflow(a, b, r); }

static uint64_t elem_size_of(uint32_t dtype) { return dtype == VFO_DTYPE_F32 ? 4u : dtype == VFO_DTYPE_F16 ? 2u : 1u; }

int vfo_layout_offsets(uint32_t n_layers, uint32_t n_kv_heads, uint32_t head_dim, uint32_t max_seq,
                       const uint32_t* per_layer_head_dim, const uint32_t* per_layer_n_kv_heads,
                       uint32_t dtype, uint64_t* offsets_out) {
    const uint64_t es = elem_size_of(dtype);
    uint64_t acc = 0;
    offsets_out[0] = 0;
    for (uint32_t i = 0; i < n_layers; ++i) {
        const uint64_t hd = per_layer_head_dim ? per_layer_head_dim[i] : head_dim;
        const uint64_t kvh = per_layer_n_kv_heads ? per_layer_n_kv_heads[i] : n_kv_heads;
        uint64_t b;
        if (mul_ovf((uint64_t)max_seq, kvh, &b) || mul_ovf(b, hd, &b) || mul_ovf(b, es, &b)) return -1;
        if (add_ovf(acc, b, &acc)) return -1;
        offsets_out[i + 1] = acc;
    }
    return 0;
}

/* kv_cache.rs:186-202 -- bytes of K+V per context token, saturating. */
uint64_t vfo_kv_bytes_per_token(uint32_t n_layers, uint32_t n_kv_heads, uint32_t head_dim,
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
    if (mul_ovf(elems, elem_size, &r)) return UINT64_MAX;
    if (mul_ovf(r, 2u, &r)) return UINT64_MAX;
    return r;
}

/* gemma4.rs:59-73 -- sliding-window lower bound for decode at `position`. */
uint32_t vfo_kv_start_decode(uint32_t position, uint32_t sliding_window) {
    const uint32_t seq = position + 1u;
    return seq > sliding_window ? seq - sliding_window : 0u;
}
/* executor/attention.rs:2215-2219 -- batch prefill uses the LAST query's window for all rows. */
uint32_t vfo_kv_start_batch(uint32_t base_pos, uint32_t seq_len, uint32_t window) {
    if (window == 0u) return 0u;
    const uint32_t end = base_pos + seq_len;
    return end > window ? end - window : 0u;
}

/* ------------------------------------------------------------------------------------------
 * Element fetch by cache dtype  (flash_attn_split.comp:29-58 load_k/load_v)
 * ---------------------------------------------------------------------------------------- */
static float g_e4m3_lut[256];
static int g_e4m3_lut_ready = 0;
__attribute__((constructor)) static void init_e4m3_lut(void) {
    for (int i = 0; i < 256; ++i) g_e4m3_lut[i] = vfo_e4m3_to_f32((uint8_t)i);
    g_e4m3_lut_ready = 1;
}

static inline float load_kv(const void* base, uint32_t dtype, uint64_t idx) {
    if (dtype == VFO_DTYPE_F32) return ((const float*)base)[idx];
    if (dtype == VFO_DTYPE_F16) return vfo_f16_to_f32(((const uint16_t*)base)[idx]);
    return g_e4m3_lut[((const uint8_t*)base)[idx]]; /* table of vfo_e4m3_to_f32 over all 256 codes */
}

static inline float softcap_f32(float s, float cap) { return cap > 0.0f ? cap * tanhf(s / cap) : s; }

/* ------------------------------------------------------------------------------------------
 * Mathematical decode oracle  (tests/correctness.rs:2567-2617), extended with kv_start and
 * soft-cap.  f64 dot, score rounded to f32 then *scale in f32, f32 exp, f64 sum, one final
 * rounding -- the same mixed precision as the reference function.
 * ---------------------------------------------------------------------------------------- */
void vfo_attn_decode_ref(const float* q, const void* k, const void* v, uint32_t dtype,
                         uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                         uint32_t seq_len, uint32_t kv_start, float scale, float softcap,
                         float* out, int n_threads) {
    const uint32_t g = n_heads / n_kv_heads;
    const uint64_t pos_stride = (uint64_t)n_kv_heads * head_dim;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (uint32_t h = 0; h < n_heads; ++h) {
        const uint32_t kvh = h / g;
        const float* qh = q + (uint64_t)h * head_dim;
        const uint64_t head_off = (uint64_t)kvh * head_dim;
        const uint32_t n = seq_len > kv_start ? seq_len - kv_start : 0u;
        float* scores = (float*)malloc(sizeof(float) * (n ? n : 1u));
        float mx = -INFINITY;
        for (uint32_t i = 0; i < n; ++i) {
            const uint64_t kt = (uint64_t)(kv_start + i) * pos_stride + head_off;
            double s = 0.0;
            for (uint32_t d = 0; d < head_dim; ++d) s += (double)qh[d] * (double)load_kv(k, dtype, kt + d);
            float sf = softcap_f32((float)s * scale, softcap);
            scores[i] = sf;
            if (sf > mx) mx = sf;
        }
        double sum = 0.0;
        for (uint32_t i = 0; i < n; ++i) {
            scores[i] = expf(scores[i] - mx);
            sum += (double)scores[i];
        }
        const float inv = 1.0f / (float)sum;
        float* o = out + (uint64_t)h * head_dim;
        for (uint32_t d = 0; d < head_dim; ++d) {
            double acc = 0.0;
            for (uint32_t i = 0; i < n; ++i) {
                const uint64_t vt = (uint64_t)(kv_start + i) * pos_stride + head_off;
                acc += (double)scores[i] * (double)load_kv(v, dtype, vt + d);
            }
            o[d] = (float)(acc * (double)inv);
        }
        free(scores);
    }
}

/* ------------------------------------------------------------------------------------------
 * Shader-exact split worker  (flash_attn_split.comp:82-162) for an arbitrary tile length
 * (reference TILE = 64): f32 everywhere, d ascending, -1e30 sentinel for masked lanes.
 * scratch_out[(h*n_tiles + j)*D + d], scratch_max/sum[h*n_tiles + j].
 * ---------------------------------------------------------------------------------------- */
void vfo_attn_split(const float* q, const void* k, const void* v, uint32_t dtype,
                    uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                    uint32_t seq_len, uint32_t kv_start, float scale, float softcap,
                    uint32_t tile, uint32_t n_tiles,
                    float* scratch_out, float* scratch_max, float* scratch_sum, int n_threads) {
    const uint32_t g = n_heads / n_kv_heads;
    const uint64_t pos_stride = (uint64_t)n_kv_heads * head_dim;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (uint32_t h = 0; h < n_heads; ++h) {
        const uint32_t kvh = h / g;
        const float* qh = q + (uint64_t)h * head_dim;
        const uint64_t head_off = (uint64_t)kvh * head_dim;
        float* p = (float*)malloc(sizeof(float) * tile);
        for (uint32_t j = 0; j < n_tiles; ++j) {
            const uint64_t base = (uint64_t)j * tile;
            float tmax = -1e30f;
            for (uint32_t i = 0; i < tile; ++i) {
                const uint64_t t = base + i;
                const int valid = (t < seq_len) && (t >= kv_start);
                float sc = -1e30f;
                if (valid) {
                    const uint64_t kt = t * pos_stride + head_off;
                    float s = 0.0f;
                    for (uint32_t d = 0; d < head_dim; ++d) s += qh[d] * load_kv(k, dtype, kt + d);
                    sc = softcap_f32(s * scale, softcap);
                }
                p[i] = sc;
                if (sc > tmax) tmax = sc;
            }
            float tsum = 0.0f;
            for (uint32_t i = 0; i < tile; ++i) {
                const uint64_t t = base + i;
                const int valid = (t < seq_len) && (t >= kv_start);
                p[i] = valid ? expf(p[i] - tmax) : 0.0f;
                tsum += p[i];
            }
            const uint64_t pidx = (uint64_t)h * n_tiles + j;
            float* o = scratch_out + pidx * head_dim;
            for (uint32_t d = 0; d < head_dim; ++d) o[d] = 0.0f;
            const uint64_t rows = base < seq_len ? ((seq_len - base) < tile ? (seq_len - base) : tile) : 0u;
            for (uint64_t i = 0; i < rows; ++i) {
                const uint64_t vt = (base + i) * pos_stride + head_off;
                const float pi = p[i];
                for (uint32_t d = 0; d < head_dim; ++d) o[d] += pi * load_kv(v, dtype, vt + d);
            }
            scratch_max[pidx] = tmax;
            scratch_sum[pidx] = tsum;
        }
        free(p);
    }
}

/* flash_attn_reduce.comp:35-81 -- sequential log-sum-exp merge, M = -1e30, L = 0 at start. */
void vfo_attn_reduce(const float* scratch_out, const float* scratch_max, const float* scratch_sum,
                     uint32_t n_heads, uint32_t head_dim, uint32_t n_tiles, float* out) {
    float* acc = (float*)malloc(sizeof(float) * head_dim);
    for (uint32_t h = 0; h < n_heads; ++h) {
        for (uint32_t d = 0; d < head_dim; ++d) acc[d] = 0.0f;
        float gmax = -1e30f, gsum = 0.0f;
        for (uint32_t j = 0; j < n_tiles; ++j) {
            const uint64_t pidx = (uint64_t)h * n_tiles + j;
            const float tmax = scratch_max[pidx], tsum = scratch_sum[pidx];
            const float nmax = gmax > tmax ? gmax : tmax;
            const float ko = expf(gmax - nmax), kn = expf(tmax - nmax);
            const float* o = scratch_out + pidx * head_dim;
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] = acc[d] * ko + o[d] * kn;
            gsum = gsum * ko + tsum * kn;
            gmax = nmax;
        }
        const float inv = 1.0f / gsum;
        for (uint32_t d = 0; d < head_dim; ++d) out[(uint64_t)h * head_dim + d] = acc[d] * inv;
    }
    free(acc);
}

/* ------------------------------------------------------------------------------------------
 * Mathematical prefill oracle  (tests/correctness.rs:3016-3071): all f64, one final rounding.
 * Extended with kv_start (one lower bound for the whole batch, executor/attention.rs:2215-2219;
 * flash_attn_batch.comp:145-150) and the soft-cap.  Q, O are [m, H, D] row-major f32.
 * ---------------------------------------------------------------------------------------- */
void vfo_attn_batch_ref(const float* q, const void* k, const void* v, uint32_t dtype,
                        uint32_t m, uint32_t n_kv, uint32_t n_heads, uint32_t n_kv_heads,
                        uint32_t head_dim, uint32_t q_start, uint32_t kv_start,
                        float scale, float softcap, float* out, int n_threads) {
    const uint32_t g = n_heads / n_kv_heads;
    const uint64_t pos_stride = (uint64_t)n_kv_heads * head_dim;
    const double scale_d = (double)scale, cap = (double)softcap;
    if (n_threads < 1) n_threads = 1;
    const uint64_t total = (uint64_t)m * n_heads;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 4)
    for (uint64_t idx = 0; idx < total; ++idx) {
        const uint32_t qi = (uint32_t)(idx / n_heads), h = (uint32_t)(idx % n_heads);
        uint32_t causal_len = q_start + qi + 1u;
        if (causal_len > n_kv) causal_len = n_kv;
        const uint32_t lo = kv_start < causal_len ? kv_start : causal_len;
        const uint32_t n = causal_len - lo;
        const uint32_t kvh = h / g;
        const float* qh = q + ((uint64_t)qi * n_heads + h) * head_dim;
        const uint64_t head_off = (uint64_t)kvh * head_dim;
        double* w = (double*)malloc(sizeof(double) * (n ? n : 1u));
        double mx = -INFINITY;
        for (uint32_t i = 0; i < n; ++i) {
            const uint64_t kt = (uint64_t)(lo + i) * pos_stride + head_off;
            double dot = 0.0;
            for (uint32_t d = 0; d < head_dim; ++d) dot += (double)qh[d] * (double)load_kv(k, dtype, kt + d);
            double s = dot * scale_d;
            if (cap > 0.0) s = cap * tanh(s / cap);
            w[i] = s;
            if (s > mx) mx = s;
        }
        double sum = 0.0;
        for (uint32_t i = 0; i < n; ++i) {
            w[i] = exp(w[i] - mx);
            sum += w[i];
        }
        for (uint32_t i = 0; i < n; ++i) w[i] /= sum;
        float* o = out + ((uint64_t)qi * n_heads + h) * head_dim;
        for (uint32_t d = 0; d < head_dim; ++d) {
            double acc = 0.0;
            for (uint32_t i = 0; i < n; ++i) {
                const uint64_t vt = (uint64_t)(lo + i) * pos_stride + head_off;
                acc += w[i] * (double)load_kv(v, dtype, vt + d);
            }
            o[d] = (float)acc;
        }
        free(w);
    }
}

/* ------------------------------------------------------------------------------------------
 * Shader-exact batched attention  (flash_attn_batch.comp:105-208): f32, 64-key tiles starting
 * at window_lo = (kv_start/64)*64, online max/sum with -1e30 sentinel.
 * ---------------------------------------------------------------------------------------- */
void vfo_attn_batch_shader(const float* q, const void* k, const void* v, uint32_t dtype,
                           uint32_t m, uint32_t n_kv, uint32_t n_heads, uint32_t n_kv_heads,
                           uint32_t head_dim, uint32_t q_start, uint32_t kv_start,
                           float scale, float softcap, float* out, int n_threads) {
    enum { TILE = 64 };
    const uint32_t g = n_heads / n_kv_heads;
    const uint64_t pos_stride = (uint64_t)n_kv_heads * head_dim;
    if (n_threads < 1) n_threads = 1;
    const uint64_t total = (uint64_t)m * n_heads;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 4)
    for (uint64_t idx = 0; idx < total; ++idx) {
        const uint32_t qi = (uint32_t)(idx / n_heads), h = (uint32_t)(idx % n_heads);
        uint32_t causal_len = q_start + qi + 1u;
        if (causal_len > n_kv) causal_len = n_kv;
        const uint32_t kvh = h / g;
        const float* qh = q + ((uint64_t)qi * n_heads + h) * head_dim;
        const uint64_t head_off = (uint64_t)kvh * head_dim;
        float* acc = (float*)calloc(head_dim, sizeof(float));
        float my_max = -1e30f, my_sum = 0.0f;
        float p[TILE];
        for (uint32_t base = (kv_start / TILE) * TILE; base < causal_len; base += TILE) {
            float tmax = -1e30f;
            for (uint32_t i = 0; i < TILE; ++i) {
                const uint32_t t = base + i;
                const int valid = (t < causal_len) && (t >= kv_start);
                float sc = -1e30f;
                if (valid) {
                    const uint64_t kt = (uint64_t)t * pos_stride + head_off;
                    float s = 0.0f;
                    for (uint32_t d = 0; d < head_dim; ++d) s += qh[d] * load_kv(k, dtype, kt + d);
                    sc = softcap_f32(s * scale, softcap);
                }
                p[i] = sc;
                if (sc > tmax) tmax = sc;
            }
            const float nmax = my_max > tmax ? my_max : tmax;
            const float kf = expf(my_max - nmax);
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] *= kf;
            my_sum *= kf;
            float tsum = 0.0f;
            for (uint32_t i = 0; i < TILE; ++i) {
                const uint32_t t = base + i;
                const int valid = (t < causal_len) && (t >= kv_start);
                p[i] = valid ? expf(p[i] - nmax) : 0.0f;
                tsum += p[i];
            }
            my_sum += tsum;
            my_max = nmax;
            const uint32_t rows = (causal_len - base) < TILE ? (causal_len - base) : TILE;
            for (uint32_t i = 0; i < rows; ++i) {
                const uint64_t vt = (uint64_t)(base + i) * pos_stride + head_off;
                const float pi = p[i];
                for (uint32_t d = 0; d < head_dim; ++d) acc[d] += pi * load_kv(v, dtype, vt + d);
            }
        }
        const float inv = 1.0f / my_sum;
        float* o = out + ((uint64_t)qi * n_heads + h) * head_dim;
        for (uint32_t d = 0; d < head_dim; ++d) o[d] = acc[d] * inv;
        free(acc);
    }
}

/* ------------------------------------------------------------------------------------------
 * K (or Q) RMS-norm * weight followed by RoPE, the step in front of the KV append
 * (rms_norm.comp:36-129 with RMS_NORM_ROPE_FUSION, rope_funcs.glsl:17-112; host: run_rms_norm_mul_rope
 * runs.rs:2492-2600, run_rope_neox_with_pos_offset runs.rs:647-720).
 *
 * x, out: [m][heads][head_dim] f32 (out may alias x).  weight: [head_dim] or NULL (plain RoPE).
 * pos: [m] token positions.  ff: [n_dims / 2] frequency factors or NULL.  mode 0 = NORM: pairs
 * (i0, i0 + 1); mode 2 = NEOX: pairs (i0 / 2, i0 / 2 + n_dims / 2); dims >= n_dims pass through.
 * The reference's callers pass freq_scale = 1, ext_factor = 0 (no YaRN ramp), attn_factor = 1; the
 * ext_factor != 0 branch of rope_yarn is not restated.
 *
 * Arithmetic: the shader works in f32 (sum of squares by a tree, theta = pos * pow(theta_scale, i0/2),
 * cos / sin of the GPU).  Here the sum of squares is accumulated in f64, theta is formed in f32 exactly
 * as the shader writes it (so the angle is the same number), and the trigonometry and the rotation are
 * evaluated in f64 and rounded once.
 * ---------------------------------------------------------------------------------------- */
void vfo_rms_norm_rope(const float* x, const float* weight, const int32_t* pos, const float* ff, float* out,
                       uint32_t m, uint32_t heads, uint32_t head_dim, uint32_t mode, uint32_t n_dims,
                       float theta_scale, float freq_scale, float attn_factor, float eps) {
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t t = 0; t < m; ++t)
        for (uint32_t h = 0; h < heads; ++h) {
            const float* row = x + ((size_t)t * heads + h) * head_dim;
            float* dst = out + ((size_t)t * heads + h) * head_dim;
            float* y = (float*)malloc(sizeof(float) * head_dim);
            if (weight) {                                   /* rms_norm.comp:61-112 */
                double ss = 0.0;
                for (uint32_t d = 0; d < head_dim; ++d) ss += (double)row[d] * (double)row[d];
                const float mean = (float)(ss / (double)head_dim);
                const float scale = (float)(1.0 / sqrt((double)mean + (double)eps));
                for (uint32_t d = 0; d < head_dim; ++d) y[d] = (scale * row[d]) * weight[d];
            } else {
                for (uint32_t d = 0; d < head_dim; ++d) y[d] = row[d];
            }
            for (uint32_t d = 0; d < head_dim; ++d) dst[d] = y[d];          /* dims >= n_dims: rope_funcs.glsl:56-61,90-95 */
            for (uint32_t i0 = 0; i0 + 1 < n_dims; i0 += 2) {
                const float theta_base = (float)pos[t] * powf(theta_scale, (float)i0 / 2.0f);   /* :63,97 */
                const float freq_factor = ff ? ff[i0 / 2] : 1.0f;                              /* :65,99 */
                const float theta = freq_scale * (theta_base / freq_factor);                   /* rope_yarn :20-22 */
                const double c = cos((double)theta) * (double)attn_factor, sn = sin((double)theta) * (double)attn_factor;
                const uint32_t a = mode == 2u ? i0 / 2 : i0, b = mode == 2u ? i0 / 2 + n_dims / 2 : i0 + 1;
                const double x0 = y[a], x1 = y[b];
                dst[a] = (float)(x0 * c - x1 * sn);                                            /* :73-74, :107-108 */
                dst[b] = (float)(x0 * sn + x1 * c);
            }
            free(y);
        }
}

int vfo_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * Gated attention output (vk_shaders/sigmoid_mul.comp:40-53):
 *   data[i] *= sigmoid(gate[(i / chunk) * stride + gate_offset + i % chunk]),  sigmoid(g) = 1 / (1 + exp(-g)).
 * The sigmoid is evaluated in f64 and rounded to f32 once; the product is an f32 multiply as in the shader.
 * ---------------------------------------------------------------------------------------- */
void vfo_sigmoid_mul(const float* gate, float* data, uint64_t ne, uint32_t chunk, uint32_t stride, uint32_t gate_offset) {
    for (uint64_t i = 0; i < ne; ++i) {
        const uint64_t token = i / chunk, within = i - token * chunk;
        const double g = (double)gate[token * stride + gate_offset + within];
        const float sg = (float)(1.0 / (1.0 + exp(-g)));
        data[i] = data[i] * sg;
    }
}
