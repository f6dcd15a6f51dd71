// Device-side helpers shared by the gfx950 kernels: OCP E4M3 <-> f32/f16 conversions on the
// native conversion instructions, 16-byte loads, and wavefront (64-lane) reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vfkv {

typedef float float2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;
constexpr float kMasked = -1e30f;  // the reference's "minus infinity" (flash_attn_split.comp:102)

enum : uint32_t { kF32 = 0, kF16 = 1, kF8 = 2 };

__host__ __device__ constexpr uint32_t elem_size(uint32_t dtype) { return dtype == kF32 ? 4u : dtype == kF16 ? 2u : 1u; }

// ---- E4M3FN encode -------------------------------------------------------------------------
// Saturating round-to-nearest-even E4M3FN with the reference's corner cases
// (src/backend/vulkan/fp8_ext.rs:126-186): NaN -> 0x7F (sign dropped), |x| >= 448 and +-Inf ->
// sign|0x7E.  v_cvt_pk_fp8_f32 rounds to nearest even including subnormals; the clamp supplies
// the saturation and the select canonicalises NaN before the conversion.
__device__ __forceinline__ float e4m3_presat(float x) {
    float c = __builtin_amdgcn_fmed3f(x, -448.0f, 448.0f);
    return (x != x) ? __builtin_bit_cast(float, 0x7FC00000u) : c;
}
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_presat(a), e4m3_presat(b), 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(e4m3_presat(c), e4m3_presat(d), w, true);
    return (uint32_t)w;
}

// ---- E4M3FN decode -------------------------------------------------------------------------
template <int BYTE>
__device__ __forceinline__ float e4m3_byte_to_f32(uint32_t w) {
    return __builtin_amdgcn_cvt_f32_fp8((int)w, BYTE);
}
__device__ __forceinline__ float e4m3_to_f32_dyn(uint32_t w, uint32_t byte) {
    return __builtin_amdgcn_cvt_f32_fp8((int)(w >> (byte * 8u)), 0);
}
// word of 4 codes -> 4 floats
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float* out) {
    float2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    float2_t hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    out[0] = lo.x; out[1] = lo.y; out[2] = hi.x; out[3] = hi.y;
}
// word of 4 codes -> 2 packed f16 pairs (exact: every E4M3 value is an f16 value)
__device__ __forceinline__ void e4m3x4_to_h2(uint32_t w, half2_t& lo, half2_t& hi) {
    lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w, 1.0f, false);
    hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w, 1.0f, true);
}

__device__ __forceinline__ float h16_bits_to_f32(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
__device__ __forceinline__ uint32_t f32_to_h16_bits(float x) {  // round to nearest even
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
}

// Element `idx` of a K/V slab in the cache dtype (flash_attn_split.comp:29-58 load_k / load_v).
__device__ __forceinline__ float load_kv_elem(const void* base, uint32_t dtype, uint64_t idx) {
    if (dtype == kF32) return ((const float*)base)[idx];
    if (dtype == kF16) return h16_bits_to_f32(((const uint16_t*)base)[idx]);
    return __builtin_amdgcn_cvt_f32_fp8((int)((const uint8_t*)base)[idx], 0);
}

// ---- wavefront reductions ------------------------------------------------------------------
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {  // all lanes of each aligned WIDTH-group get the sum
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

__device__ __forceinline__ float softcap_apply(float s, float cap) {
    // cap * tanh(s / cap); tanh(x) = 1 - 2 / (exp(2x) + 1) stays finite for large |x|
    float x = s / cap;
    float e = __expf(2.0f * x);
    float t = 1.0f - 2.0f / (e + 1.0f);
    return cap * t;
}

}  // namespace vfkv
