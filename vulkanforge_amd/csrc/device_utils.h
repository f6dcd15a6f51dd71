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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kMasked = -1e30f;  // the reference's "minus infinity" (flash_attn_split.comp:102)

enum : uint32_t { kF32 = 0, kF16 = 1, kF8 = 2 };

__host__ __device__ constexpr uint32_t elem_size(uint32_t dtype) { return dtype == kF32 ? 4u : dtype == kF16 ? 2u : 1u; }

// ---- E4M3FN encode -------------------------------------------------------------------------
// Saturating round-to-nearest-even E4M3FN with the reference's corner cases
// (src/backend/vulkan/fp8_ext.rs:126-186): NaN -> 0x7F (sign dropped), |x| >= 448 and +-Inf ->
// sign|0x7E.  v_cvt_pk_fp8_f32 rounds to nearest even including subnormals; the clamp supplies
// the saturation (it also maps +-Inf to +-448).  The instruction encodes a NaN input as 0xFF, so
// NaN lanes are converted as zero and their byte is then set to the reference's 0x7F.
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    const float in[4] = {a, b, c, d};
    float s[4];
    uint32_t nan_bytes = 0u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const bool is_nan = in[j] != in[j];
        s[j] = is_nan ? 0.0f : __builtin_amdgcn_fmed3f(in[j], -448.0f, 448.0f);
        nan_bytes |= is_nan ? (0x7Fu << (8 * j)) : 0u;
    }
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(s[0], s[1], 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(s[2], s[3], w, true);
    return (uint32_t)w | nan_bytes;
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

// Packed f16 remainders of two f32 values against their packed f16 roundings `h`: f16(p - f32(h)) per element.
// One mixed-precision FMA per element (the f16 source is widened inside the instruction), bit-identical to
// converting back, subtracting and converting again.
__device__ __forceinline__ uint32_t pack_f16_remainder(float p0, float p1, uint32_t h) {
    uint32_t r;
    asm("v_fma_mixlo_f16 %0, %1, 1.0, -%3 op_sel:[0,0,0] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %0, %2, 1.0, -%3 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
        : "=&v"(r) : "v"(p0), "v"(p1), "v"(h));
    return r;
}

// Logit soft-cap in log2 units: cap * tanh(y / cap) with tanh(x) = 1 - 2 / (exp(2 x) + 1) on the hardware exponential and
// reciprocal: no branch and no division (the library tanhf branches per element); exact limits for large |x| (exp2 -> inf or
// 0), absolute error of tanh about 1e-7, i.e. below 1e-5 of a score at cap 50.
__device__ __forceinline__ float softcap_l2(float y, float cap_l2, float inv_cap_l2) {
    const float t = __builtin_amdgcn_exp2f(y * inv_cap_l2 * 2.88539008177793f);      // exp(2 x), 2 * log2(e)
    return __builtin_fmaf(-2.0f * cap_l2, __builtin_amdgcn_rcpf(t + 1.0f), cap_l2);
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

// ---- wavefront (64-lane) data movement -----------------------------------------------------
// DPP controls (gfx9 encoding): quad permutes for lane^1 / lane^2, mirrors for the 8- and 16-lane
// steps, row broadcasts for the cross-row steps of a full-wave reduction.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_keep(float old, float x) {   // lanes of rows outside ROWMASK receive `old`
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, x),
                                                                 CTRL, ROWMASK, 0xf, false));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140, kDppRor8 = 0x128;
constexpr int kDppBcast15 = 0x142, kDppBcast31 = 0x143;

// In-place lane swaps of gfx950.  The instructions are issued directly: the two-result compiler
// builtins were observed to return the first result twice.  Both operands are read and written.
__device__ __forceinline__ void swap32(float& a, float& b) {   // a.lanes[32..63] <-> b.lanes[0..31]
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap16(float& a, float& b) {   // odd 16-lane rows of a <-> even rows of b
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float xor16_sum(float x) { float y = x; swap16(x, y); return x + y; }
__device__ __forceinline__ float xor32_sum(float x) { float y = x; swap32(x, y); return x + y; }

// Sum over each aligned group of W lanes; every lane of the group gets the result.
template <int W>
__device__ __forceinline__ float group_sum(float x) {
    if (W >= 2) x += dpp_f<kDppXor1>(x);
    if (W >= 4) x += dpp_f<kDppXor2>(x);
    if (W >= 8) x += dpp_f<kDppHalfMirror>(x);
    if (W >= 16) x += dpp_f<kDppMirror>(x);
    if (W >= 32) x = xor16_sum(x);
    if (W >= 64) x = xor32_sum(x);
    return x;
}
// Wavefront-wide max / sum as a uniform (scalar register) value: in-row butterflies, then the two
// row broadcasts leave the total in lane 63.
__device__ __forceinline__ float wave_max_uniform(float x) {
    x = fmaxf(x, dpp_f<kDppXor1>(x));
    x = fmaxf(x, dpp_f<kDppXor2>(x));
    x = fmaxf(x, dpp_f<kDppHalfMirror>(x));
    x = fmaxf(x, dpp_f<kDppMirror>(x));
    x = fmaxf(x, dpp_keep<kDppBcast15, 0xa>(x, x));
    x = fmaxf(x, dpp_keep<kDppBcast31, 0xc>(x, x));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}
__device__ __forceinline__ float wave_sum_uniform(float x) {
    x += dpp_f<kDppXor1>(x);
    x += dpp_f<kDppXor2>(x);
    x += dpp_f<kDppHalfMirror>(x);
    x += dpp_f<kDppMirror>(x);
    x += dpp_keep<kDppBcast15, 0xa>(0.f, x);
    x += dpp_keep<kDppBcast31, 0xc>(0.f, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}
// Transposing LDS read (ds_read_b64_tr_b16): within each group of 16 lanes, lane i receives element
// i%4 of the four 4-element (8-byte) chunks addressed by lanes i/4, i/4+4, i/4+8 and i/4+12 of the group.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half4_t lds_read_tr16(const _Float16* p) {
    const short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)p);
    return __builtin_bit_cast(half4_t, r);
}

// Shuffle-based all-lane variants for the generic kernels (vector result in every lane).
__device__ __forceinline__ float wave_sum_all(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max_all(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// vk_shaders/sigmoid_mul.comp:50-52: x * 1 / (1 + exp(-g)), f32 throughout
__device__ __forceinline__ float sigmoid_gate(float x, float g) { return x * (1.0f / (1.0f + expf(-g))); }
// vk_shaders/sigmoid_mul.comp:44-48
template <typename G>
__device__ __forceinline__ uint64_t gate_index(const G& g, uint64_t i) {
    const uint64_t token = i / g.chunk;
    return token * g.stride + g.gate_offset + (i - token * g.chunk);
}

}  // namespace vfkv
