// KV append and expansion kernels for gfx950.
//
//   kv_store_fp8   f32 -> E4M3FN bytes      (vk_shaders/kv_store_fp8.comp:42-67)
//   kv_copy_fp16   f32 -> f16               (vk_shaders/kv_copy_fp16.comp:39-51)
//   kv_copy_f32    f32 -> f32               (the vkCmdCopyBuffer branch, executor/attention.rs:575-581)
//   kv_fp8_to_f16  E4M3FN bytes -> f16      (vk_shaders/kv_fp8_to_f16.comp:28-33)
//
// All are pure streaming kernels (HBM bound).  One thread converts one 32-bit destination word
// for the two append kernels -- 16-byte coalesced loads, 4-byte coalesced stores -- so the only
// alignment the destination needs is the 4 bytes the reference also demands.  K and V of one
// append go out in a single launch (blockIdx.y selects the tensor).
#include "device_utils.h"
#include "kernels.h"

namespace vfkv {

struct AppendArgs {
    const float* src[2];
    uint8_t* dst[2];   // already offset by dst_byte_offset
    uint32_t n;        // elements per tensor
};

// mode: 0 = fp8, 1 = f16, 2 = f32 copy
template <int MODE>
__global__ __launch_bounds__(256) void kv_append_kernel(AppendArgs a) {
    const float* __restrict__ src = a.src[blockIdx.y];
    uint8_t* __restrict__ dst = a.dst[blockIdx.y];
    constexpr uint32_t EPW = MODE == 0 ? 4u : MODE == 1 ? 2u : 1u;  // elements per 32-bit word
    const uint32_t n = a.n;
    const uint32_t n_words = (n + EPW - 1u) / EPW;
    const bool src16 = (((uintptr_t)src) & 15u) == 0u;
    for (uint32_t w = blockIdx.x * blockDim.x + threadIdx.x; w < n_words; w += gridDim.x * blockDim.x) {
        const uint32_t e0 = w * EPW;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (MODE == 0 && src16 && e0 + 4u <= n) {
            const float4 f = *reinterpret_cast<const float4*>(src + e0);
            v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
        } else {
#pragma unroll
            for (uint32_t j = 0; j < EPW; ++j)
                if (e0 + j < n) v[j] = src[e0 + j];  // ragged tail is zero-padded to the word
        }
        uint32_t out;
        if (MODE == 0) {
            out = pack4_e4m3(v[0], v[1], v[2], v[3]);
        } else if (MODE == 1) {
            out = f32_to_h16_bits(v[0]) | (f32_to_h16_bits(v[1]) << 16);
        } else {
            out = __builtin_bit_cast(uint32_t, v[0]);
        }
        reinterpret_cast<uint32_t*>(dst)[w] = out;
    }
}

template <int MODE>
static hipError_t launch_append(const float* k_src, const float* v_src, void* k_dst, void* v_dst, uint32_t n,
                                int n_tensors, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    AppendArgs a;
    a.src[0] = k_src; a.src[1] = v_src;
    a.dst[0] = (uint8_t*)k_dst; a.dst[1] = (uint8_t*)v_dst;
    a.n = n;
    constexpr uint32_t EPW = MODE == 0 ? 4u : MODE == 1 ? 2u : 1u;
    const uint32_t n_words = (n + EPW - 1u) / EPW;
    uint32_t blocks = (n_words + 255u) / 256u;
    if (blocks > 4096u) blocks = 4096u;
    hipLaunchKernelGGL(kv_append_kernel<MODE>, dim3(blocks, n_tensors), dim3(256), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_kv_append(uint32_t dtype, const float* k_src, const float* v_src, void* k_dst, void* v_dst,
                            uint32_t n, int n_tensors, hipStream_t stream) {
    if (dtype == kF8) return launch_append<0>(k_src, v_src, k_dst, v_dst, n, n_tensors, stream);
    if (dtype == kF16) return launch_append<1>(k_src, v_src, k_dst, v_dst, n, n_tensors, stream);
    return launch_append<2>(k_src, v_src, k_dst, v_dst, n, n_tensors, stream);
}

// ---- E4M3 -> f16 expansion -------------------------------------------------------------------
// 8 codes per piece: one 8-byte load, four packed conversions, one 16-byte store, so that both the loads and the stores of
// a wavefront are contiguous (whole 128-byte lines per store instruction).  The output is written once and not read back
// by this kernel: the stores carry the non-temporal hint.  A thread takes four pieces per round and requests all four
// before it converts the first.  (One 16-byte load and two 16-byte stores per thread, every line written by two
// instructions: 22.9 us for 33.5 M codes; this form: 15.2 us = 6.6 TB/s of read + write traffic.)
constexpr int kExpandPieces = 4;
__global__ __launch_bounds__(256) void kv_fp8_to_f16_kernel(const uint8_t* __restrict__ src,
                                                            uint16_t* __restrict__ dst, uint64_t n, int vec_ok) {
    const uint64_t n_vec = vec_ok ? n / 8u : 0u;
    const uint64_t threads = (uint64_t)gridDim.x * blockDim.x;
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    // round r covers pieces [r * threads * 4, (r + 1) * threads * 4); inside it a workgroup's pieces are contiguous
    for (uint64_t base = (uint64_t)blockIdx.x * blockDim.x * kExpandPieces; base < n_vec; base += threads * kExpandPieces) {
        u32x2 w[kExpandPieces];
#pragma unroll
        for (int u = 0; u < kExpandPieces; ++u) {
            const uint64_t i = base + (uint64_t)u * blockDim.x + threadIdx.x;
            w[u] = i < n_vec ? reinterpret_cast<const u32x2*>(src)[i] : u32x2{0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < kExpandPieces; ++u) {
            const uint64_t i = base + (uint64_t)u * blockDim.x + threadIdx.x;
            if (i >= n_vec) continue;
            half2_t a0, a1, b0, b1;
            e4m3x4_to_h2(w[u][0], a0, a1);
            e4m3x4_to_h2(w[u][1], b0, b1);
            const u32x4 out = u32x4{__builtin_bit_cast(uint32_t, a0), __builtin_bit_cast(uint32_t, a1),
                                    __builtin_bit_cast(uint32_t, b0), __builtin_bit_cast(uint32_t, b1)};
            __builtin_nontemporal_store(out, reinterpret_cast<u32x4*>(dst) + i);
        }
    }
    for (uint64_t i = n_vec * 8u + tid; i < n; i += threads)
        dst[i] = (uint16_t)f32_to_h16_bits(__builtin_amdgcn_cvt_f32_fp8((int)src[i], 0));
}

hipError_t launch_fp8_to_f16(const void* src, void* dst, uint64_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    const int vec_ok = (((uintptr_t)src) & 7u) == 0u && (((uintptr_t)dst) & 15u) == 0u;
    uint64_t work = vec_ok ? (n / 8u + kExpandPieces - 1u) / kExpandPieces : n;
    uint64_t blocks = (work + 255u) / 256u;
    if (blocks == 0u) blocks = 1u;
    if (blocks > 65536u) blocks = 65536u;
    hipLaunchKernelGGL(kv_fp8_to_f16_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream,
                       (const uint8_t*)src, (uint16_t*)dst, n, vec_ok);
    return hipGetLastError();
}

// KvCache::zero_fill / zero_layer (kv_cache.rs:357-407) as a kernel, so that a caller may capture it into a HIP graph (memset
// nodes are avoided on purpose): 16-byte stores over the aligned body, single bytes at the two ends.
__global__ __launch_bounds__(256) void zero_bytes_kernel(uint8_t* __restrict__ p, uint64_t head, uint64_t n_vec, uint64_t n) {
    const uint64_t tid = (uint64_t)blockIdx.x * 256u + threadIdx.x, stride = (uint64_t)gridDim.x * 256u;
    uint4* body = reinterpret_cast<uint4*>(p + head);
    for (uint64_t i = tid; i < n_vec; i += stride) body[i] = make_uint4(0u, 0u, 0u, 0u);
    const uint64_t tail0 = head + n_vec * 16u;
    for (uint64_t i = tid; i < head; i += stride) p[i] = 0;
    for (uint64_t i = tail0 + tid; i < n; i += stride) p[i] = 0;
}

hipError_t launch_zero_bytes(void* dst, uint64_t n, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    if (dst == nullptr) return hipErrorInvalidValue;
    uint64_t head = (16u - (((uintptr_t)dst) & 15u)) & 15u;
    if (head > n) head = n;
    const uint64_t n_vec = (n - head) / 16u;
    uint64_t blocks = (n_vec + 255u) / 256u;
    if (blocks == 0u) blocks = 1u;
    if (blocks > 4096u) blocks = 4096u;
    hipLaunchKernelGGL(zero_bytes_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, (uint8_t*)dst, head, n_vec, n);
    return hipGetLastError();
}

}  // namespace vfkv
