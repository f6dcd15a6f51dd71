// Reference points for the decode worker's roofline entry, built into libvfkv_calib.so (loaded by the benchmark only; the
// product library does not contain or need them).  All three read the K and V slabs of one layer of a KV cache in the
// layout the attention kernels read (kv_cache.rs:3-12: [pos][kv_head][d]) and compute nothing:
//
//   calib_stream_read    every wavefront reads contiguous 1 KiB pieces (whole position rows), eight 16-byte loads per lane
//                        in flight: what the memory system delivers for the plainest read of the same bytes
//   calib_pattern_read   the walk of split_mfma_kernel at head_dim 128 over FP8 rows: grid (KV head, tile), four
//                        wavefronts, runs of 32 rows dealt round-robin over all wavefronts of a KV head, per run the
//                        worker's K requests (lane (n16, kg): row n16 of each 16-row tile, bytes kg*32 + x*16) and V requests
//                        (lane: row lane / 8 (+ 8c), bytes (lane % 8) * 16), one run in flight ahead of the one consumed
//   calib_empty          the same grid with no work: the cost of a launch
//
// The loaded values are folded into an XOR that is stored only if it equals a constant, so the compiler keeps the loads.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kOOB = 0x80000000u;

__device__ __forceinline__ uint32_t fold(uint32_t acc, const u32x4& x) { return acc ^ x.x ^ x.y ^ x.z ^ x.w; }

template <int NL>
__global__ __launch_bounds__(256) void calib_stream_read(const u32x4* __restrict__ k, const u32x4* __restrict__ v,
                                                         uint32_t* __restrict__ sink, uint32_t n16) {
    // n16 = 16-byte pieces per buffer; workgroup b reads pieces [b * 256 * NL, (b + 1) * 256 * NL) of K, then of V
    const uint32_t per_wg = 256u * NL;
    const uint32_t wgs_per_buf = (n16 + per_wg - 1u) / per_wg;
    const u32x4* src = blockIdx.x < wgs_per_buf ? k : v;
    const uint32_t b = blockIdx.x < wgs_per_buf ? blockIdx.x : blockIdx.x - wgs_per_buf;
    u32x4 r[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const uint32_t idx = b * per_wg + i * 256u + threadIdx.x;
        r[i] = idx < n16 ? src[idx] : u32x4{0u, 0u, 0u, 0u};
    }
    uint32_t acc = 0u;
#pragma unroll
    for (int i = 0; i < NL; ++i) acc = fold(acc, r[i]);
    if (acc == 0x12345678u) sink[threadIdx.x] = acc;
}

__global__ __launch_bounds__(256) void calib_pattern_read(const uint8_t* __restrict__ k, const uint8_t* __restrict__ v,
                                                          uint32_t* __restrict__ sink, uint32_t seq_len, uint32_t n_kv_heads,
                                                          uint32_t n_tiles) {
    constexpr int D = 128, RUN = 32, NP = 4;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n16 = lane & 15, kg = lane >> 4;
    const uint32_t kvh = blockIdx.x, jl = blockIdx.y;
    const uint32_t row_stride = n_kv_heads * D;
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)k, 0, seq_len * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)v, 0, seq_len * row_stride, 0x00020000);
    const uint32_t head_b = kvh * D;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * 32;
    const uint32_t lane_voff = (lane / 8) * row_stride + head_b + (lane % 8) * 16;
    const uint32_t n_runs = (seq_len + RUN - 1) / RUN;
    const uint32_t rs = NP * n_tiles, r0 = jl * NP + w;
    auto run_off = [&](uint32_t r) -> uint32_t { return r < n_runs ? r * RUN * row_stride : kOOB; };
    u32x4 kraw[2][2], vraw[4];
    auto issue = [&](uint32_t off) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int x = 0; x < 2; ++x)
                kraw[t][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * 16, off + (uint32_t)(t * 16) * row_stride, 0);
#pragma unroll
        for (int c = 0; c < 4; ++c)
            vraw[c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, off + (uint32_t)(c * 8) * row_stride, 0);
    };
    uint32_t acc = 0u;
    issue(run_off(r0));
    for (uint32_t r = r0; r < n_runs; r += rs) {
        u32x4 ck[2][2], cv[4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int x = 0; x < 2; ++x) ck[t][x] = kraw[t][x];
#pragma unroll
        for (int c = 0; c < 4; ++c) cv[c] = vraw[c];
        issue(run_off(r + rs));
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int x = 0; x < 2; ++x) acc = fold(acc, ck[t][x]);
#pragma unroll
        for (int c = 0; c < 4; ++c) acc = fold(acc, cv[c]);
    }
    if (acc == 0x12345678u) sink[threadIdx.x] = acc;
}

__global__ __launch_bounds__(256) void calib_empty(uint32_t* __restrict__ sink, uint32_t never) {
    if (never == 0x12345678u) sink[threadIdx.x] = never;
}

}  // namespace

#pragma GCC visibility push(default)    // the library is built with hidden visibility: only these entry points are exported
extern "C" {

// Reads `bytes` of K and `bytes` of V (16-byte aligned, multiples of 16) with contiguous loads.  0 on success.
int vfkv_calib_stream_read(const void* k, const void* v, uint64_t bytes, void* sink, void* stream) {
    if (!k || !v || !sink || bytes == 0 || bytes % 16u != 0u || bytes >= (1ull << 35)) return -1;
    constexpr int NL = 8;
    const uint32_t n16 = (uint32_t)(bytes / 16u);
    const uint32_t per_wg = 256u * NL;
    const uint32_t wgs = (n16 + per_wg - 1u) / per_wg;
    hipLaunchKernelGGL((calib_stream_read<NL>), dim3(2u * wgs), dim3(256), 0, (hipStream_t)stream, (const u32x4*)k,
                       (const u32x4*)v, (uint32_t*)sink, n16);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

// Reads rows [0, seq_len) of an FP8 layer slab with head_dim 128 in the decode worker's pattern, `n_tiles` workgroups per
// KV head.  The slab must be smaller than 2 GiB.  0 on success.
int vfkv_calib_pattern_read(const void* k, const void* v, uint32_t seq_len, uint32_t n_kv_heads, uint32_t n_tiles,
                            void* sink, void* stream) {
    if (!k || !v || !sink || seq_len == 0 || n_kv_heads == 0 || n_tiles == 0) return -1;
    if ((uint64_t)seq_len * n_kv_heads * 128u >= 0x7FFF0000ull) return -1;
    hipLaunchKernelGGL(calib_pattern_read, dim3(n_kv_heads, n_tiles), dim3(256), 0, (hipStream_t)stream, (const uint8_t*)k,
                       (const uint8_t*)v, (uint32_t*)sink, seq_len, n_kv_heads, n_tiles);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

int vfkv_calib_empty(uint32_t n_kv_heads, uint32_t n_tiles, void* sink, void* stream) {
    if (!sink || n_kv_heads == 0 || n_tiles == 0) return -1;
    hipLaunchKernelGGL(calib_empty, dim3(n_kv_heads, n_tiles), dim3(256), 0, (hipStream_t)stream, (uint32_t*)sink, 0u);
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // extern "C"
#pragma GCC visibility pop
