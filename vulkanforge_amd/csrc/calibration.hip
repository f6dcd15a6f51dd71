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
//
// Two more, for the prefill kernels' roofline entry (no memory traffic at all): what the instructions of their inner loop
// cost a SIMD to issue, and how far matrix and vector instructions overlap:
//
//   calib_issue          one kind of vector instruction, 64 per loop pass on eight independent registers, in workgroups of one
//                        or two wavefronts per SIMD; wavefront 0 reports its shader-clock and 100 MHz wall-clock ticks
//   calib_overlap        per loop pass 48 v_mfma_f32_16x16x32_f16 and NV v_fma_f32 per wavefront, two wavefronts per SIMD:
//                        in two phases, the same with the two wavefronts of a SIMD held in opposite phases by workgroup
//                        barriers, or in one basic block left to the compiler's scheduler
//   calib_overlap_kind   the two-phase pass with 100 vector instructions of one of calib_issue's kinds
// (calibration_prefill.hip adds the FP8 prefill kernel compiled with wall-clock stamps.)
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

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// OP: 0 v_fma_f32, 1 v_exp_f32, 2 v_cvt_scalef32_pk_f16_fp8, 3 v_max_f32, 4 v_fma_mixlo_f16, 5 v_xor_b32
template <int OP>
__global__ __launch_bounds__(512) void calib_issue(uint32_t* __restrict__ sink, uint64_t* __restrict__ clk, int iters, float seed) {
    float v[8];
    uint32_t u[8];
    for (int i = 0; i < 8; ++i) { v[i] = seed + i + threadIdx.x; u[i] = 0x38404448u + i + threadIdx.x; }
    const float c0 = seed * 1.0001f, c1 = seed * 0.37f;
    const uint64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int n = 0; n < 64; ++n) {
            const int i = n % 8, j = (n + 1) % 8;
            if (OP == 0) v[i] = __builtin_fmaf(v[i], c0, c1);
            if (OP == 1) v[i] = __builtin_amdgcn_exp2f(v[i]);
            if (OP == 2) asm volatile("v_cvt_scalef32_pk_f16_fp8 %0, %1, 1.0" : "=v"(u[i]) : "v"(u[j]));
            if (OP == 3) v[i] = fmaxf(v[i], v[(n + 3) % 8]);
            if (OP == 4) asm volatile("v_fma_mixlo_f16 %0, %1, 1.0, -%2 op_sel:[0,0,0] op_sel_hi:[0,0,1]" : "=v"(u[i]) : "v"(v[i]), "v"(u[j]));
            if (OP == 5) u[i] ^= u[j];
        }
    }
    const uint64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    float r = 0.f;
    for (int i = 0; i < 8; ++i) r += v[i] + (float)u[i];
    if (r == 1234.5f) sink[threadIdx.x] = (uint32_t)r;
    if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = r1 - r0; }
}

// MODE 0: 48 matrix instructions, then NV vector instructions; 1: the same, the second wavefront of every SIMD (threads
// 256..511) starting with the vector phase and a workgroup barrier after every phase; 2: both kinds in one basic block
template <int NV, int MODE>
__global__ __launch_bounds__(512) void calib_overlap(uint32_t* __restrict__ sink, uint64_t* __restrict__ clk, int iters, float seed) {
    constexpr int NM = 48;
    half8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(seed + threadIdx.x * 0.001f + i); b[i] = (_Float16)(seed * 0.5f + i); }
    float4_t acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = seed + i + threadIdx.x;
    const float c0 = seed * 1.0001f, c1 = seed * 0.37f;
    const bool second = (threadIdx.x >> 8) & 1;
    auto matrix = [&]() {
#pragma unroll
        for (int m = 0; m < NM; ++m) acc[m % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[m % 8], 0, 0, 0);
    };
    auto vector = [&]() {
#pragma unroll
        for (int n = 0; n < NV; ++n) v[n % 8] = __builtin_fmaf(v[n % 8], c0, c1);
    };
    const uint64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        if (MODE == 0) {
            matrix();
            __builtin_amdgcn_sched_barrier(0);
            vector();
            __builtin_amdgcn_sched_barrier(0);
        } else if (MODE == 1) {
            if (second) vector(); else matrix();
            __syncthreads();
            if (second) matrix(); else vector();
            __syncthreads();
        } else {
            matrix();
            vector();
        }
    }
    const uint64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    float r = 0.f;
    for (int i = 0; i < 8; ++i) r += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + v[i];
    if (r == 1234.5f) sink[threadIdx.x] = (uint32_t)r;
    if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = r1 - r0; }
}

// Per pass NM v_mfma_f32_16x16x32_f16 (0 or 48), then 100 vector instructions of kind OP (the kinds of calib_issue) per
// wavefront, two wavefronts per SIMD, free running: how much of each kind of vector work hides behind the other wavefront's
// matrix instructions.
template <int OP, int NM>
__global__ __launch_bounds__(512) void calib_overlap_kind(uint32_t* __restrict__ sink, uint64_t* __restrict__ clk, int iters, float seed) {
    half8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(seed + threadIdx.x * 0.001f + i); b[i] = (_Float16)(seed * 0.5f + i); }
    float4_t acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float v[8];
    uint32_t u[8];
    for (int i = 0; i < 8; ++i) { v[i] = seed + i + threadIdx.x; u[i] = 0x38404448u + i + threadIdx.x; }
    const float c0 = seed * 1.0001f, c1 = seed * 0.37f;
    const uint64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < NM; ++m) acc[m % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[m % 8], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < 100; ++n) {
            const int i = n % 8, j = (n + 3) % 8;
            if (OP == 0) v[i] = __builtin_fmaf(v[i], c0, c1);
            if (OP == 1) v[i] = __builtin_amdgcn_exp2f(v[i]);
            if (OP == 2) asm volatile("v_cvt_scalef32_pk_f16_fp8 %0, %1, 1.0" : "=v"(u[i]) : "v"(u[j]));
            if (OP == 3) v[i] = fmaxf(v[i], v[j]);
            if (OP == 4) asm volatile("v_fma_mixlo_f16 %0, %1, 1.0, -%2 op_sel:[0,0,0] op_sel_hi:[0,0,1]" : "=v"(u[i]) : "v"(v[i]), "v"(u[j]));
            if (OP == 5) u[i] ^= u[j];
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    const uint64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    float r = 0.f;
    for (int i = 0; i < 8; ++i) r += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + v[i] + (float)u[i];
    if (r == 1234.5f) sink[threadIdx.x] = (uint32_t)r;
    if (blockIdx.x == 0 && threadIdx.x == 0) { clk[0] = t1 - t0; clk[1] = r1 - r0; }
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

// 256 workgroups of `waves_per_simd` x 256 threads issue `iters` x 64 instructions of kind `op` (0 v_fma_f32, 1 v_exp_f32,
// 2 v_cvt_scalef32_pk_f16_fp8, 3 v_max_f32, 4 v_fma_mixlo_f16, 5 v_xor_b32).  clk (device, two uint64): shader-clock and 100 MHz
// ticks of wavefront 0 of workgroup 0.  0 on success.
int vfkv_calib_issue(int op, int waves_per_simd, int iters, void* sink, void* clk, void* stream) {
    if (!sink || !clk || iters <= 0 || (waves_per_simd != 1 && waves_per_simd != 2)) return -1;
    const dim3 grid(256), block(256 * waves_per_simd);
#define VFKV_CALIB_OP(N) case N: hipLaunchKernelGGL((calib_issue<N>), grid, block, 0, (hipStream_t)stream, (uint32_t*)sink, (uint64_t*)clk, iters, 1.0f); break;
    switch (op) {
        VFKV_CALIB_OP(0) VFKV_CALIB_OP(1) VFKV_CALIB_OP(2) VFKV_CALIB_OP(3) VFKV_CALIB_OP(4) VFKV_CALIB_OP(5)
        default: return -1;
    }
#undef VFKV_CALIB_OP
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

// 256 workgroups of two wavefronts per SIMD run `iters` passes of 48 matrix instructions + `n_vector` (0, 100, 200 or 400)
// v_fma_f32 per wavefront; mode 0: two phases, 1: the wavefronts of a SIMD in opposite phases behind barriers, 2: one basic
// block.  clk as above.  0 on success.
int vfkv_calib_overlap(int n_vector, int mode, int iters, void* sink, void* clk, void* stream) {
    if (!sink || !clk || iters <= 0 || mode < 0 || mode > 2) return -1;
    const dim3 grid(256), block(512);
#define VFKV_CALIB_OV(NV, M) if (n_vector == NV && mode == M) { hipLaunchKernelGGL((calib_overlap<NV, M>), grid, block, 0, (hipStream_t)stream, (uint32_t*)sink, (uint64_t*)clk, iters, 1.0f); return hipGetLastError() == hipSuccess ? 0 : -5; }
    VFKV_CALIB_OV(0, 0) VFKV_CALIB_OV(100, 0) VFKV_CALIB_OV(200, 0) VFKV_CALIB_OV(400, 0)
    VFKV_CALIB_OV(200, 1) VFKV_CALIB_OV(200, 2)
#undef VFKV_CALIB_OV
    return -1;
}

// 256 workgroups of two wavefronts per SIMD run `iters` passes of (48 matrix instructions if with_matrix) + 100 vector
// instructions of kind `op` (as in vfkv_calib_issue) per wavefront.  clk as above.  0 on success.
int vfkv_calib_overlap_kind(int op, int with_matrix, int iters, void* sink, void* clk, void* stream) {
    if (!sink || !clk || iters <= 0) return -1;
    const dim3 grid(256), block(512);
#define VFKV_CALIB_OK(N)                                                                                                     \
    case N:                                                                                                                  \
        if (with_matrix) hipLaunchKernelGGL((calib_overlap_kind<N, 48>), grid, block, 0, (hipStream_t)stream, (uint32_t*)sink, (uint64_t*)clk, iters, 1.0f); \
        else hipLaunchKernelGGL((calib_overlap_kind<N, 0>), grid, block, 0, (hipStream_t)stream, (uint32_t*)sink, (uint64_t*)clk, iters, 1.0f);  \
        break;
    switch (op) {
        VFKV_CALIB_OK(0) VFKV_CALIB_OK(1) VFKV_CALIB_OK(2) VFKV_CALIB_OK(3) VFKV_CALIB_OK(4) VFKV_CALIB_OK(5)
        default: return -1;
    }
#undef VFKV_CALIB_OK
    return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // extern "C"
#pragma GCC visibility pop
