// Chunked-prefill causal attention over the cache (flash_attn_batch.comp:105-208) for gfx950.
//
// batch_generic_kernel: one wavefront per (query, head); covers every dtype and head_dim <= 512.
#include "device_utils.h"
#include "kernels.h"

namespace vfkv {

struct BatchArgs {
    const float* q;
    const uint8_t* k;
    const uint8_t* v;
    float* o;
    uint32_t n_heads, n_kv_heads, head_dim;
    uint32_t m, n_kv, q_start, kv_start;
    float scale, softcap;
    uint32_t dtype;
};

__global__ __launch_bounds__(kWave) void batch_generic_kernel(BatchArgs a) {
    __shared__ float p_lds[kWave];
    const int lane = threadIdx.x;
    const uint32_t h = blockIdx.x;
    const uint32_t qi = blockIdx.y;
    const uint32_t D = a.head_dim;
    const uint32_t kvh = h / (a.n_heads / a.n_kv_heads);
    uint32_t causal_len = a.q_start + qi + 1u;
    if (causal_len > a.n_kv) causal_len = a.n_kv;
    const uint32_t lo = a.kv_start;
    const uint64_t pos_stride = (uint64_t)a.n_kv_heads * D;
    const uint64_t head_off = (uint64_t)kvh * D;
    const float* q = a.q + ((size_t)qi * a.n_heads + h) * D;

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    float m_run = kMasked, l_run = 0.f;
    for (uint32_t base = (lo / kWave) * kWave; base < causal_len; base += kWave) {
        const uint32_t t = base + lane;
        const bool valid = t < causal_len && t >= lo;
        float sc = kMasked;
        if (valid) {
            const uint64_t ko = (uint64_t)t * pos_stride + head_off;
            float s = 0.f;
            for (uint32_t d = 0; d < D; ++d) s = fmaf(q[d], load_kv_elem(a.k, a.dtype, ko + d), s);
            s *= a.scale;
            if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
            sc = s;
        }
        const float bm = wave_max_all(sc);
        const float m_new = fmaxf(m_run, bm);
        const float alpha = __expf(m_run - m_new);
        const float p = valid ? __expf(sc - m_new) : 0.f;
        l_run = l_run * alpha + wave_sum_all(p);
        m_run = m_new;
        __syncthreads();
        p_lds[lane] = p;
        __syncthreads();
        const uint32_t rows = causal_len - base < (uint32_t)kWave ? causal_len - base : (uint32_t)kWave;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= alpha;
        for (uint32_t i = 0; i < rows; ++i) {
            const float pi = p_lds[i];
            const uint64_t vo = (uint64_t)(base + i) * pos_stride + head_off;
#pragma unroll
            for (int di = 0; di < 8; ++di) {
                const uint32_t d = lane + di * kWave;
                if (d < D) acc[di] = fmaf(pi, load_kv_elem(a.v, a.dtype, vo + d), acc[di]);
            }
        }
    }
    const float inv = 1.0f / l_run;
    float* o = a.o + ((size_t)qi * a.n_heads + h) * D;
#pragma unroll
    for (int di = 0; di < 8; ++di) {
        const uint32_t d = lane + di * kWave;
        if (d < D) o[d] = acc[di] * inv;
    }
}

hipError_t launch_batch(const BatchLaunch& L, hipStream_t stream) {
    if (L.dtype > kF8 || L.head_dim == 0u || L.head_dim > 512u) return hipErrorInvalidValue;
    if (L.m == 0u) return hipSuccess;
    BatchArgs a;
    a.q = L.q; a.k = (const uint8_t*)L.k; a.v = (const uint8_t*)L.v; a.o = L.o;
    a.n_heads = L.n_heads; a.n_kv_heads = L.n_kv_heads; a.head_dim = L.head_dim;
    a.m = L.m; a.n_kv = L.n_kv; a.q_start = L.q_start; a.kv_start = L.kv_start;
    a.scale = L.scale; a.softcap = L.softcap; a.dtype = L.dtype;
    hipLaunchKernelGGL(batch_generic_kernel, dim3(L.n_heads, L.m), dim3(kWave), 0, stream, a);
    return hipGetLastError();
}

}  // namespace vfkv
