// Split-K decode attention for gfx950: worker (flash_attn_split.comp:82-162) and log-sum-exp
// merge (flash_attn_reduce.comp:35-81), re-designed around the HBM stream.
//
// Worker layout.  One workgroup (4 wavefronts) owns one (tile of keys, KV head, group of GT query
// heads).  A K or V row of one KV head is D*elem bytes; LPR = D*elem/16 lanes cover it with one
// 16-byte load each, so a wavefront load instruction fetches RPI = 64/LPR complete rows and every
// byte of the row is requested exactly once per KV head -- the GT query heads of the GQA group are
// all served from the same registers.  Lane (r, c) keeps the c-th 16-byte slice of Q for each of the
// GT heads in registers, accumulates GT partial dot products per K row, and the LPR lanes of a row
// combine them with a butterfly.  Scores of a block of BI row-iterations stay in registers; the
// block maximum is made wavefront-uniform, weights are exponentiated once, and the same lanes then
// stream the V rows and accumulate GT x (16/elem) outputs each.  Row groups, wavefronts and finally
// workgroups are merged by log-sum-exp weights.  All arithmetic after the element decode is f32.
#include "device_utils.h"
#include "kernels.h"

namespace vfkv {

struct SplitArgs {
    const float* q;
    const uint8_t* k;
    const uint8_t* v;
    float* so;
    float* sm;
    float* ss;
    uint32_t n_heads, n_kv_heads;
    uint32_t seq_len, kv_start;
    uint32_t tile, tile_first, n_tiles;
    float scale, softcap;
};

template <int DT>
struct ElemBytes { static constexpr int value = DT == kF32 ? 4 : DT == kF16 ? 2 : 1; };

// Decode the 16 bytes a lane loaded into EPL floats.
template <int DT>
__device__ __forceinline__ void decode16(const uint4& raw, float* out) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    if (DT == kF8) {
#pragma unroll
        for (int j = 0; j < 4; ++j) e4m3x4_to_f32(w[j], out + 4 * j);
    } else if (DT == kF16) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            out[2 * j] = h16_bits_to_f32(w[j] & 0xFFFFu);
            out[2 * j + 1] = h16_bits_to_f32(w[j] >> 16);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) out[j] = __builtin_bit_cast(float, w[j]);
    }
}

constexpr int kSplitWaves = 4;

template <int DT, int D, int GT, int BI>
__global__ __launch_bounds__(kSplitWaves * kWave) void split_kernel(SplitArgs a) {
    constexpr int ES = ElemBytes<DT>::value;
    constexpr int EPL = 16 / ES;        // elements per lane per row
    constexpr int LPR = D / EPL;        // lanes per row
    constexpr int RPI = kWave / LPR;    // rows per wavefront load
    constexpr int NW = kSplitWaves;
    constexpr int ROWS_WG = NW * RPI;   // rows per workgroup iteration
    static_assert(LPR >= 1 && LPR <= kWave && (LPR & (LPR - 1)) == 0, "row must map onto a power-of-two lane group");

    __shared__ float lds_o[NW][GT][D];
    __shared__ float lds_m[NW][GT];
    __shared__ float lds_l[NW][GT];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = tid >> 6;
    const int c = lane % LPR;
    const int r = lane / LPR;

    const uint32_t jl = blockIdx.x;                 // tile index local to this launch
    const uint32_t kvh = blockIdx.y;
    const uint32_t g_per_kv = a.n_heads / a.n_kv_heads;
    const uint32_t h0 = kvh * g_per_kv + blockIdx.z * GT;

    const uint32_t tile_base = (a.tile_first + jl) * a.tile;
    uint32_t tile_end = tile_base + a.tile;
    if (tile_end > a.seq_len) tile_end = a.seq_len;
    const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;

    // Q slice of this lane for each head of the group.
    float qf[GT][EPL];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        const float4* qp = reinterpret_cast<const float4*>(a.q + (size_t)(h0 + g) * D + c * EPL);
#pragma unroll
        for (int e4 = 0; e4 < EPL / 4; ++e4) {
            const float4 f = qp[e4];
            qf[g][4 * e4 + 0] = f.x; qf[g][4 * e4 + 1] = f.y; qf[g][4 * e4 + 2] = f.z; qf[g][4 * e4 + 3] = f.w;
        }
    }

    float m_run[GT], l_run[GT], acc[GT][EPL];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
        m_run[g] = kMasked;
        l_run[g] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
    }

    const size_t row_stride = (size_t)a.n_kv_heads * D * ES;   // bytes between consecutive positions
    const size_t head_byte = (size_t)kvh * D * ES + (size_t)c * 16;
    const uint32_t last_row = a.seq_len - 1u;

    if (lo < tile_end) {
        for (uint32_t blk = tile_base; blk < tile_end; blk += BI * ROWS_WG) {
            if (blk + BI * ROWS_WG <= lo) continue;          // block entirely below the window
            uint4 kraw[BI], vraw[BI];
            uint32_t valid_bits = 0u;
#pragma unroll
            for (int i = 0; i < BI; ++i) {
                const uint32_t t = blk + i * ROWS_WG + w * RPI + r;
                const uint32_t tc = t < last_row ? t : last_row;   // stay inside the populated slab
                if (t < tile_end && t >= lo) valid_bits |= (1u << i);
                kraw[i] = *reinterpret_cast<const uint4*>(a.k + (size_t)tc * row_stride + head_byte);
            }
#pragma unroll
            for (int i = 0; i < BI; ++i) {
                const uint32_t t = blk + i * ROWS_WG + w * RPI + r;
                const uint32_t tc = t < last_row ? t : last_row;
                vraw[i] = *reinterpret_cast<const uint4*>(a.v + (size_t)tc * row_stride + head_byte);
            }

            // ---- scores of the block ----
            float s[BI][GT];
            float bmax[GT];
#pragma unroll
            for (int g = 0; g < GT; ++g) bmax[g] = kMasked;
#pragma unroll
            for (int i = 0; i < BI; ++i) {
                float kd[EPL];
                decode16<DT>(kraw[i], kd);
                const bool valid = (valid_bits >> i) & 1u;
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    float p = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) p = fmaf(qf[g][e], kd[e], p);
                    p = group_sum<LPR>(p) * a.scale;
                    if (a.softcap > 0.f) p = a.softcap * tanhf(p / a.softcap);
                    p = valid ? p : kMasked;
                    s[i][g] = p;
                    bmax[g] = fmaxf(bmax[g], p);
                }
            }
            // wavefront-uniform running maximum, rescale what has been accumulated so far
#pragma unroll
            for (int g = 0; g < GT; ++g) {
                float bm = bmax[g];
#pragma unroll
                for (int off = LPR; off < kWave; off <<= 1) bm = fmaxf(bm, __shfl_xor(bm, off, kWave));
                const float m_new = fmaxf(m_run[g], bm);
                if (m_new > m_run[g]) {   // wavefront-uniform
                    const float alpha = __expf(m_run[g] - m_new);
                    l_run[g] *= alpha;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[g][e] *= alpha;
                    m_run[g] = m_new;
                }
            }
            // ---- weights and V accumulation ----
#pragma unroll
            for (int i = 0; i < BI; ++i) {
                float vd[EPL];
                decode16<DT>(vraw[i], vd);
                const bool valid = (valid_bits >> i) & 1u;
#pragma unroll
                for (int g = 0; g < GT; ++g) {
                    const float p = valid ? __expf(s[i][g] - m_run[g]) : 0.f;
                    l_run[g] += p;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[g][e] = fmaf(p, vd[e], acc[g][e]);
                }
            }
        }
    }

    // ---- merge the RPI row groups of the wavefront (all share m_run) ----
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            l_run[g] += __shfl_xor(l_run[g], off, kWave);
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[g][e] += __shfl_xor(acc[g][e], off, kWave);
        }
    }
    if (r == 0) {
#pragma unroll
        for (int g = 0; g < GT; ++g) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) lds_o[w][g][c * EPL + e] = acc[g][e];
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < GT; ++g) {
            lds_m[w][g] = m_run[g];
            lds_l[w][g] = l_run[g];
        }
    }
    __syncthreads();

    // ---- merge the wavefronts and write the tile partial ----
    for (int idx = tid; idx < GT * D; idx += NW * kWave) {
        const int g = idx / D;
        const int d = idx - g * D;
        float M = lds_m[0][g];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) M = fmaxf(M, lds_m[ww][g]);
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) {
            const float f = __expf(lds_m[ww][g] - M);
            o = fmaf(f, lds_o[ww][g][d], o);
            l = fmaf(f, lds_l[ww][g], l);
        }
        const size_t pidx = (size_t)(h0 + g) * a.n_tiles + jl;
        a.so[pidx * D + d] = o;
        if (d == 0) {
            a.sm[pidx] = M;
            a.ss[pidx] = l;
        }
    }
}

// ---- generic worker: any head_dim <= 512, any dtype; one wavefront per (tile, head) -----------
// Lanes walk the keys of the tile 64 at a time (one key per lane, serial dot over d), then walk the
// output dimensions for the V sum.  Covers shapes the register-tiled kernel does not.
__global__ __launch_bounds__(kWave) void split_generic_kernel(SplitArgs a, uint32_t dtype, uint32_t D) {
    __shared__ float p_lds[kWave];
    const int lane = threadIdx.x;
    const uint32_t jl = blockIdx.x;
    const uint32_t h = blockIdx.y;
    const uint32_t kvh = h / (a.n_heads / a.n_kv_heads);
    const uint32_t tile_base = (a.tile_first + jl) * a.tile;
    uint32_t tile_end = tile_base + a.tile;
    if (tile_end > a.seq_len) tile_end = a.seq_len;
    const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;
    const uint64_t pos_stride = (uint64_t)a.n_kv_heads * D;
    const uint64_t head_off = (uint64_t)kvh * D;
    const float* q = a.q + (size_t)h * D;

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    float m_run = kMasked, l_run = 0.f;
    const uint32_t start = lo < tile_end ? (lo / kWave) * kWave : tile_end;
    for (uint32_t base = start; base < tile_end; base += kWave) {
        const uint32_t t = base + lane;
        const bool valid = t < tile_end && t >= lo;
        float sc = kMasked;
        if (valid) {
            const uint64_t ko = (uint64_t)t * pos_stride + head_off;
            float s = 0.f;
            for (uint32_t d = 0; d < D; ++d) s = fmaf(q[d], load_kv_elem(a.k, dtype, ko + d), s);
            s *= a.scale;
            if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
            sc = s;
        }
        const float bm = group_max<kWave>(sc);
        const float m_new = fmaxf(m_run, bm);
        const float alpha = __expf(m_run - m_new);
        const float p = valid ? __expf(sc - m_new) : 0.f;
        l_run = l_run * alpha + group_sum<kWave>(p);
        m_run = m_new;
        __syncthreads();
        p_lds[lane] = p;
        __syncthreads();
        const uint32_t rows = tile_end - base < (uint32_t)kWave ? tile_end - base : (uint32_t)kWave;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] *= alpha;
        for (uint32_t i = 0; i < rows; ++i) {
            const float pi = p_lds[i];
            const uint64_t vo = (uint64_t)(base + i) * pos_stride + head_off;
#pragma unroll
            for (int di = 0; di < 8; ++di) {
                const uint32_t d = lane + di * kWave;
                if (d < D) acc[di] = fmaf(pi, load_kv_elem(a.v, dtype, vo + d), acc[di]);
            }
        }
    }
    const size_t pidx = (size_t)h * a.n_tiles + jl;
#pragma unroll
    for (int di = 0; di < 8; ++di) {
        const uint32_t d = lane + di * kWave;
        if (d < D) a.so[pidx * D + d] = acc[di];
    }
    if (lane == 0) {
        a.sm[pidx] = m_run;
        a.ss[pidx] = l_run;
    }
}

// ---- log-sum-exp merge of the tile partials (flash_attn_reduce.comp:35-81) ---------------------
// One workgroup per head.  The global maximum over tiles is taken first so that the weighted sums
// have no serial dependency; mathematically this is the reference's running merge.
constexpr int kReduceThreads = 256;
__global__ __launch_bounds__(kReduceThreads) void reduce_kernel(const float* __restrict__ so,
                                                                const float* __restrict__ sm,
                                                                const float* __restrict__ ss,
                                                                float* __restrict__ o, uint32_t D,
                                                                uint32_t n_tiles) {
    extern __shared__ float lds[];   // [parts][D] partial sums, then [parts] partial L
    __shared__ float red[kReduceThreads / kWave];
    const uint32_t h = blockIdx.x;
    const int tid = threadIdx.x;
    const float* hm = sm + (size_t)h * n_tiles;
    const float* hs = ss + (size_t)h * n_tiles;
    const float* ho = so + (size_t)h * n_tiles * D;

    float M = kMasked;
    for (uint32_t j = tid; j < n_tiles; j += kReduceThreads) M = fmaxf(M, hm[j]);
    M = group_max<kWave>(M);
    if ((tid & (kWave - 1)) == 0) red[tid >> 6] = M;
    __syncthreads();
    M = red[0];
#pragma unroll
    for (int i = 1; i < kReduceThreads / kWave; ++i) M = fmaxf(M, red[i]);
    __syncthreads();

    float L = 0.f;
    for (uint32_t j = tid; j < n_tiles; j += kReduceThreads) L += __expf(hm[j] - M) * hs[j];
    L = group_sum<kWave>(L);
    if ((tid & (kWave - 1)) == 0) red[tid >> 6] = L;
    __syncthreads();
    L = 0.f;
#pragma unroll
    for (int i = 0; i < kReduceThreads / kWave; ++i) L += red[i];

    // threads = (part, d4): each sums its share of the tiles for four consecutive d
    const uint32_t d4n = D / 4u;                       // D is a multiple of 4 on this path
    const uint32_t parts = kReduceThreads / d4n > 0 ? kReduceThreads / d4n : 1u;
    const uint32_t part = tid / d4n, d4 = tid % d4n;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (part < parts) {
        for (uint32_t j = part; j < n_tiles; j += parts) {
            const float wj = __expf(hm[j] - M);
            const float4 x = *reinterpret_cast<const float4*>(ho + (size_t)j * D + 4u * d4);
            acc.x = fmaf(wj, x.x, acc.x); acc.y = fmaf(wj, x.y, acc.y);
            acc.z = fmaf(wj, x.z, acc.z); acc.w = fmaf(wj, x.w, acc.w);
        }
        float* dst = lds + (size_t)part * D + 4u * d4;
        dst[0] = acc.x; dst[1] = acc.y; dst[2] = acc.z; dst[3] = acc.w;
    }
    __syncthreads();
    const float inv = 1.0f / L;
    for (uint32_t d = tid; d < D; d += kReduceThreads) {
        float sum = 0.f;
        for (uint32_t p = 0; p < parts; ++p) sum += lds[(size_t)p * D + d];
        o[(size_t)h * D + d] = sum * inv;
    }
}

// scalar variant for head_dim not a multiple of 4 (or > 1024 threads' worth): one thread per d
__global__ __launch_bounds__(kWave) void reduce_generic_kernel(const float* __restrict__ so,
                                                               const float* __restrict__ sm,
                                                               const float* __restrict__ ss,
                                                               float* __restrict__ o, uint32_t D, uint32_t n_tiles) {
    const uint32_t h = blockIdx.x;
    const float* hm = sm + (size_t)h * n_tiles;
    const float* hs = ss + (size_t)h * n_tiles;
    const float* ho = so + (size_t)h * n_tiles * D;
    float M = kMasked;
    for (uint32_t j = 0; j < n_tiles; ++j) M = fmaxf(M, hm[j]);
    float L = 0.f;
    for (uint32_t j = 0; j < n_tiles; ++j) L += __expf(hm[j] - M) * hs[j];
    const float inv = 1.0f / L;
    for (uint32_t d = threadIdx.x; d < D; d += kWave) {
        float acc = 0.f;
        for (uint32_t j = 0; j < n_tiles; ++j) acc = fmaf(__expf(hm[j] - M), ho[(size_t)j * D + d], acc);
        o[(size_t)h * D + d] = acc * inv;
    }
}

// ---- dispatch -----------------------------------------------------------------------------------
template <int DT, int D>
struct SplitTraits {
    static constexpr int ES = ElemBytes<DT>::value;
    static constexpr int LPR = D * ES / 16;
    static constexpr int RPI = kWave / LPR;
    static constexpr int BI = 8;
    static constexpr uint32_t granule = kSplitWaves * RPI;   // rows per workgroup iteration
};

template <int DT, int D, int GT>
static hipError_t launch_split_t(const SplitArgs& a, uint32_t groups, hipStream_t stream) {
    constexpr int BI = SplitTraits<DT, D>::BI;
    dim3 grid(a.n_tiles, a.n_kv_heads, groups);
    hipLaunchKernelGGL((split_kernel<DT, D, GT, BI>), grid, dim3(kSplitWaves * kWave), 0, stream, a);
    return hipGetLastError();
}

template <int DT, int D>
static hipError_t launch_split_d(const SplitArgs& a, uint32_t g, hipStream_t stream) {
    if (g % 4u == 0u) return launch_split_t<DT, D, 4>(a, g / 4u, stream);
    if (g % 2u == 0u) return launch_split_t<DT, D, 2>(a, g / 2u, stream);
    return launch_split_t<DT, D, 1>(a, g, stream);
}

static bool fast_shape(uint32_t dtype, uint32_t D) {
    if (D != 64u && D != 128u && D != 256u && D != 512u) return false;
    return D * elem_size(dtype) / 16u <= (uint32_t)kWave;
}

uint32_t split_tile_granule(uint32_t dtype, uint32_t D) {
    if (dtype > kF8 || D == 0u || D > 512u) return 0u;
    if (!fast_shape(dtype, D)) return (uint32_t)kWave;
    const uint32_t lpr = D * elem_size(dtype) / 16u;
    return kSplitWaves * (kWave / lpr);
}

hipError_t launch_split(const SplitLaunch& L, hipStream_t stream) {
    if (L.dtype > kF8 || L.head_dim == 0u || L.head_dim > 512u) return hipErrorInvalidValue;
    if (L.n_tiles == 0u) return hipSuccess;
    SplitArgs a;
    a.q = L.q; a.k = (const uint8_t*)L.k; a.v = (const uint8_t*)L.v;
    a.so = L.scratch_out; a.sm = L.scratch_max; a.ss = L.scratch_sum;
    a.n_heads = L.n_heads; a.n_kv_heads = L.n_kv_heads;
    a.seq_len = L.seq_len; a.kv_start = L.kv_start;
    a.tile = L.tile; a.tile_first = L.tile_first; a.n_tiles = L.n_tiles;
    a.scale = L.scale; a.softcap = L.softcap;
    const uint32_t g = L.n_heads / L.n_kv_heads;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q)) & 15u) == 0u;
    if (fast_shape(L.dtype, L.head_dim) && aligned) {
#define VFKV_CASE(DT, DD) \
    if (L.dtype == DT && L.head_dim == DD) return launch_split_d<DT, DD>(a, g, stream);
        VFKV_CASE(kF8, 64) VFKV_CASE(kF8, 128) VFKV_CASE(kF8, 256) VFKV_CASE(kF8, 512)
        VFKV_CASE(kF16, 64) VFKV_CASE(kF16, 128) VFKV_CASE(kF16, 256) VFKV_CASE(kF16, 512)
        VFKV_CASE(kF32, 64) VFKV_CASE(kF32, 128) VFKV_CASE(kF32, 256)
#undef VFKV_CASE
    }
    dim3 grid(L.n_tiles, L.n_heads, 1);
    hipLaunchKernelGGL(split_generic_kernel, grid, dim3(kWave), 0, stream, a, L.dtype, L.head_dim);
    return hipGetLastError();
}

hipError_t launch_reduce(const float* so, const float* sm, const float* ss, float* o, uint32_t n_heads,
                         uint32_t D, uint32_t n_tiles, hipStream_t stream) {
    if (n_heads == 0u || D == 0u || n_tiles == 0u) return hipErrorInvalidValue;
    const bool vec = (D % 4u == 0u) && (D / 4u <= (uint32_t)kReduceThreads) &&
                     ((((uintptr_t)so) & 15u) == 0u);
    if (vec) {
        const uint32_t d4n = D / 4u;
        const uint32_t parts = kReduceThreads / d4n;
        const size_t lds = (size_t)parts * D * sizeof(float);
        hipLaunchKernelGGL(reduce_kernel, dim3(n_heads), dim3(kReduceThreads), lds, stream, so, sm, ss, o, D, n_tiles);
    } else {
        hipLaunchKernelGGL(reduce_generic_kernel, dim3(n_heads), dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles);
    }
    return hipGetLastError();
}

}  // namespace vfkv
