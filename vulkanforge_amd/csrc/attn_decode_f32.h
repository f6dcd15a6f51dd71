// Matrix-core worker of the split-K decode attention (flash_attn_split.comp:82-162) over F32 caches (the reference's
// VULKANFORGE_FP16_KV=0 mode, kv_cache.rs:85-101, and the dtype its own attention tests run on); included by
// attn_decode.hip.  Every product is an f32 x f32 product accumulated in f32 on v_mfma_f32_16x16x4_f32, as in the shader.
//
// One workgroup (NW wavefronts) owns one (share of the keys, KV head, slice of up to 16 query heads of the GQA group);
// every K / V byte is requested once and serves all heads of the slice.  A wavefront walks its share in runs of 16 rows,
// one run in flight ahead of the one being computed:
//
//   S^T[row, head]  = K[row, :] . Q[head, :]   A = K straight from 16-byte loads: lane (row l % 16, group l / 16) holds the
//                                              pieces x * 4 + l / 16 (x = 0, 1, ...) of its row, so one load instruction
//                                              covers 64 contiguous bytes of each row and a 128-byte line is complete
//                                              after two; B = the same elements of the lane's query head, loaded once.
//                                              The sum over head_dim does not care in which order the MFMA steps take
//                                              the elements: step c multiplies element c of every lane group.
//   softmax         in the accumulator layout (a lane owns rows 4 * (l / 16) + i of ONE head): exact running maximum
//                   over the run through two lane swaps, exp2, the accumulators rescaled only when a maximum moved.
//   O^T[d, head]   += V^T[d, row] . P[row, head]  A = V^T: lane (l % 16, row l / 16 of a group of four) reads 16 bytes, the
//                                              elements d = 64 b + 4 (l % 16) + j, j < 4, of its row, and uses element j
//                                              in output tile 4 b + j (which d an output tile's row m stands for is free:
//                                              here d = 64 b + 4 m + j, so that loads are 16 bytes wide and 256 contiguous
//                                              bytes per row; the stores at the end use the same map); B = P needs row
//                                              4 * g + l / 16 where the accumulator layout holds row 4 * (l / 16) + i: a
//                                              4 x 4 transpose between registers and 16-lane rows, four lane swaps.
//
// Partials, the workgroup merge through LDS, the two ways of dealing rows (tile j = partial j, or interleaved runs) and the
// single-tile form that writes the output itself are those of split_mfma_kernel (attn_decode_mfma.h).
#pragma once
#include <type_traits>

namespace vfkv {

// PAD: the heads are `head_dim` < D elements wide (a multiple of 16).  The kernel works on rows of D elements whose tail
// does not exist: a lane's query elements past head_dim are zeros, its 16-byte pieces of a K or V row past the head are
// the head's first piece read again (finite values that meet the zeros, or output elements nobody stores), and output
// elements past head_dim are not stored.  Rows, queries and partials keep their real stride of head_dim.
template <int D, int NW, bool CAP, bool PAD = false>
__global__ __launch_bounds__(NW * 64) void split_mfma_f32_kernel(SplitArgs a, uint32_t gt, uint32_t head_dim) {
    constexpr int RUN = 16;                      // rows per run: one MFMA tile
    constexpr int NC = D / 4;                    // MFMA steps of the first product = elements of a row per lane group
    constexpr int KV4 = NC / 4;                  // 16-byte loads per lane and run (K)
    constexpr int DTILES = D / 16;
    constexpr int VB = DTILES / 4;                // 64-element blocks of a row: one 16-byte V load per lane, row group and block
    static_assert(D % 64 == 0 && NC % 4 == 0 && DTILES % NW == 0, "unsupported head_dim");

    __shared__ __attribute__((aligned(16))) float4_t slot[NW * DTILES * 64];    // the wavefronts' accumulators, for the merge
    __shared__ float lds_m[NW][16], lds_l[NW][16];

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n16 = lane & 15, kg = lane >> 4;
    const uint32_t kvh = blockIdx.x, jl = blockIdx.y;
    const uint32_t g_all = a.group;
    const uint32_t hz = blockIdx.z * gt;
    const uint32_t gcount = g_all - hz < gt ? g_all - hz : gt;     // <= 16
    const uint32_t h0 = kvh * g_all + hz;
    const bool il = a.interleave != 0u;
    const uint32_t tile_base = il ? a.tile_first * a.tile : (a.tile_first + jl) * a.tile;
    uint32_t tile_end = tile_base + a.tile; if (il || tile_end > a.seq_len) tile_end = a.seq_len;
    const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;

    const uint32_t dr = PAD ? head_dim : (uint32_t)D;                           // elements per head as the cache holds them
    const uint32_t row_stride = a.n_kv_heads * dr * 4u;
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.seq_len * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.seq_len * row_stride, 0x00020000);
    const uint32_t head_b = kvh * dr * 4u;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * 16;              // row l % 16, pieces kg, kg + 4, ...
    const uint32_t lane_voff = kg * row_stride + head_b + n16 * 16;              // row l / 16 of a group of four, elements 4 (l % 16) .. + 3 of a block
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;
    const float inv_cap_l2 = CAP ? 1.0f / cap_l2 : 0.f;

    const uint32_t first_run = (lo - tile_base) / RUN;
    const uint32_t n_runs = tile_end > tile_base ? (tile_end - tile_base + RUN - 1) / RUN : 0;
    auto run_off = [&](uint32_t r) -> uint32_t { return r < n_runs ? (tile_base + r * RUN) * row_stride : kOOB; };
    const uint32_t rs = il ? NW * a.n_tiles : NW;                              // distance between two runs of a wavefront
    const uint32_t r0 = first_run + (il ? jl * NW : 0u) + (uint32_t)w;
    const bool active = lo < tile_end && r0 < n_runs;

    u32x4 kraw[KV4];
    u32x4 vraw[4][VB];
    auto issue_k = [&](uint32_t off) {
#pragma unroll
        for (int x = 0; x < KV4; ++x)
            kraw[x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, (PAD && (uint32_t)(kg * 16 + x * 64) >= dr * 4u) ? n16 * row_stride + head_b
                                                                                                                : lane_koff + x * 64, off, 0);
    };
    auto issue_v = [&](uint32_t off) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
            for (int b = 0; b < VB; ++b)
                vraw[g4][b] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, (PAD && (uint32_t)(n16 * 16 + b * 256) >= dr * 4u) ? kg * row_stride + head_b
                                                                                                                          : lane_voff + b * 256,
                                                                    off + (uint32_t)(g4 * 4) * row_stride, 0);
    };
    const uint32_t off0 = active ? run_off(r0) : kOOB;
    issue_k(off0);
    // ---- this lane's elements of its query head, in the order the K pieces come: the B operand of every first product.
    // Requested between the K and the V rows of the first run: loads return in order, so waiting for it covers K only.
    float qf[NC];
    {
        const bool col_ok = (uint32_t)n16 < gcount;
        const float* qrow = a.q + (size_t)(h0 + (col_ok ? n16 : 0)) * dr + kg * 4;
#pragma unroll
        for (int x = 0; x < KV4; ++x) {
            const bool piece_ok = !PAD || (uint32_t)(kg * 4 + x * 16) < dr;
            float4 v = *reinterpret_cast<const float4*>(qrow + (piece_ok ? x * 16 : -kg * 4));
            if (!piece_ok) v = make_float4(0.f, 0.f, 0.f, 0.f);
            qf[4 * x] = col_ok ? v.x : 0.f; qf[4 * x + 1] = col_ok ? v.y : 0.f;
            qf[4 * x + 2] = col_ok ? v.z : 0.f; qf[4 * x + 3] = col_ok ? v.w : 0.f;
        }
    }
    issue_v(off0);

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;

    if (active) {
        for (uint32_t r = r0; r < n_runs; r += rs) {
            const uint32_t noff = run_off(r + rs);
            const uint32_t rb = tile_base + r * RUN;
            // ---- operands of this run out of the load registers, the next run requested ----
            float kf[NC], va[4][DTILES];
#pragma unroll
            for (int x = 0; x < KV4; ++x) {
                const u32x4 v = kraw[x];                 // (the whole vector is copied before its elements are taken)
                kf[4 * x] = __builtin_bit_cast(float, (uint32_t)v[0]); kf[4 * x + 1] = __builtin_bit_cast(float, (uint32_t)v[1]);
                kf[4 * x + 2] = __builtin_bit_cast(float, (uint32_t)v[2]); kf[4 * x + 3] = __builtin_bit_cast(float, (uint32_t)v[3]);
            }
            issue_k(noff);
            // ---- S^T = K Q^T (two accumulators: the steps of one chain depend on each other) ----
            float4_t s0 = float4_t{0.f, 0.f, 0.f, 0.f}, s1 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; c += 2) {
                s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[c], qf[c], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[c + 1], qf[c + 1], s1, 0, 0, 0);
            }
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
                for (int b = 0; b < VB; ++b) {
                    const u32x4 v = vraw[g4][b];
                    va[g4][4 * b] = __builtin_bit_cast(float, (uint32_t)v[0]); va[g4][4 * b + 1] = __builtin_bit_cast(float, (uint32_t)v[1]);
                    va[g4][4 * b + 2] = __builtin_bit_cast(float, (uint32_t)v[2]); va[g4][4 * b + 3] = __builtin_bit_cast(float, (uint32_t)v[3]);
                }
            issue_v(noff);
            // ---- softmax: this lane owns rows rb + 4 * kg + i of head n16 ----
            const bool interior = rb >= lo && rb + RUN <= tile_end;      // wavefront-uniform
            float p[4];
            auto softmax = [&](auto masked_tag) {
                constexpr bool MASKED = decltype(masked_tag)::value;
                float x[4];
                float tmax = kMasked;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = (s0[i] + s1[i]) * scale_l2;
                    if (CAP) y = softcap_l2(y, cap_l2, inv_cap_l2);
                    if (MASKED) {
                        const uint32_t row = rb + kg * 4 + i;
                        y = (row >= lo && row < tile_end) ? y : kMasked;
                    }
                    x[i] = y;
                    tmax = fmaxf(tmax, y);
                }
                { float y = tmax; swap16(tmax, y); tmax = fmaxf(tmax, y); y = tmax; swap32(tmax, y); tmax = fmaxf(tmax, y); }
                const float m_new = fmaxf(m_run, tmax);
                if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0ull) {
                    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                    l_run *= alpha;
#pragma unroll
                    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] *= alpha;
                    m_run = m_new;
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float pv = __builtin_amdgcn_exp2f(x[i] - m_run);
                    if (MASKED) pv = x[i] > -1e29f ? pv : 0.f;
                    p[i] = pv;
                    l_run += pv;
                }
            };
            if (interior) softmax(std::false_type{}); else softmax(std::true_type{});
            // ---- registers x 16-lane rows transpose: afterwards p[g] of lane group k is the weight of row rb + 4 * g + k ----
            swap32(p[0], p[2]);
            swap32(p[1], p[3]);
            swap16(p[0], p[1]);
            swap16(p[2], p[3]);
            // ---- O^T += V^T P ----
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt)
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[g4][dt], p[g4], oacc[dt], 0, 0, 0);
        }
    }

    // ---------------- wavefront totals, then the workgroup merge through LDS ----------------
    // Every wavefront parks its accumulators in LDS in register order (lane-major: conflict-free 16-byte accesses), then
    // wavefront w merges the d-tiles w, w + NW, ... of all wavefronts and stores them straight from registers.
    l_run = xor32_sum(xor16_sum(l_run));
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) slot[(w * DTILES + dt) * 64 + lane] = oacc[dt];
    if (kg == 0) { lds_m[w][n16] = m_run; lds_l[w][n16] = l_run; }
    __syncthreads();
    constexpr int MT = DTILES / NW;
    float mw[NW], lw[NW];
    float4_t part[MT][NW];
#pragma unroll
    for (int pp = 0; pp < NW; ++pp) { mw[pp] = lds_m[pp][n16]; lw[pp] = lds_l[pp][n16]; }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int pp = 0; pp < NW; ++pp) part[t][pp] = slot[(pp * DTILES + t * NW + w) * 64 + lane];
    float M = mw[0];
#pragma unroll
    for (int pp = 1; pp < NW; ++pp) M = fmaxf(M, mw[pp]);
    float fw[NW];
    float l = 0.f;
#pragma unroll
    for (int pp = 0; pp < NW; ++pp) {
        fw[pp] = __builtin_amdgcn_exp2f(mw[pp] - M);
        l = fmaf(fw[pp], lw[pp], l);
    }
    const bool writer = (uint32_t)n16 < gcount;
    const size_t pidx = (size_t)(h0 + n16) * a.n_tiles + jl;
    // a single tile covers every visible key (the reference's single-workgroup shader for seq <= 64,
    // forward/runs.rs:776-821): the merge is a plain normalisation, done here, and no merge launch follows
    const bool direct = a.o_direct != nullptr;
    const float inv_l = direct ? __builtin_amdgcn_rcpf(l) : 1.0f;
    float* const obase = direct ? a.o_direct + (size_t)(h0 + n16) * dr : a.so + pidx * dr;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        float4_t o = fw[0] * part[t][0];
#pragma unroll
        for (int pp = 1; pp < NW; ++pp) o += fw[pp] * part[t][pp];
        if (direct) {                                  // one Newton step brings the reciprocal to f32 accuracy
            const float rcp = inv_l * (2.0f - l * inv_l);
            o *= rcp;
        }
        if (writer) {      // output tile dt = 4 b + j, accumulator row m = 4 kg + i  <->  d = 64 b + 4 m + j
            const int dt = t * NW + w;
            float* const dst = obase + (dt / 4) * 64 + (kg * 4) * 4 + (dt % 4);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (!PAD || (uint32_t)((dt / 4) * 64 + (kg * 4 + i) * 4 + (dt % 4)) < dr) dst[i * 4] = o[i];
        }
    }
    if (writer && w == 0 && kg == 0 && !direct) {
        a.sm[pidx] = M > -1e29f ? M * 0.693147180559945f : kMasked;
        a.ss[pidx] = l;
    }
}

}  // namespace vfkv
