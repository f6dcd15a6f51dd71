// Chunked-prefill causal attention on the f32 matrix-core instruction (v_mfma_f32_16x16x4_f32).
//
// Replaces flash_attn_batch.comp:105-208 for the reference's FP32-KV mode (kv_cache.rs:76-102, VULKANFORGE_FP16_KV=0) and for
// head_dim 96, which the f16 matrix-core kernel does not cover: FP8 / F16 rows are widened to f32 in registers (exact),
// every product is an f32 x f32 product accumulated in f32, as in the shader.  One wavefront per (16 queries, query head,
// slice of head_dim): four heads of a KV head per workgroup, no LDS, no barrier.  With NH = 2 (head_dim 512) two
// wavefronts share a head: both compute the scores over the whole head_dim, each accumulates and stores one half of the
// output (the accumulators of a 512-wide head do not fit one wavefront).  Per tile of 16 keys:
//   S^T = K Q^T     A = K: lane (key l % 16, group l / 16) holds the group's quarter of the key row (contiguous bytes, so the
//                   loads are wide loads); B = Q: the same quarter of the lane's query row, loaded once.  The sum over
//                   head_dim does not care in which order the MFMA steps take the elements, so step c multiplies element
//                   c of every quarter.
//   softmax         in the C layout (lane = query l % 16, keys 4 * (l / 16) + r): lazy reference maximum (it only moves
//                   when a score exceeds it by 2^8), exp2, row sums per lane (reduced once at the end).
//   O^T += V^T P^T  B = P^T needs key 4 * g + (l / 16) of step g where the C layout holds key 4 * (l / 16) + r: a 4 x 4
//                   transpose between registers and 16-lane rows, four lane-swap instructions.  A = V^T: lane (d l % 16,
//                   key l / 16) reads single elements, 16 contiguous elements per 16 lanes.
// MFMA bound: (head_dim + head_dim / NH) / 4 instructions of 32 cycles per tile and wavefront; the f32 matrix rate of the
// GPU is 1/16 of its f16 rate.
#pragma once

namespace vfkv {

template <int DT, int D, int NH, bool CAP>
__global__ __launch_bounds__(256) void batch_mfma_f32_kernel(BatchArgs a) {
    constexpr int ES = DT == kF32 ? 4 : DT == kF16 ? 2 : 1;
    constexpr int NC = D / 4;                    // MFMA steps of the first product = elements of a key row per lane group
    constexpr int QB = NC * ES;                  // bytes of that quarter of a row
    constexpr bool WIDE = QB % 16 == 0;          // 16-byte loads, else 4-byte loads
    constexpr int KDW = QB / 4;                  // dwords per lane and K tile
    constexpr int QLD = NC / 4;                  // 16-byte loads of the query quarter
    constexpr int DV = D / NH;                   // output elements of this wavefront
    constexpr int DTILES = DV / 16;
    constexpr int KT = 16;                       // keys per tile
    constexpr float kMaxSlack = 8.0f;            // log2 units by which a score may exceed the running reference maximum
    constexpr uint32_t kNoTile = 0x80000000u;    // byte offset past any slab: the load returns zeros, no memory access
    static_assert(D % 16 == 0 && DV % 16 == 0 && QB % 4 == 0, "unsupported head_dim");

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n16 = lane & 15, kg = lane >> 4;
    const uint32_t G = a.n_heads / a.n_kv_heads;
    const uint32_t half = blockIdx.z % NH;                      // which slice of the output this wavefront accumulates
    const uint32_t g = (blockIdx.z / NH) * 4u + (uint32_t)w;    // head inside the GQA group
    if (g >= G) return;                                         // wavefronts never meet at a barrier
    const uint32_t kvh = blockIdx.y, h = kvh * G + g;
    const uint32_t q0 = (gridDim.x - 1u - blockIdx.x) * 16u, qi = q0 + n16;   // this lane's query (column of S^T); later blocks see more keys: longest first
    const bool q_ok = qi < a.m;
    const uint32_t row_stride = a.n_kv_heads * D * ES;          // bytes between two keys

    uint32_t kmax = a.q_start + q0 + 16u;                       // one past the last key any of the 16 queries sees
    if (kmax > a.n_kv) kmax = a.n_kv;
    const uint32_t my_len = q_ok ? (a.q_start + qi + 1u < a.n_kv ? a.q_start + qi + 1u : a.n_kv) : 0u;
    const uint32_t t_first = (a.kv_start / KT) * KT;
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;

    // ---- this lane's quarter of its query row: the B operand of every first product ----
    float qf[NC];
    {
        const float* qrow = a.q + ((size_t)(q_ok ? qi : 0u) * a.n_heads + h) * D + kg * NC;
#pragma unroll
        for (int c4 = 0; c4 < QLD; ++c4) {
            const float4 v = *reinterpret_cast<const float4*>(qrow + 4 * c4);
            qf[4 * c4] = q_ok ? v.x : 0.f; qf[4 * c4 + 1] = q_ok ? v.y : 0.f;
            qf[4 * c4 + 2] = q_ok ? v.z : 0.f; qf[4 * c4 + 3] = q_ok ? v.w : 0.f;
        }
    }
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.n_kv * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.n_kv * row_stride, 0x00020000);
    const uint32_t head_b = kvh * D * ES;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * QB;                      // key l % 16, quarter l / 16
    const uint32_t lane_voff = kg * row_stride + head_b + (half * DV + n16) * ES;        // key l / 16 of a group of four, element l % 16

    constexpr int KV4 = WIDE ? KDW / 4 : 1;
    u32x4 kraw4[KV4];                            // WIDE: the quarter row as 16-byte pieces
    uint32_t kraw[WIDE ? 1 : KDW];
    uint32_t vraw[4][DTILES];
    auto issue = [&](uint32_t toff) {
        if constexpr (WIDE) {
#pragma unroll
            for (int x = 0; x < KV4; ++x) kraw4[x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * 16, toff, 0);
        } else {
#pragma unroll
            for (int x = 0; x < KDW; ++x) kraw[x] = __builtin_amdgcn_raw_buffer_load_b32(krsrc, lane_koff + x * 4, toff, 0);
        }
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const uint32_t so = toff + (uint32_t)(g4 * 4) * row_stride;
                if (DT == kF32) vraw[g4][dt] = __builtin_amdgcn_raw_buffer_load_b32(vrsrc, lane_voff + dt * 16 * ES, so, 0);
                else if (DT == kF16) vraw[g4][dt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(vrsrc, lane_voff + dt * 16 * ES, so, 0);
                else vraw[g4][dt] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b8(vrsrc, lane_voff + dt * 16 * ES, so, 0);
            }
    };
    // element c of the lane's key-row quarter / a gathered V element, widened to f32 (exact)
    auto k_elem = [&](const uint32_t (&raw)[KDW], int c) -> float {
        if (DT == kF32) return __builtin_bit_cast(float, raw[c]);
        if (DT == kF16) { const half2_t h2 = __builtin_bit_cast(half2_t, raw[c / 2]); return (float)h2[c % 2]; }
        switch (c % 4) {
            case 0: return __builtin_amdgcn_cvt_f32_fp8((int)raw[c / 4], 0);
            case 1: return __builtin_amdgcn_cvt_f32_fp8((int)raw[c / 4], 1);
            case 2: return __builtin_amdgcn_cvt_f32_fp8((int)raw[c / 4], 2);
            default: return __builtin_amdgcn_cvt_f32_fp8((int)raw[c / 4], 3);
        }
    };
    auto v_elem = [&](uint32_t raw) -> float {
        if (DT == kF32) return __builtin_bit_cast(float, raw);
        if (DT == kF16) return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
        return __builtin_amdgcn_cvt_f32_fp8((int)raw, 0);
    };
    auto tile_off = [&](uint32_t t) -> uint32_t { return t < kmax ? t * row_stride : kNoTile; };

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;

    issue(tile_off(t_first));
    for (uint32_t t = t_first; t < kmax; t += KT) {
        // ---- operands of this tile out of the load registers, next tile requested ----
        uint32_t kcur[KDW];
        float va[4][DTILES];
        if constexpr (WIDE) {
#pragma unroll
            for (int x = 0; x < KV4; ++x) {
                const u32x4 v = kraw4[x];                                // (the whole vector is copied before its elements are taken)
                kcur[4 * x] = v[0]; kcur[4 * x + 1] = v[1]; kcur[4 * x + 2] = v[2]; kcur[4 * x + 3] = v[3];
            }
        } else {
#pragma unroll
            for (int x = 0; x < KDW; ++x) kcur[x] = kraw[x];
        }
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) va[g4][dt] = v_elem(vraw[g4][dt]);
        issue(tile_off(t + KT));
        // ---- S^T = K Q^T (two accumulators: the steps of one chain depend on each other) ----
        float4_t s0 = float4_t{0.f, 0.f, 0.f, 0.f}, s1 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; c += 2) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(k_elem(kcur, c), qf[c], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(k_elem(kcur, c + 1), qf[c + 1], s1, 0, 0, 0);
        }
        // ---- softmax: this lane owns keys t + 4 * kg + r of query n16 ----
        float y[4], p[4];
        float tmax = kMasked;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = (s0[r] + s1[r]) * scale_l2;
            if (CAP) v = cap_l2 * tanhf(v / cap_l2);
            const uint32_t tk = t + 4u * kg + r;
            v = (tk < my_len && tk >= a.kv_start) ? v : kMasked;
            y[r] = v;
            tmax = fmaxf(tmax, v);
        }
        if (__builtin_amdgcn_ballot_w64(tmax > m_run + kMaxSlack) != 0ull) {    // the four lanes of a query share m_run
            { float z = tmax; swap16(tmax, z); tmax = fmaxf(tmax, z); z = tmax; swap32(tmax, z); tmax = fmaxf(tmax, z); }
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) oacc[dt] *= alpha;
            m_run = m_new;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = y[r] > -1e29f ? __builtin_amdgcn_exp2f(y[r] - m_run) : 0.f;
            l_run += p[r];
        }
        // ---- registers x 16-lane rows transpose: afterwards p[g] of lane group k is the weight of key t + 4 * g + k ----
        swap32(p[0], p[2]);
        swap32(p[1], p[3]);
        swap16(p[0], p[1]);
        swap16(p[2], p[3]);
        // ---- O^T += V^T P^T ----
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[g4][dt], p[g4], oacc[dt], 0, 0, 0);
    }
    // ---- normalise and store: the lane holds O[query n16][half * DV + dt * 16 + 4 * kg + r] ----
    l_run = xor32_sum(xor16_sum(l_run));
    if (!q_ok) return;
    const float inv = 1.0f / l_run;
    float* orow = a.o + ((size_t)qi * a.n_heads + h) * D + half * DV + 4 * kg;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
        *reinterpret_cast<float4*>(orow + dt * 16) = make_float4(oacc[dt][0] * inv, oacc[dt][1] * inv, oacc[dt][2] * inv, oacc[dt][3] * inv);
}

}  // namespace vfkv
