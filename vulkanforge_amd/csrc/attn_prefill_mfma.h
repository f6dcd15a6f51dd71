// MFMA (matrix-core) kernel of the chunked-prefill attention for gfx950; included by attn_prefill.hip.
//
// Workgroup = one KV head x 16 consecutive queries x NSPLIT key splits; wavefront w serves query head
// kvh*G + w%G and the key tiles  w/G, w/G + NSPLIT, ...; the G wavefronts of a split share every K and V
// tile, and the splits (which only exist to put more wavefronts on each SIMD) are merged through LDS at
// the end with log-sum-exp weights.  Per tile of 32 keys each wavefront computes, with
// v_mfma_f32_16x16x32_f16 (f32 accumulation):
//
//   S^T[key, query]  = K[key, :] . Q[query, :]        A = K rows straight from global memory (each lane
//                                                     reads a contiguous quarter of a key row; FP8 is
//                                                     widened to f16 in registers, which is exact),
//                                                     B = Q^T held in registers for the whole kernel
//   softmax (online) : the S^T accumulator layout gives every lane 8 scores of ONE query, so max / sum
//                      need two cross-row lane exchanges per tile and the weights are already in the
//                      layout the next product wants as its B operand -- P never leaves registers
//   O^T[d, query]   += V^T[d, key] . P^T[key, query]   A = V^T, read from a row-major f16 copy of the V
//                                                     tile in LDS with the transposing LDS read
//                                                     (ds_read_b64_tr_b16), B = P^T
//
// The contraction index of an MFMA may be permuted freely as long as both operands agree; that is used
// twice: K rows are split over the four lane groups in contiguous quarters (coalesced 16-byte loads),
// and the 8 key slots of a lane in the second product are keys {4g..4g+3} of each 16-key half of the
// tile (exactly the keys whose scores that lane already owns).
//
// Q is used as f16: hi = f16(q); when some q is not exactly representable the products are repeated
// with lo = f16(q - hi), which restores f32-level accuracy.  P enters the second product as
// f16(p) + f16(p - f16(p)) (two MFMAs), so the weights keep ~22 significant bits as well.
#pragma once

namespace vfkv {

template <int DT, int D, bool CAP, int MAXT, int NSPLIT, int PFD>
__global__ __launch_bounds__(MAXT) void batch_mfma_kernel(BatchArgs a) {
    constexpr int ES = DT == kF16 ? 2 : 1;
    constexpr int KT = 32;                       // keys per tile
    constexpr int KS = D / 32;                   // MFMA k-steps of the first product
    constexpr int DTILES = D / 16;               // 16-wide d tiles of the output
    constexpr int SEG = D / 4;                   // elements of a key row owned by one lane group
    constexpr int SEGB = SEG * ES;               // ... in bytes (32 for FP8 D=128, 64 for F16 D=128)
    constexpr int KLD = SEGB / 16;               // 16-byte loads per lane per key row
    constexpr int VPITCH = D + 16;               // halves per V row in LDS (+32 B against bank conflicts)
    static_assert(D % 32 == 0 && SEGB % 16 == 0, "unsupported head_dim");

    extern __shared__ __attribute__((aligned(16))) _Float16 vlds[];   // [NSPLIT][2][KT][VPITCH]; reused for the merge

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int G = a.n_heads / a.n_kv_heads;
    const int nthreads = G * 64;                                // threads of one key split
    const int sp = w / G, wg = w - sp * G;                      // key split, head within the GQA group
    const int stid = tid - sp * nthreads;                       // thread index inside the split
    const int n16 = lane & 15, kg = lane >> 4;
    const uint32_t kvh = blockIdx.y;
    const uint32_t q0 = blockIdx.x * 16;
    const uint32_t h = kvh * G + wg;
    const uint32_t qi = q0 + n16;                              // this lane's query (column of S^T)
    const bool q_ok = qi < a.m;
    const uint32_t row_stride = a.n_kv_heads * D * ES;         // bytes between positions

    // ---- Q^T as B operands: lane (query n16, group kg) holds q[kg*SEG + c*8 + j], j < 8, per k-step c
    half8_t qhi[KS], qlo[KS];
    bool any_lo = false;
    {
        const float* qp = a.q + ((size_t)(q_ok ? qi : 0) * a.n_heads + h) * D + kg * SEG;
#pragma unroll
        for (int c = 0; c < KS; ++c) {
#pragma unroll
            for (int j4 = 0; j4 < 2; ++j4) {
                float4 f = *reinterpret_cast<const float4*>(qp + c * 8 + j4 * 4);
                if (!q_ok) f = make_float4(0.f, 0.f, 0.f, 0.f);
                const float v[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const _Float16 hv = (_Float16)v[j];
                    const _Float16 lv = (_Float16)(v[j] - (float)hv);
                    qhi[c][j4 * 4 + j] = hv;
                    qlo[c][j4 * 4 + j] = lv;
                    any_lo |= lv != (_Float16)0;
                }
            }
        }
    }
    const bool has_lo = __builtin_amdgcn_ballot_w64(any_lo) != 0ull;     // wavefront-uniform

    // ---- key range of this workgroup ----
    uint32_t kmax = a.q_start + q0 + 16;                        // one past the last key any of the 16 queries sees
    if (kmax > a.n_kv) kmax = a.n_kv;
    const uint32_t my_len = q_ok ? (a.q_start + qi + 1 < a.n_kv ? a.q_start + qi + 1 : a.n_kv) : 0;   // causal_len of this lane's query
    const uint32_t t_first = (a.kv_start / KT) * KT;
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;

    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.n_kv * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.n_kv * row_stride, 0x00020000);
    const uint32_t head_b = kvh * D * ES;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * SEGB;   // key row (tile row n16), this group's quarter

    // V staging: the tile is KT rows of D*ES bytes = KT*D*ES/16 chunks of 16 bytes, spread over the workgroup
    constexpr int VCHUNK_ROW = D * ES / 16;                     // chunks per key row
    constexpr int VCHUNKS = KT * VCHUNK_ROW;
    constexpr int VMAX = (VCHUNKS + 63) / 64;                   // chunks per thread when G == 1 (fewer for larger G)
    constexpr uint32_t kNoTile = 0x80000000u;                   // byte offset past any slab: the load returns zeros, no memory access
    u32x4 vstage[PFD][VMAX];                                    // PFD tiles in flight per split
    auto v_issue = [&](int slot, uint32_t toff) {               // toff: byte offset of the tile's first row (or kNoTile)
#pragma unroll
        for (int c = 0; c < VMAX; ++c) {
            const int chunk = stid + c * nthreads;
            if (chunk < VCHUNKS) {
                const int row = chunk / VCHUNK_ROW, col = chunk % VCHUNK_ROW;
                vstage[slot][c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, row * row_stride + head_b + col * 16, toff, 0);
            }
        }
    };
    auto v_commit = [&](int buf, int slot) {                    // widen to f16 and store row-major
        _Float16* base = vlds + (size_t)(sp * 2 + buf) * KT * VPITCH;
#pragma unroll
        for (int c = 0; c < VMAX; ++c) {
            const int chunk = stid + c * nthreads;
            if (chunk < VCHUNKS) {
                const int row = chunk / VCHUNK_ROW, col = chunk % VCHUNK_ROW;
                if (DT == kF8) {
                    uint32_t out[8];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const uint32_t wd = vstage[slot][c][x];
                        half2_t lo2, hi2;
                        e4m3x4_to_h2(wd, lo2, hi2);
                        out[2 * x] = __builtin_bit_cast(uint32_t, lo2);
                        out[2 * x + 1] = __builtin_bit_cast(uint32_t, hi2);
                    }
                    u32x4* dst = reinterpret_cast<u32x4*>(base + row * VPITCH + col * 16);
                    dst[0] = u32x4{out[0], out[1], out[2], out[3]};
                    dst[1] = u32x4{out[4], out[5], out[6], out[7]};
                } else {
                    *reinterpret_cast<u32x4*>(base + row * VPITCH + col * 8) = vstage[slot][c];
                }
            }
        }
    };

    // K operands of one tile: [half of the tile][16-byte piece of this lane's quarter row]
    u32x4 kraw[PFD][2][KLD];
    auto k_issue = [&](int slot, uint32_t toff) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int x = 0; x < KLD; ++x)
                kraw[slot][kt][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * 16, toff + (uint32_t)(kt * 16) * row_stride, 0);
    };
    auto k_operand = [&](int slot, int kt, int c) -> half8_t {            // 8 consecutive d of this lane's quarter, k-step c
        half8_t r;
        if (DT == kF8) {
            const uint32_t w0 = kraw[slot][kt][c / 2][(c % 2) * 2], w1 = kraw[slot][kt][c / 2][(c % 2) * 2 + 1];
            half2_t p0, p1, p2, p3;
            e4m3x4_to_h2(w0, p0, p1);
            e4m3x4_to_h2(w1, p2, p3);
            r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1]; r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
        } else {
            const u32x4 wv = kraw[slot][kt][c];
            r = __builtin_bit_cast(half8_t, wv);
        }
        return r;
    };

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;

    if (t_first < kmax) {
        const uint32_t step = KT * NSPLIT;
        uint32_t tb = t_first + sp * KT;                        // this split's first tile (may already be past the end)
        auto tile_off = [&](uint32_t t) -> uint32_t { return t < kmax ? t * row_stride : kNoTile; };
#pragma unroll
        for (int sl = 0; sl < PFD; ++sl) { v_issue(sl, tile_off(tb + sl * step)); k_issue(sl, tile_off(tb + sl * step)); }
        int buf = 0;
        for (uint32_t round = t_first; round < kmax; round += PFD * step, tb += PFD * step) {
#pragma unroll
          for (int sl = 0; sl < PFD; ++sl) {
            if (round + sl * step >= kmax) break;               // workgroup-uniform
            const uint32_t tcur = tb + sl * step;
            const bool live = tcur < kmax;                      // wavefront-uniform; every wavefront still meets the barrier
            if (live) v_commit(buf, sl);
            __syncthreads();                                    // V tiles visible; the other buffers are free again
            const int cbuf = buf;
            buf ^= 1;
            if (!live) continue;
            // operands of this tile, then request the tile PFD steps ahead into the freed registers
            half8_t ka[2][KS];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int c = 0; c < KS; ++c) ka[kt][c] = k_operand(sl, kt, c);
            { const uint32_t noff = tile_off(tcur + PFD * step); v_issue(sl, noff); k_issue(sl, noff); }
            const uint32_t tbk = tcur;                          // first key of this tile

            float4_t s[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int c = 0; c < KS; ++c) s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[kt][c], qhi[c], s[kt], 0, 0, 0);
            if (has_lo) {
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int c = 0; c < KS; ++c) s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[kt][c], qlo[c], s[kt], 0, 0, 0);
            }
            // ---- online softmax: this lane owns keys tb + kt*16 + kg*4 + i of query n16 ----
            float x[8];
            float tmax = kMasked;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t t = tbk + kt * 16 + kg * 4 + i;
                    float y = s[kt][i] * scale_l2;
                    if (CAP) y = cap_l2 * tanhf(y / cap_l2);
                    y = (t < my_len && t >= a.kv_start) ? y : kMasked;
                    x[kt * 4 + i] = y;
                    tmax = fmaxf(tmax, y);
                }
            { float y = tmax; swap16(tmax, y); tmax = fmaxf(tmax, y); y = tmax; swap32(tmax, y); tmax = fmaxf(tmax, y); }
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = exp2f(m_run - m_new);
            m_run = m_new;
            half8_t pb, pl;
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float p = x[j] > -1e29f ? exp2f(x[j] - m_new) : 0.f;
                const _Float16 ph = (_Float16)p;
                pb[j] = ph;
                pl[j] = (_Float16)(p - (float)ph);
                psum += p;
            }
            l_run = l_run * alpha + psum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0ull) {
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) oacc[dt] *= alpha;
            }
            // ---- O^T += V^T P^T ----
            const _Float16* vb = vlds + (size_t)(sp * 2 + cbuf) * KT * VPITCH;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                // supplier lane s of a 16-lane group points at V[key = 4*kg + s/4 (+16)][d = dt*16 + 4*(s%4)]
                const _Float16* p0 = vb + (kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                const half4_t v0 = lds_read_tr16(p0);
                const half4_t v1 = lds_read_tr16(p0 + 16 * VPITCH);
                half8_t va;
                va[0] = v0[0]; va[1] = v0[1]; va[2] = v0[2]; va[3] = v0[3]; va[4] = v1[0]; va[5] = v1[1]; va[6] = v1[2]; va[7] = v1[3];
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb, oacc[dt], 0, 0, 0);
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pl, oacc[dt], 0, 0, 0);
            }
          }
        }
    }
    l_run = xor32_sum(xor16_sum(l_run));                        // every lane of a query column now has its split's sum
    // ---- merge the key splits through LDS (split 0 collects) ----
    if (NSPLIT > 1) {
        __syncthreads();                                        // all V tiles consumed: the LDS is free
        float* mbuf = reinterpret_cast<float*>(vlds);           // [NSPLIT-1][G][64][DTILES*4 + 2]
        constexpr int REC = DTILES * 4 + 2;
        if (sp > 0) {
            float* rec = mbuf + ((size_t)((sp - 1) * G + wg) * 64 + lane) * REC;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) rec[dt * 4 + i] = oacc[dt][i];
            rec[DTILES * 4] = m_run;
            rec[DTILES * 4 + 1] = l_run;
        }
        __syncthreads();
        if (sp > 0) return;
#pragma unroll 1
        for (int s2 = 1; s2 < NSPLIT; ++s2) {
            const float* rec = mbuf + ((size_t)((s2 - 1) * G + wg) * 64 + lane) * REC;
            const float m2 = rec[DTILES * 4], l2 = rec[DTILES * 4 + 1];
            const float mm = fmaxf(m_run, m2);
            const float f1 = exp2f(m_run - mm), f2 = exp2f(m2 - mm);
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) oacc[dt][i] = oacc[dt][i] * f1 + rec[dt * 4 + i] * f2;
            l_run = l_run * f1 + l2 * f2;
            m_run = mm;
        }
    }
    // ---- normalise and store: lane (query n16) holds d = dt*16 + kg*4 + i ----
    if (q_ok) {
        const float inv = 1.0f / l_run;
        float* op = a.o + ((size_t)qi * a.n_heads + h) * D + kg * 4;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
            const float4_t r = oacc[dt] * inv;
            *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
        }
    }
}

}  // namespace vfkv
