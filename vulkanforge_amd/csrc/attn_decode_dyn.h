// Matrix-core worker of the split-K decode attention (flash_attn_split.comp:82-162) with a late-rebalanced deal of the
// rows; included by attn_decode.hip.  Arithmetic, operand layouts and the workgroup merge are those of split_mfma_kernel
// (attn_decode_mfma.h); what differs is which rows a wavefront walks.
//
// The visible rows are cut into runs of RUN rows.  The wavefronts of a KV head (run streams: NW per workgroup, n_tiles
// workgroups) take the LAST runs of the span statically, `static_rounds` runs each, interleaved (run n_runs - 1 - (j * S + s)
// is the j-th run of stream s: the ragged last run and a freshly appended row are somebody's first run, handled while
// everything still waits for memory).  The remaining front of the span is handed out in arrival order through one
// counter per (KV head, head slice): a wavefront that finishes early draws more units than one that runs late, so the
// launch no longer waits for the slowest of its statically dealt streams.  A draw is issued one unit ahead of its use
// (the atomic's round trip hides behind a unit's arithmetic) by a single lane of the wavefront (a buffer atomic whose
// other lanes are out of range).  Units of the dynamic part are RUN rows, or RUN / 2 when HU is set (finer grain at the
// end, where nothing is left to overlap a unit's arithmetic with).  Every wavefront draws until it receives the first
// ticket past the last unit, so a launch makes exactly n_units + S draws and the wavefront that receives the last one
// puts the counter back to zero for the next launch.
#pragma once
#include <type_traits>

namespace vfkv {

#ifdef VFKV_DECODE_STAMPS
#define VFKV_DSTAMP(i)                                                                                                       \
    do { if (a.stamps != nullptr && lane == 0)                                                                               \
        a.stamps[((((size_t)blockIdx.x * gridDim.y + blockIdx.y) * gridDim.z + blockIdx.z) * NW + w) * 4 + (i)] = wall_clock64(); } while (0)
#else
#define VFKV_DSTAMP(i) do { } while (0)
#endif

template <int DT, int D, int RUN, int NW, bool CAP, bool HU>
__global__ __launch_bounds__(NW * 64) void split_mfma_dyn_kernel(SplitArgs a, uint32_t gt) {
    constexpr int ES = DT == kF16 ? 2 : 1;
    constexpr int RT = RUN / 16;                 // 16-row tiles per run
    constexpr int PKS = RUN / 32;                // k-steps (32 rows) of the second product
    constexpr int KS = D / 32;                   // k-steps of the first product
    constexpr int DTILES = D / 16;
    constexpr int SEG = D / 4, SEGB = SEG * ES;  // a lane group's quarter of a K row
    constexpr int KLD = SEGB / 16;               // 16-byte loads per lane per K row
    constexpr bool KIL = SEGB >= 64;             // wide rows: the lane groups read consecutive 16-byte pieces
    constexpr int VPITCH = D + 16;               // halves per V row in LDS (+32 B against bank conflicts)
    constexpr int VCHUNK_ROW = D * ES / 16;      // 16-byte chunks per V row
    constexpr int VLD = RUN * VCHUNK_ROW / 64;   // V loads per lane per run
    constexpr int VROWS = 64 / VCHUNK_ROW;       // rows covered by one V load of the wavefront
    constexpr int UROWS = HU ? RUN / 2 : RUN;    // rows of a unit of the dynamic part
    static_assert(D % 32 == 0 && SEGB % 16 == 0 && RUN % 32 == 0 && VCHUNK_ROW <= 64 && VLD >= 2 && VLD % 2 == 0, "unsupported shape");
    static_assert(NW * RUN * VPITCH * 2 >= NW * (D / 16) * 64 * 16, "merge buffer must fit in the V staging area");
    static_assert(DTILES % NW == 0, "d-tiles must divide evenly among the wavefronts");

    __shared__ __attribute__((aligned(16))) _Float16 vlds[NW][RUN * VPITCH];
    __shared__ float lds_m[NW][8], lds_l[NW][8];
    __shared__ __attribute__((aligned(16))) _Float16 qlds[16][D + 8];   // rows 0-7: f16(q) per head, rows 8-15: remainders

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    VFKV_DSTAMP(0);                              // wavefront start
    const int n16 = lane & 15, kg = lane >> 4;
    const int col = n16 & 7;
    const bool is_lo = n16 >= 8;
    const uint32_t kvh = blockIdx.x, jl = blockIdx.y;
    const uint32_t g_all = a.group;
    const uint32_t hz = blockIdx.z * gt;
    const uint32_t gcount = g_all - hz < gt ? g_all - hz : gt;
    const uint32_t h0 = kvh * g_all + hz;
    const uint32_t tile_base = a.tile_first * a.tile;
    const uint32_t tile_end = a.seq_len;
    const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;

    const uint32_t row_stride = a.n_kv_heads * D * ES;
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.seq_len * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.seq_len * row_stride, 0x00020000);
    const uint32_t head_b = kvh * D * ES;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * (KIL ? 16 : SEGB);
    const int vrow = lane / VCHUNK_ROW, vcol = lane % VCHUNK_ROW;
    const uint32_t lane_voff = vrow * row_stride + head_b + vcol * 16;
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;

    // ---- the deal ----
    const uint32_t first_run = (lo - tile_base) / RUN;
    const uint32_t n_runs = tile_end > tile_base ? (tile_end - tile_base + RUN - 1) / RUN : 0;
    const uint32_t nv = n_runs > first_run ? n_runs - first_run : 0u;          // runs that reach the window
    const uint32_t S = NW * a.n_tiles, sidx = jl * NW + (uint32_t)w;            // run streams of the KV head, this one
    const uint32_t ns_cap = a.static_rounds * S;
    const uint32_t ns_tot = nv < ns_cap ? nv : ns_cap;                          // runs dealt statically, from the end
    const uint32_t n_units = (nv - ns_tot) * (HU ? 2u : 1u);                    // units handed out by the counter
    const uint32_t dyn_base = tile_base + first_run * RUN;                      // first row of the dynamic part
    constexpr uint32_t kNone = 0xFFFFFFFFu;
    // a unit is (first row, tiles of 16 rows); both wavefront-uniform
    auto static_rb = [&](uint32_t j) -> uint32_t {
        const uint32_t e = j * S + sidx;
        return e < ns_tot ? tile_base + (n_runs - 1u - e) * RUN : kNone;
    };
    auto unit_off = [&](uint32_t rb) -> uint32_t { return rb != kNone ? rb * row_stride : kOOB; };

    uint32_t kfront = 0;                           // units of the front part this stream has taken
    auto front_rb = [&]() -> uint32_t {            // the stream's next unit of the front part (units dealt round-robin)
        const uint32_t u = kfront * S + sidx;
        ++kfront;
        return u < n_units ? dyn_base + u * UROWS : kNone;
    };

    u32x4 kraw[RT][KLD];
    u32x4 vraw[VLD];
    auto issue_k = [&](int t, uint32_t off) {
#pragma unroll
        for (int x = 0; x < KLD; ++x)
            kraw[t][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * (KIL ? 64 : 16), off + (uint32_t)(t * 16) * row_stride, 0);
    };
    auto issue_v = [&](int c, uint32_t off) {
        vraw[c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, off + (uint32_t)(c * VROWS) * row_stride, 0);
    };

    // ---- optional fused append (step_kv_write, executor/attention.rs:546): the workgroup whose first static run holds the
    // new position converts and stores this KV head's slice of the new K and V rows before anything reads them (the
    // launcher only passes rows that lie in the statically dealt part).
    if (a.k_new != nullptr) {
        const uint32_t e_app = n_runs - 1u - (a.append_pos - tile_base) / RUN;
        if ((e_app % S) / NW == jl) {
            constexpr int EPW = 4 / ES;
            if (tid < D / EPW) {
                const size_t src = (size_t)kvh * D + (size_t)tid * EPW;
                const size_t dst = ((size_t)a.append_pos * a.n_kv_heads + kvh) * D * ES + (size_t)tid * 4;
                uint32_t kw, vw;
                if (DT == kF8) {
                    const float4 kf = *reinterpret_cast<const float4*>(a.k_new + src);
                    const float4 vf = *reinterpret_cast<const float4*>(a.v_new + src);
                    kw = pack4_e4m3(kf.x, kf.y, kf.z, kf.w);
                    vw = pack4_e4m3(vf.x, vf.y, vf.z, vf.w);
                } else {
                    const float2 kf = *reinterpret_cast<const float2*>(a.k_new + src);
                    const float2 vf = *reinterpret_cast<const float2*>(a.v_new + src);
                    kw = f32_to_h16_bits(kf.x) | (f32_to_h16_bits(kf.y) << 16);
                    vw = f32_to_h16_bits(vf.x) | (f32_to_h16_bits(vf.y) << 16);
                }
                *reinterpret_cast<uint32_t*>(const_cast<uint8_t*>(a.k) + dst) = kw;
                *reinterpret_cast<uint32_t*>(const_cast<uint8_t*>(a.v) + dst) = vw;
            }
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
    }

    uint32_t cur_rb = static_rb(0);
    const bool active = cur_rb != kNone;
    uint32_t cur_tiles = RT;
    uint32_t jnext = 1;                               // next run of this stream in the part dealt from the end
    {
        const uint32_t off0 = unit_off(cur_rb);
#pragma unroll
        for (int t = 0; t < RT; ++t) issue_k(t, off0);
    }

    // ---- Q^T operands (as in split_mfma_kernel) ----
    constexpr int QLD = (8 * D / 4 + NW * 64 - 1) / (NW * 64);
    const int nq4 = (int)gcount * D / 4;
    float4 qf[QLD];
#pragma unroll
    for (int i = 0; i < QLD; ++i) {
        const int idx = tid + i * NW * 64;
        qf[i] = *reinterpret_cast<const float4*>(a.q + (size_t)h0 * D + (idx < nq4 ? idx : 0) * 4);
    }
    {
        const uint32_t off0 = unit_off(cur_rb);
#pragma unroll
        for (int c = 0; c < VLD; ++c) issue_v(c, off0);
    }
    {
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * NW * 64;
            if (idx >= nq4) continue;
            const float4 f = qf[i];
            const int g = (idx * 4) / D, d = (idx * 4) % D;
            const float v4[4] = {f.x, f.y, f.z, f.w};
            _Float16 hv[4], lv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) { hv[j] = (_Float16)v4[j]; lv[j] = (_Float16)(v4[j] - (float)hv[j]); }
            *reinterpret_cast<half4_t*>(&qlds[g][d]) = half4_t{hv[0], hv[1], hv[2], hv[3]};
            *reinterpret_cast<half4_t*>(&qlds[8 + g][d]) = half4_t{lv[0], lv[1], lv[2], lv[3]};
        }
    }
    __syncthreads();
    half8_t qb[KS];
    {
        const bool col_ok = (uint32_t)col < gcount;
#pragma unroll
        for (int c = 0; c < KS; ++c) {
            const int qe = !KIL ? kg * SEG + c * 8 : ES == 2 ? (c * 4 + kg) * 8 : ((c / 2) * 4 + kg) * 16 + (c % 2) * 8;
            const u32x4 raw = *reinterpret_cast<const u32x4*>(&qlds[col_ok ? n16 : 0][qe]);
            qb[c] = __builtin_bit_cast(half8_t, col_ok ? raw : u32x4{0u, 0u, 0u, 0u});
        }
    }

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;
    _Float16* const vb = &vlds[w][0];
    VFKV_DSTAMP(1);                              // queries staged, first run requested

    // One unit: NT tiles of 16 rows from row rb on (NT = RT, or RT / 2 for a half unit).  The K / V registers it consumes are
    // refilled at once with the rows of the next unit (ntiles tiles from byte offset noff; none past that: those loads are
    // out of range and return zeros without traffic).
    auto process = [&](auto nt_tag, uint32_t rb, uint32_t noff, uint32_t ntiles) {
        constexpr int NT = decltype(nt_tag)::value;
        constexpr int NVL = VLD * NT / RT;                   // V loads that hold this unit's rows
        constexpr int NPK = (NT * 16 + 31) / 32;             // k-steps of 32 rows (the last one half empty when NT is odd)
        float4_t s[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            half8_t ka[KS];
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                if (DT == kF8) {
                    const uint32_t w0 = kraw[t][c / 2][(c % 2) * 2], w1 = kraw[t][c / 2][(c % 2) * 2 + 1];
                    half2_t p0, p1, p2, p3;
                    e4m3x4_to_h2(w0, p0, p1);
                    e4m3x4_to_h2(w1, p2, p3);
                    ka[c][0] = p0[0]; ka[c][1] = p0[1]; ka[c][2] = p1[0]; ka[c][3] = p1[1];
                    ka[c][4] = p2[0]; ka[c][5] = p2[1]; ka[c][6] = p3[0]; ka[c][7] = p3[1];
                } else {
                    const u32x4 wv = kraw[t][c % KLD];
                    ka[c] = __builtin_bit_cast(half8_t, wv);
                }
            }
            issue_k(t, (uint32_t)t < ntiles ? noff : kOOB);
            s[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KS; ++c) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], qb[c], s[t], 0, 0, 0);
        }
        const bool interior = rb >= lo && rb + NT * 16 <= tile_end;      // wavefront-uniform
        uint32_t pbits[NPK][4];
#pragma unroll
        for (int ks = 0; ks < NPK; ++ks)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) pbits[ks][r4] = 0u;
        auto softmax = [&](auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            constexpr bool FOLD = !MASKED && !CAP;
            float x[NT][4];
            float tmax = kMasked;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = s[t][i];
                    y += dpp_f<kDppRor8>(y);
                    if (!FOLD) y *= scale_l2;
                    if (CAP) y = cap_l2 * tanhf(y / cap_l2);
                    if (MASKED) {
                        const uint32_t row = rb + t * 16 + kg * 4 + i;
                        y = (row >= lo && row < tile_end) ? y : kMasked;
                    }
                    x[t][i] = y;
                    tmax = fmaxf(tmax, y);
                }
            { float y = tmax; swap16(tmax, y); tmax = fmaxf(tmax, y); y = tmax; swap32(tmax, y); tmax = fmaxf(tmax, y); }
            if (FOLD) tmax *= scale_l2;
            const float m_new = fmaxf(m_run, tmax);
            if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0ull) {
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) oacc[dt] *= alpha;
                m_run = m_new;
            }
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i2 = 0; i2 < 2; ++i2) {
                    float2_t pp;
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const float xe = x[t][2 * i2 + e];
                        float pv = __builtin_amdgcn_exp2f(FOLD ? __builtin_fmaf(xe, scale_l2, -m_run) : xe - m_run);
                        if (MASKED) pv = xe > -1e29f ? pv : 0.f;
                        pp[e] = pv;
                    }
                    l_run += pp[0] + pp[1];
                    const uint32_t ph = __builtin_bit_cast(uint32_t, __builtin_convertvector(pp, half2_t));
                    const uint32_t pl = pack_f16_remainder(pp[0], pp[1], ph);
                    pbits[t / 2][(t % 2) * 2 + i2] = is_lo ? pl : ph;
                }
        };
        if (interior) softmax(std::false_type{}); else softmax(std::true_type{});
        // ---------------- V rows -> f16 row-major in LDS ----------------
#pragma unroll
        for (int c = 0; c < NVL; ++c) {
            _Float16* dst = vb + (c * VROWS + vrow) * VPITCH + vcol * (16 / ES);
            if (DT == kF8) {
                uint32_t out[8];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const uint32_t wd = vraw[c][q4];
                    half2_t lo2, hi2;
                    e4m3x4_to_h2(wd, lo2, hi2);
                    out[2 * q4] = __builtin_bit_cast(uint32_t, lo2);
                    out[2 * q4 + 1] = __builtin_bit_cast(uint32_t, hi2);
                }
                reinterpret_cast<u32x4*>(dst)[0] = u32x4{out[0], out[1], out[2], out[3]};
                reinterpret_cast<u32x4*>(dst)[1] = u32x4{out[4], out[5], out[6], out[7]};
            } else {
                *reinterpret_cast<u32x4*>(dst) = vraw[c];
            }
            issue_v(c, (uint32_t)(c * VROWS) < ntiles * 16u ? noff : kOOB);
        }
        if (NVL < VLD) {                   // a half unit leaves the other registers alone unless the next unit needs them
#pragma unroll
            for (int c = NVL; c < VLD; ++c) if ((uint32_t)(c * VROWS) < ntiles * 16u) issue_v(c, noff);
        }
        if (NT < RT) {
#pragma unroll
            for (int t = NT; t < RT; ++t) if ((uint32_t)t < ntiles) issue_k(t, noff);
        }
        // ---------------- O^T += V^T P ----------------
#pragma unroll
        for (int ks = 0; ks < NPK; ++ks)
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const _Float16* p0 = vb + (ks * 32 + kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                const half4_t v0 = lds_read_tr16(p0);
                if (NT * 16 >= ks * 32 + 32) {
                    const half4_t v1 = lds_read_tr16(p0 + 16 * VPITCH);
                    half8_t va;
                    va[0] = v0[0]; va[1] = v0[1]; va[2] = v0[2]; va[3] = v0[3]; va[4] = v1[0]; va[5] = v1[1]; va[6] = v1[2]; va[7] = v1[3];
                    const u32x4 pw = u32x4{pbits[ks][0], pbits[ks][1], pbits[ks][2], pbits[ks][3]};
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, pw), oacc[dt], 0, 0, 0);
                } else {                   // 16 rows: the 16-deep product on the lower half of the weights
                    const u32x2 pw = u32x2{pbits[ks][0], pbits[ks][1]};
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x16f16(v0, __builtin_bit_cast(half4_t, pw), oacc[dt], 0, 0, 0);
                }
            }
    };

    if (active) {
        for (;;) {
            // the unit after this one: the stream's next run of the part dealt from the end, then its units of the front part
            uint32_t nxt_rb = static_rb(jnext), nxt_tiles = RT;
            if (nxt_rb != kNone) {
                ++jnext;
            } else {
                nxt_rb = front_rb();
                nxt_tiles = UROWS / 16;
            }
            const uint32_t noff = unit_off(nxt_rb);
            if (!HU || cur_tiles == (uint32_t)RT) process(std::integral_constant<int, RT>{}, cur_rb, noff, nxt_tiles);
            else process(std::integral_constant<int, RT / 2>{}, cur_rb, noff, nxt_tiles);
            if (nxt_rb == kNone) break;
            cur_rb = nxt_rb; cur_tiles = nxt_tiles;
        }
    }

    VFKV_DSTAMP(2);                              // last unit done
    // ---------------- wavefront totals, then the workgroup merge through LDS (as in split_mfma_kernel) ----------------
    l_run = xor32_sum(xor16_sum(l_run));
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) { const float y = oacc[dt][i]; oacc[dt][i] = y + dpp_f<kDppRor8>(y); }
    __syncthreads();
    float4_t* const slot = reinterpret_cast<float4_t*>(&vlds[0][0]);     // [NW][DTILES][64 lanes]
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) slot[(w * DTILES + dt) * 64 + lane] = oacc[dt];
    if (kg == 0 && !is_lo) { lds_m[w][col] = m_run; lds_l[w][col] = l_run; }
    __syncthreads();
    constexpr int MT = DTILES / NW;
    float mw[NW], lw[NW];
    float4_t part[MT][NW];
#pragma unroll
    for (int pp = 0; pp < NW; ++pp) { mw[pp] = lds_m[pp][col]; lw[pp] = lds_l[pp][col]; }
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
    const bool writer = !is_lo && (uint32_t)col < gcount;
    const size_t pidx = (size_t)(h0 + col) * a.n_tiles + jl;
    float* const obase = a.so + pidx * D;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        float4_t o = fw[0] * part[t][0];
#pragma unroll
        for (int pp = 1; pp < NW; ++pp) o += fw[pp] * part[t][pp];
        if (writer) *reinterpret_cast<float4_t*>(obase + (t * NW + w) * 16 + kg * 4) = o;
    }
    if (writer && w == 0 && kg == 0) {
        a.sm[pidx] = M > -1e29f ? M * 0.693147180559945f : kMasked;
        a.ss[pidx] = l;
    }
#ifdef VFKV_DECODE_STAMPS
    __builtin_amdgcn_s_waitcnt(0);
#endif
    VFKV_DSTAMP(3);                              // partial stored and acknowledged
}
#undef VFKV_DSTAMP

}  // namespace vfkv
