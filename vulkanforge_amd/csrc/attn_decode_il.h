// Matrix-core worker of the split-K decode attention (flash_attn_split.comp:82-162) for launches whose partials only the
// merge reads (vfkv_decode_attention and its relatives, vfkv_flash_attn_split_interleaved); included by attn_decode.hip.
// Arithmetic and operand layouts are those of split_mfma_kernel (attn_decode_mfma.h: S^T = K Q^T and O^T += V^T P on
// v_mfma_f32_16x16x32_f16, queries and softmax weights as f16 value + remainder column pairs, K rows straight from global
// memory, V through an f16 copy in LDS and transposing LDS reads, workgroup merge through LDS).  What differs:
//
//   * The deal.  The visible rows are cut into runs of RUN rows and dealt to the run streams of the KV head (NW wavefronts
//     in each of n_tiles workgroups) from the END of the span: run n - 1 - (j S + s) is the j-th unit of stream s.  The
//     last, ragged run is therefore somebody's FIRST unit, and when it holds at most 16 rows it is not a unit of its own:
//     it rides along with the run in front of it as one unit of RUN + 16 rows (one memory round trip, 1.5 x the
//     arithmetic) instead of costing one stream a whole extra round that the launch then waits for (8 193 keys, 128
//     streams: 2 rounds and one row).
//   * Runs of one tile.  RUN = 16 is the same worker with units of a single 16-row tile: the second product is then the
//     16-deep matrix instruction (v_mfma_f32_16x16x16_f16) on the tile's own weights.  The launcher takes it where it measures
//     faster: rows of 512 bytes (32 rows of K and V would be 32 KiB in flight per wavefront, twice what the memory system
//     rewards) and launches whose run streams hold a run or two, where a smaller unit shortens the latency chain.
//   * The append of the decode token (step_kv_write, executor/attention.rs:546).  The new row is the last row of the span,
//     i.e. part of stream 0's first unit.  That wavefront converts the new K / V row itself, puts the converted K values
//     into the first product's operand and the converted V values over the row's place in its staged copy of the unit
//     (whatever the loads found at that row), and stores the same bytes to the cache.  Nothing waits for the stores: no
//     other wavefront of the launch reads that row.
//   * ROPE: the decode token's Q-norm / RoPE, K-norm / RoPE (step_q_norm_rope, step_k_norm_rope,
//     executor/attention.rs:360-530) in the same launch.  Every workgroup normalises and rotates its (up to 8) query
//     heads while its first K rows are in flight (the cos / sin table of the position is computed once per workgroup);
//     workgroup 0 of the KV head does the same for the new K row before it converts it.  Same arithmetic as
//     rope_append_kernel (rope_device.h): the cache bytes are identical to those of the separate launch.
#pragma once
#include <type_traits>

#include "rope_device.h"

namespace vfkv {

// What the ROPE form needs beyond SplitArgs (whose q / k_new are then the rows BEFORE norm and rotation).
struct RopeFoldArgs {
    const float* q_weight;       // [D] or NULL: no RMS-norm of the queries
    const float* k_weight;       // [D] or NULL
    const float* freq_factors;   // [rotary_dim / 2] or NULL
    float* q_out;                // [n_heads][D]: the rotated queries (must not overlap q), or NULL
    float* k_out;                // [n_kv_heads][D]: the rotated K row as f32, or NULL
    uint32_t rotary_dim, mode;
    float theta_scale, freq_scale, attn_factor, eps;
};

template <int DT, int D, int RUN, int NW, bool CAP, bool ROPE>
__device__ __forceinline__ void split_mfma_il_body(const SplitArgs& a, uint32_t gt, const RopeFoldArgs* rf) {
    constexpr int ES = DT == kF16 ? 2 : 1;
    constexpr int RT = RUN / 16;                 // 16-row tiles per run
    constexpr bool HALF = RUN == 16;             // runs of one tile: the second product is the 16-deep matrix instruction
    constexpr int KLD0 = (D / 4) * ES / 16, VLT0 = 16 / (64 / (D * ES / 16));
    constexpr bool LONG = RUN % 32 == 0 && (RT + 1) * (KLD0 + VLT0) <= 24;   // the long first unit costs KLD + VLT more 16-byte registers: not where rows are 512 bytes wide
    constexpr int XT = LONG ? RT + 1 : RT;       // tiles of the first unit of stream 0 at most
    constexpr int KS = D / 32;                   // k-steps of the first product
    constexpr int DTILES = D / 16;
    constexpr int SEG = D / 4, SEGB = SEG * ES;  // a lane group's quarter of a K row
    constexpr int KLD = SEGB / 16;               // 16-byte loads per lane per K row
    constexpr bool KIL = SEGB >= 64;             // wide rows: the lane groups read consecutive 16-byte pieces
    constexpr int VPITCH = D + 16;               // halves per V row in LDS (+32 B against bank conflicts)
    constexpr int VCHUNK_ROW = D * ES / 16;      // 16-byte chunks per V row
    constexpr int VROWS = 64 / VCHUNK_ROW;       // rows covered by one V load of the wavefront
    constexpr int VLT = 16 / VROWS;              // V loads per lane per tile of 16 rows
    constexpr int MAXJ = (D + 63) / 64;          // elements of a row per lane in the norm / RoPE stage
    static_assert(D % 32 == 0 && SEGB % 16 == 0 && (RUN % 32 == 0 || HALF) && VCHUNK_ROW >= 4 && VCHUNK_ROW <= 64, "unsupported shape");
    static_assert(!(HALF && LONG), "the long first unit needs runs of whole k-steps");
    static_assert(NW * (RUN + 16) * VPITCH * 2 >= NW * (D / 16) * 64 * 16, "merge buffer must fit in the V staging area");
    static_assert(DTILES % NW == 0, "d-tiles must divide evenly among the wavefronts");

    __shared__ __attribute__((aligned(16))) _Float16 vlds[NW][(RUN + 16) * VPITCH];
    __shared__ float lds_m[NW][8], lds_l[NW][8];
    __shared__ __attribute__((aligned(16))) _Float16 qlds[16][D + 8];   // rows 0-7: f16(q) per head, rows 8-15: remainders
    __shared__ __attribute__((aligned(16))) float rot[ROPE ? 9 : 1][ROPE ? D : 4];   // ROPE: rotated query heads, then the K row
    __shared__ float cs_lds[ROPE ? D / 2 : 1], sn_lds[ROPE ? D / 2 : 1];
    __shared__ __attribute__((aligned(16))) uint8_t newrow[D * ES];      // the decode token's K row in the cache's format (stream 0's wavefront)

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
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
    const float inv_cap_l2 = CAP ? 1.0f / cap_l2 : 0.f;

    // ---- the deal: units counted from the end of the span ----
    const uint32_t span = tile_end > tile_base ? tile_end - tile_base : 0u;
    const uint32_t n_runs = (span + RUN - 1) / RUN;
    const uint32_t first_run = (lo - tile_base) / RUN;
    const uint32_t r_tail = span % RUN;                                         // rows of a ragged last run (0: none)
    // (the launcher sets bit 1 of a.interleave when that saves a round: when the units then divide evenly among the streams)
    const bool long_first = LONG && (a.interleave & 2u) != 0u && r_tail != 0u && r_tail <= 16u && n_runs >= first_run + 2u;
    const uint32_t n_eff = n_runs - (long_first ? 1u : 0u);                     // units of the span
    const uint32_t nv = n_eff > first_run ? n_eff - first_run : 0u;            // units that reach the window
    const uint32_t S = NW * a.n_tiles, sidx = jl * NW + (uint32_t)w;            // run streams of the KV head, this one
    constexpr uint32_t kNone = 0xFFFFFFFFu;
    auto unit_rb = [&](uint32_t j) -> uint32_t {          // first row of this stream's j-th unit, or none
        const uint32_t e = j * S + sidx;
        return e < nv ? tile_base + (n_eff - 1u - e) * RUN : kNone;
    };
    auto unit_off = [&](uint32_t rb) -> uint32_t { return rb != kNone ? rb * row_stride : kOOB; };

    u32x4 kraw[XT][KLD];
    u32x4 vraw[XT * VLT];
    auto issue_k = [&](int t, uint32_t off) {
#pragma unroll
        for (int x = 0; x < KLD; ++x)
            kraw[t][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * (KIL ? 64 : 16), off + (uint32_t)(t * 16) * row_stride, 0);
    };
    auto issue_v = [&](int c, uint32_t off) {
        vraw[c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, off + (uint32_t)(c * VROWS) * row_stride, 0);
    };

    uint32_t cur_rb = unit_rb(0);
    const bool active = cur_rb != kNone;
    const bool first_long = long_first && sidx == 0u;       // wavefront-uniform: this stream's first unit is the long one
    {
        const uint32_t off0 = unit_off(cur_rb);
#pragma unroll
        for (int t = 0; t < RT; ++t) issue_k(t, off0);
        if (LONG && first_long) issue_k(XT - 1, off0);      // (a uniform branch: the other wavefronts never touch that tile's registers)
    }

    // ---- the new row of the decode token, in the wavefront that reads it (stream 0: the last row lies in its first unit).
    // Without ROPE its f32 values come straight from global memory: requested here (four elements per lane), converted after
    // the queries have arrived (loads return in order); the K row is parked in LDS in the cache's format and fetched from
    // there by the lanes whose K registers hold pieces of that row, the V row goes over the staged copy of its place.
    const bool appends = a.k_new != nullptr && active && sidx == 0u;            // wavefront-uniform
    const uint32_t rn = appends ? a.append_pos - cur_rb : 0u;                   // the row's index inside the unit
    const bool k_mine = appends && (uint32_t)n16 == (rn & 15u);                 // lanes whose K registers hold a piece of the row
    const bool row_lane = appends && lane * 4 < D;                              // lanes that convert four elements of the row
    float4 knew4 = make_float4(0.f, 0.f, 0.f, 0.f), vnew4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row_lane) {
        if (!ROPE) knew4 = *reinterpret_cast<const float4*>(a.k_new + (size_t)kvh * D + lane * 4);
        vnew4 = *reinterpret_cast<const float4*>(a.v_new + (size_t)kvh * D + lane * 4);
    }

    // ---- Q^T operands.  The workgroup converts its heads' queries once into f16 value / remainder planes in LDS; lane
    // (column n16, group kg) then holds its elements of every k-step.  ROPE: the rows are normalised and rotated first.
    constexpr int QLD = (8 * D / 4 + NW * 64 - 1) / (NW * 64);      // 16-byte query loads per thread (<= 8 heads)
    const int nq4 = (int)gcount * D / 4;
    float4 qf[QLD];
    float xr[3][MAXJ], wr[3][MAXJ];                                 // ROPE: rows w, w + NW, w + 2 NW of (query heads, K row)
    const bool k_row_here = ROPE && a.k_new != nullptr && jl == 0u;   // workgroup-uniform (every head slice reads the row, so every slice's workgroup 0 rotates it)
    const uint32_t n_rows = gcount + (k_row_here ? 1u : 0u);
    if (ROPE) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const uint32_t row = (uint32_t)w + i * NW;
            const bool is_k = row == gcount;
            const float* src = is_k ? a.k_new + (size_t)kvh * D : a.q + (size_t)(h0 + (row < gcount ? row : 0u)) * D;
            const float* wgt = is_k ? rf->k_weight : rf->q_weight;
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) {
                const uint32_t d = lane + j * kWave;
                xr[i][j] = (row < n_rows && d < (uint32_t)D) ? src[d] : 0.f;
                wr[i][j] = (row < n_rows && wgt != nullptr && d < (uint32_t)D) ? wgt[d] : 1.f;
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * NW * 64;
            qf[i] = *reinterpret_cast<const float4*>(a.q + (size_t)h0 * D + (idx < nq4 ? idx : 0) * 4);
        }
    }
    {
        const uint32_t off0 = unit_off(cur_rb);
#pragma unroll
        for (int c = 0; c < RT * VLT; ++c) issue_v(c, off0);
        if (LONG && first_long) {
#pragma unroll
            for (int c = RT * VLT; c < XT * VLT; ++c) issue_v(c, off0);
        }
    }
    if (ROPE) {
        const uint32_t half = rf->rotary_dim / 2u;
        rope_table(cs_lds, sn_lds, half, (float)a.append_pos, rf->theta_scale, rf->freq_scale, rf->attn_factor, rf->freq_factors,
                   (uint32_t)tid, NW * kWave);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const uint32_t row = (uint32_t)w + i * NW;
            if (row >= n_rows) continue;                           // wavefront-uniform
            const bool is_k = row == gcount;
            const float* wgt = is_k ? rf->k_weight : rf->q_weight;
            rope_row<MAXJ>(xr[i], wr[i], wgt != nullptr, rf->eps, D, half, rf->mode, true, cs_lds, sn_lds, rot[row], lane);
            float* out = is_k ? (rf->k_out ? rf->k_out + (size_t)kvh * D : nullptr)
                              : (rf->q_out && jl == 0u ? rf->q_out + (size_t)(h0 + row) * D : nullptr);
            if (out != nullptr)
                for (uint32_t d = lane; d < (uint32_t)D; d += kWave) out[d] = rot[row][d];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * NW * 64;
            const int ii = idx < nq4 ? idx : 0;
            qf[i] = *reinterpret_cast<const float4*>(&rot[(ii * 4) / D][(ii * 4) % D]);
        }
        if (row_lane) knew4 = *reinterpret_cast<const float4*>(&rot[gcount][lane * 4]);    // the rotated K row (this is workgroup 0)
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
            // first query element of k-step c in this lane group (16-byte pieces hold 8 halves or 16 FP8 values = two k-steps)
            const int qe = !KIL ? kg * SEG + c * 8 : ES == 2 ? (c * 4 + kg) * 8 : ((c / 2) * 4 + kg) * 16 + (c % 2) * 8;
            const u32x4 raw = *reinterpret_cast<const u32x4*>(&qlds[col_ok ? n16 : 0][qe]);
            qb[c] = __builtin_bit_cast(half8_t, col_ok ? raw : u32x4{0u, 0u, 0u, 0u});
        }
    }

    // ---- the new row in the cache's format: four elements per lane (kept for the store to the cache after the last unit:
    // stores count in the same in-order counter as the loads, so issued now, every later wait for rows would also wait for
    // their acknowledgement) and as a whole in LDS for the lanes that patch their registers inside the first unit.
    uint32_t kw0 = 0u, kw1 = 0u, vw0 = 0u, vw1 = 0u;
    const uint32_t tk = rn >> 4;                                // the tile that holds the row (wavefront-uniform)
    if (appends) {
        if (row_lane) {
            if (DT == kF8) {
                kw0 = pack4_e4m3(knew4.x, knew4.y, knew4.z, knew4.w);
                vw0 = pack4_e4m3(vnew4.x, vnew4.y, vnew4.z, vnew4.w);
                reinterpret_cast<uint32_t*>(&newrow[0])[lane] = kw0;
            } else {
                kw0 = f32_to_h16_bits(knew4.x) | (f32_to_h16_bits(knew4.y) << 16); kw1 = f32_to_h16_bits(knew4.z) | (f32_to_h16_bits(knew4.w) << 16);
                vw0 = f32_to_h16_bits(vnew4.x) | (f32_to_h16_bits(vnew4.y) << 16); vw1 = f32_to_h16_bits(vnew4.z) | (f32_to_h16_bits(vnew4.w) << 16);
                reinterpret_cast<u32x2*>(&newrow[0])[lane] = u32x2{kw0, kw1};
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");     // (the row is read back by lanes of this wavefront only)
    }
    // the pieces of the K row that this lane's K registers hold, fetched now: the LDS round trip runs while the unit's rows
    // are still on their way, and the patch inside the first unit is a select between registers
    u32x4 knw[KLD];
#pragma unroll
    for (int x = 0; x < KLD; ++x) knw[x] = u32x4{0u, 0u, 0u, 0u};
    if (appends) {
#pragma unroll
        for (int x = 0; x < KLD; ++x) knw[x] = *reinterpret_cast<const u32x4*>(&newrow[(KIL ? x * 4 + kg : kg * KLD + x) * 16]);
    }

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;
    _Float16* const vb = &vlds[w][0];

    // One unit: RUN rows from row rb on, plus 16 more when `extra` (the long first unit; wavefront-uniform).  The K / V registers
    // it consumes are refilled at once with the rows of the next unit (RUN rows from byte offset noff, or nothing: loads past
    // the end of the slab return zeros without traffic).  One body for both forms, so that the loop has a single shape.
    auto process = [&](uint32_t rb, uint32_t noff, bool extra, bool patch) {
        constexpr int PKS = RUN / 32;                        // k-steps of 32 rows of the second product
        float4_t s[XT];
        // k-step c of a row's pieces as the first product's A operand
        auto k_operand = [&](const u32x4 (&raw)[KLD], int c) -> half8_t {
            half8_t r;
            if (DT == kF8) {
                const uint32_t w0 = raw[c / 2][(c % 2) * 2], w1 = raw[c / 2][(c % 2) * 2 + 1];
                half2_t p0, p1, p2, p3;
                e4m3x4_to_h2(w0, p0, p1);
                e4m3x4_to_h2(w1, p2, p3);
                r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
                r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
            } else {
                r = __builtin_bit_cast(half8_t, raw[c % KLD]);
            }
            return r;
        };
        auto score_tile = [&](int t) {
            half8_t ka[KS];
#pragma unroll
            for (int c = 0; c < KS; ++c) ka[c] = k_operand(kraw[t], c);
            // The new row replaces what the loads found at its place, in the operand rather than in the registers the loads
            // fill: a branch that reads load destinations makes every later wait of the unit a full one.
            if (patch && (uint32_t)t == tk) {                // wavefront-uniform
#pragma unroll
                for (int c = 0; c < KS; ++c) {
                    const half8_t kn = k_operand(knw, c);
                    ka[c] = k_mine ? kn : ka[c];
                }
            }
            if (t < RT) issue_k(t, noff);
            s[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KS; ++c) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], qb[c], s[t], 0, 0, 0);
        };
#pragma unroll
        for (int t = 0; t < RT; ++t) score_tile(t);          // (one basic block: the widening of one tile overlaps the products of another)
        if (LONG) { s[XT - 1] = float4_t{0.f, 0.f, 0.f, 0.f}; if (extra) score_tile(XT - 1); }
        const bool interior = rb >= lo && rb + RUN <= tile_end && !extra;      // wavefront-uniform
        uint32_t pbits[PKS > 0 ? PKS : 1][4], pext[2] = {0u, 0u};
        auto softmax = [&](auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            constexpr bool FOLD = !MASKED && !CAP;                   // scores stay unscaled until the exponent
            constexpr int NTS = MASKED ? XT : RT;                    // the extra tile only exists in the masked form
            float x[NTS][4];
            float tmax = kMasked;
#pragma unroll
            for (int t = 0; t < NTS; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = s[t][i];
                    y += dpp_f<kDppRor8>(y);                         // f16(q) part + remainder part
                    if (!FOLD) y *= scale_l2;
                    if (CAP) y = softcap_l2(y, cap_l2, inv_cap_l2);
                    if (MASKED) {
                        const uint32_t row = rb + t * 16 + kg * 4 + i;
                        y = (row >= lo && row < tile_end && (t < RT || extra)) ? y : kMasked;
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
            // weights as f16 value (columns 0-7) or f16 remainder (columns 8-15), two rows per register
#pragma unroll
            for (int t = 0; t < NTS; ++t) {
                if (t >= RT && !extra) continue;
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
                    if (t < RT && !HALF) pbits[t / 2][(t % 2) * 2 + i2] = is_lo ? pl : ph;
                    else pext[i2] = is_lo ? pl : ph;
                }
            }
        };
        if (interior) softmax(std::false_type{}); else softmax(std::true_type{});
        // ---------------- V rows -> f16 row-major in LDS ----------------
        auto stage_v = [&](int c) {
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
            if (c < RT * VLT) issue_v(c, noff);
        };
#pragma unroll
        for (int c = 0; c < RT * VLT; ++c) stage_v(c);
        if (LONG && extra) {
#pragma unroll
            for (int c = RT * VLT; c < XT * VLT; ++c) stage_v(c);
        }
        if (patch && row_lane) {           // the new V row over the staged copy of its place (this wavefront's LDS accesses run in order)
            uint32_t h0w, h1w;
            if (DT == kF8) {
                half2_t lo2, hi2;
                e4m3x4_to_h2(vw0, lo2, hi2);
                h0w = __builtin_bit_cast(uint32_t, lo2); h1w = __builtin_bit_cast(uint32_t, hi2);
            } else {
                h0w = vw0; h1w = vw1;
            }
            *reinterpret_cast<u32x2*>(vb + rn * VPITCH + lane * 4) = u32x2{h0w, h1w};
        }
        // ---------------- O^T += V^T P ----------------
#pragma unroll
        for (int ks = 0; ks < PKS; ++ks)
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                // supplier lane s of a 16-lane group points at V[row = ks*32 + 4*kg + s/4 (+16)][d = dt*16 + 4*(s%4)]
                const _Float16* p0 = vb + (ks * 32 + kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                const half4_t v0 = lds_read_tr16(p0);
                const half4_t v1 = lds_read_tr16(p0 + 16 * VPITCH);
                half8_t va;
                va[0] = v0[0]; va[1] = v0[1]; va[2] = v0[2]; va[3] = v0[3]; va[4] = v1[0]; va[5] = v1[1]; va[6] = v1[2]; va[7] = v1[3];
                const u32x4 pw = u32x4{pbits[ks][0], pbits[ks][1], pbits[ks][2], pbits[ks][3]};
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, pw), oacc[dt], 0, 0, 0);
            }
        if (HALF || (LONG && extra)) {     // the 16 rows behind the run (or a run of 16 rows): the 16-deep product
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const _Float16* p0 = vb + ((HALF ? 0 : RUN) + kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                const half4_t v0 = lds_read_tr16(p0);
                const u32x2 pw = u32x2{pext[0], pext[1]};
                oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x16f16(v0, __builtin_bit_cast(half4_t, pw), oacc[dt], 0, 0, 0);
            }
        }
    };

    if (active) {
        uint32_t jnext = 1;
        bool extra = first_long, patch = appends;
        for (;;) {
            const uint32_t nxt_rb = unit_rb(jnext);
            ++jnext;
            process(cur_rb, unit_off(nxt_rb), extra, patch);
            if (nxt_rb == kNone) break;
            cur_rb = nxt_rb;
            extra = false; patch = false;
        }
    }
    if (row_lane) {                                    // the new row's bytes to the cache
        uint8_t* const krow = const_cast<uint8_t*>(a.k) + (size_t)a.append_pos * row_stride + head_b;
        uint8_t* const vrowp = const_cast<uint8_t*>(a.v) + (size_t)a.append_pos * row_stride + head_b;
        if (DT == kF8) {
            reinterpret_cast<uint32_t*>(krow)[lane] = kw0;
            reinterpret_cast<uint32_t*>(vrowp)[lane] = vw0;
        } else {
            reinterpret_cast<u32x2*>(krow)[lane] = u32x2{kw0, kw1};
            reinterpret_cast<u32x2*>(vrowp)[lane] = u32x2{vw0, vw1};
        }
    }

    // ---------------- wavefront totals, then the workgroup merge through LDS (as in split_mfma_kernel) ----------------
    l_run = xor32_sum(xor16_sum(l_run));
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) { const float y = oacc[dt][i]; oacc[dt][i] = y + dpp_f<kDppRor8>(y); }
    __syncthreads();                                   // every wavefront is done with its V staging area
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
    // a single workgroup per KV head covers every visible key (the reference's single-workgroup shader for seq <= 64,
    // forward/runs.rs:776-821): the merge is a plain normalisation, done here, and no merge launch follows
    const bool direct = a.o_direct != nullptr;
    const float inv_l = direct ? __builtin_amdgcn_rcpf(l) : 1.0f;
    float* const obase = direct ? a.o_direct + (size_t)(h0 + col) * D : a.so + pidx * D;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        float4_t o = fw[0] * part[t][0];
#pragma unroll
        for (int pp = 1; pp < NW; ++pp) o += fw[pp] * part[t][pp];
        if (direct) {                                  // one Newton step brings the reciprocal to f32 accuracy
            const float rcp = inv_l * (2.0f - l * inv_l);
            o *= rcp;
        }
        if (writer) *reinterpret_cast<float4_t*>(obase + (t * NW + w) * 16 + kg * 4) = o;
    }
    if (writer && w == 0 && kg == 0 && !direct) {
        a.sm[pidx] = M > -1e29f ? M * 0.693147180559945f : kMasked;
        a.ss[pidx] = l;
    }
}

template <int DT, int D, int RUN, int NW, bool CAP>
__global__ __launch_bounds__(NW * 64) void split_mfma_il_kernel(SplitArgs a, uint32_t gt) {
    split_mfma_il_body<DT, D, RUN, NW, CAP, false>(a, gt, nullptr);
}

template <int DT, int D, int RUN, int NW, bool CAP>
__global__ __launch_bounds__(NW * 64) void split_mfma_il_rope_kernel(SplitArgs a, uint32_t gt, RopeFoldArgs rf) {
    split_mfma_il_body<DT, D, RUN, NW, CAP, true>(a, gt, &rf);
}

}  // namespace vfkv
