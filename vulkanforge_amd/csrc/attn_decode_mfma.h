// Matrix-core worker of the split-K decode attention (flash_attn_split.comp:82-162) for gfx950;
// included by attn_decode.hip.
//
// One workgroup (NW wavefronts) owns one (share of the keys, KV head, slice of up to 8 query heads of the
// GQA group); every K / V byte is requested from memory once and serves all heads of the slice.  The
// share is either one tile of consecutive keys (partial j = tile j, the reference's meaning) or, in
// interleaved mode, every n_tiles-th group of NW runs of the visible span.  Each wavefront walks its
// runs of RUN rows and keeps both products on
// v_mfma_f32_16x16x32_f16 (f32 accumulation), so the vector ALU only converts FP8, does the softmax
// and packs the weights:
//
//   S^T[row, col]  = K[row, :] . Q[col, :]     A = K rows straight from global memory (each lane owns a
//                                              contiguous quarter of a row; FP8 widens to f16 exactly),
//                                              B = Q^T, resident in registers.  The 16 columns are
//                                              cols 0..7 = f16(q) of head col, cols 8..15 = f16(q - f16(q))
//                                              of head col-8: adding column c+8 to column c (one DPP
//                                              rotate) gives scores of f32-level accuracy for any f32 Q.
//   softmax        in the accumulator layout: a lane owns 4 rows per 16-row tile of ONE column, so the
//                  running maximum needs two cross-row lane swaps per run and the weights are already
//                  where the second product wants its B operand.
//   O^T[d, col]   += V^T[d, row] . P[row, col]  A = V^T through a row-major f16 copy of the run in LDS read
//                                              with the transposing LDS load, B = P: columns 0..7 carry
//                                              f16(p), columns 8..15 carry f16(p - f16(p)); the two halves
//                                              of O^T are added once, at the end of the tile.
//
// K and V rows of the next run are requested as soon as the registers of the current run are consumed,
// through raw buffer loads whose descriptor ends at the last populated row (rows past it read as zero
// without touching memory, which is also how the prefetch is fed when there is no next run).
#pragma once
#include <type_traits>

namespace vfkv {

// NH > 1 (head_dim 512): NH wavefronts walk the same runs.  Each computes the scores over the whole head_dim and stages,
// accumulates, merges and stores its own slice of D / NH output columns (the accumulators of a 512-wide head do not fit
// one wavefront); the workgroup then walks NW / NH runs at a time.
//
// PAD (NH == 1): the heads of the cache are `head_dim` < D elements wide (a multiple of 16: 80 / 96 / 112 on the kernel for
// 128, 160 / 192 / 224 on the one for 256).  The kernel works on rows of D elements whose tail does not exist: the query
// planes hold zeros there, the lanes whose 16-byte piece of a K or V row would lie past the head read the head's first
// piece again (finite cache values that meet query zeros, or output columns nobody stores), and the d-tiles past head_dim
// are neither multiplied nor stored.  Rows, queries, partials and the appended row keep their real stride of head_dim.
//
// PAIR (D == 128, NH == 1): the cache holds heads of 64 elements, and the kernel takes two neighbouring KV heads as one row
// of 128 (over FP8 rows a head's 64 bytes are half a memory line: as separate heads, possibly on different XCDs, every line
// is fetched twice).  a.n_kv_heads counts the pairs and a.group the query heads of a pair (2 G <= 8, those of the first KV
// head first, as the model numbers them).  A query occupies its own KV head's half of the 128-wide plane row and zeros the
// other half, so its scores only see its own K; of its output row only its own V half is stored.  The cache side
// (rows, the appended row) is exactly that of a head_dim 128 cache with half as many heads.
template <int DT, int D, int RUN, int PF, int NW, bool CAP, int NH = 1, bool PAD = false, bool PAIR = false>
__global__ __launch_bounds__(NW * 64) void split_mfma_kernel(SplitArgs a, uint32_t gt, uint32_t head_dim) {
    constexpr int ES = DT == kF16 ? 2 : 1;
    constexpr int DV = D / NH;                   // output columns of a wavefront
    constexpr int NP = NW / NH;                  // run streams of the workgroup
    constexpr int RT = RUN / 16;                 // 16-row tiles per run
    constexpr int PKS = RUN / 32;                // k-steps (32 rows) of the second product
    constexpr bool HALF = RUN == 16;             // runs of one tile: the second product is the 16-deep matrix instruction
    constexpr int KS = D / 32;                   // k-steps of the first product
    constexpr int DTILES = DV / 16;
    constexpr int SEG = D / 4, SEGB = SEG * ES;  // a lane group's quarter of a K row
    constexpr int KLD = SEGB / 16;               // 16-byte loads per lane per K row
    // Wide rows (a lane's quarter row would be half a 128-byte line or a whole one, read by 4 or 8 loads between which
    // other traffic can evict the line from the CU's cache: 27 % more requests to L2 than lines at 128 bytes): the four
    // lane groups read consecutive 16-byte pieces instead, piece x of group kg at byte (x * 4 + kg) * 16, so a load
    // instruction covers 64 contiguous bytes of each row and a line is done after two.  The query operand is permuted
    // the same way.  (At 32 bytes per quarter both forms touch a line twice.)
    constexpr bool KIL = SEGB >= 64;
    constexpr int VPITCH = DV + 16;              // halves per V row in LDS (+32 B against bank conflicts)
    constexpr int VCHUNK_ROW = DV * ES / 16;     // 16-byte chunks per V row (this wavefront's columns)
    constexpr int VLD = RUN * VCHUNK_ROW / 64;   // V loads per lane per run
    constexpr int VROWS = 64 / VCHUNK_ROW;       // rows covered by one V load of the wavefront
    static_assert(D % 32 == 0 && SEGB % 16 == 0 && (RUN % 32 == 0 || HALF) && VCHUNK_ROW <= 64 && VLD >= 1, "unsupported shape");
    constexpr int MERGE_ROWS = ((DV / 16) * 64 * 16 + VPITCH * 2 - 1) / (VPITCH * 2);    // rows of the staging area the merge needs
    constexpr int LROWS = RUN > MERGE_ROWS ? RUN : MERGE_ROWS;
    static_assert(NW % NH == 0, "whole run streams");
    static_assert(!PAD || NH == 1, "padded heads: one wavefront per run");
    static_assert(!PAIR || (D == 128 && NH == 1 && !PAD), "pairs of 64-wide heads");
    constexpr int QD = PAIR ? 64 : D;                                   // elements of a query / output row (PAD: dr)
    const uint32_t dr = PAD ? head_dim : (uint32_t)D;                   // elements per head as the cache holds them

    __shared__ __attribute__((aligned(16))) _Float16 vlds[NW][LROWS * VPITCH];
    __shared__ float lds_m[NW][8], lds_l[NW][8];
    __shared__ __attribute__((aligned(16))) _Float16 qlds[16][D + 8];   // rows 0-7: f16(q) per head, rows 8-15: remainders

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wp = w / NH, ds = w % NH;          // run stream of this wavefront, its slice of the output columns
    const int n16 = lane & 15, kg = lane >> 4;
    const int col = n16 & 7;
    const bool is_lo = n16 >= 8;
    // KV head fastest: the workgroups of one tile start together.  PAD: a head's slice of a row is not a whole number of
    // 128-byte lines, so neighbouring KV heads share lines; consecutive workgroups go to different XCDs (each with its own
    // L2), so the heads are dealt such that every XCD gets a block of neighbours.
    const uint32_t jl = blockIdx.y;
    const uint32_t kvh = (PAD && (a.n_kv_heads & 7u) == 0u) ? (blockIdx.x & 7u) * (a.n_kv_heads >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t g_all = a.group;                        // n_heads / n_kv_heads, divided on the host
    const uint32_t hz = blockIdx.z * gt;
    const uint32_t gcount = g_all - hz < gt ? g_all - hz : gt;
    const uint32_t h0 = kvh * g_all + hz;
    // Two ways to hand the visible rows to the workgroups.  Contiguous: workgroup jl owns tile jl (the reference's
    // split, partial jl = tile jl).  Interleaved (a.interleave): the rows from the first launched tile to seq_len are
    // one sequence of runs dealt round-robin to all wavefronts of the KV head, so at any moment the whole chip reads
    // one narrow band of position rows front to back -- measurably faster than n_tiles separate streams -- and the
    // partial of workgroup jl covers a comb of runs (the merge does not care which rows a partial covers).
    const bool il = a.interleave != 0u;
    const uint32_t tile_base = il ? a.tile_first * a.tile : (a.tile_first + jl) * a.tile;
    uint32_t tile_end = tile_base + a.tile; if (il || tile_end > a.seq_len) tile_end = a.seq_len;
    const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;

    const uint32_t row_stride = a.n_kv_heads * dr * ES;
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.seq_len * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.seq_len * row_stride, 0x00020000);
    const uint32_t head_b = kvh * dr * ES;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * (KIL ? 16 : SEGB);
    const int vrow = lane / VCHUNK_ROW, vcol = lane % VCHUNK_ROW;
    const uint32_t lane_voff = vrow * row_stride + head_b + ds * DV * ES + (PAD && (uint32_t)vcol * 16u >= dr * ES ? 0 : vcol * 16);
    uint32_t kpiece[KLD];                        // PAD: byte offset of piece x in the head's row (0 where the piece does not exist)
#pragma unroll
    for (int x = 0; x < KLD; ++x) {
        const uint32_t bo = (uint32_t)(kg * (KIL ? 16 : SEGB) + x * (KIL ? 64 : 16));
        kpiece[x] = bo < dr * ES ? bo : 0u;
    }
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;
    const float inv_cap_l2 = CAP ? 1.0f / cap_l2 : 0.f;

    // runs of this wavefront: w, w + NW, ... counted from the first run that reaches the window
    const uint32_t first_run = (lo - tile_base) / RUN;
    const uint32_t n_runs = tile_end > tile_base ? (tile_end - tile_base + RUN - 1) / RUN : 0;
    auto run_off = [&](uint32_t r) -> uint32_t {   // byte offset of a run's first row, or out of bounds when there is none
        return r < n_runs ? (tile_base + r * RUN) * row_stride : kOOB;
    };

    u32x4 kraw[PF][RT][KLD];             // PF runs in flight per wavefront
    u32x4 vraw[PF][VLD];
    auto issue_k = [&](int b, int t, uint32_t off) {
#pragma unroll
        for (int x = 0; x < KLD; ++x)
            kraw[b][t][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, PAD ? n16 * row_stride + head_b + kpiece[x] : lane_koff + x * (KIL ? 64 : 16),
                                                                  off + (uint32_t)(t * 16) * row_stride, 0);
    };
    auto issue_v = [&](int b, int c, uint32_t off) {
        vraw[b][c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, off + (uint32_t)(c * VROWS) * row_stride, 0);
    };

    if (PAD || PAIR) {                                              // the query planes' tails stay zero (nothing is in flight yet: the barrier is cheap here)
        for (int i = tid; i < 16 * (D + 8) / 8; i += NW * 64) reinterpret_cast<u32x4*>(&qlds[0][0])[i] = u32x4{0u, 0u, 0u, 0u};
        __syncthreads();
    }

    // ---- optional fused append (step_kv_write, executor/attention.rs:546): the workgroup whose tile holds the new
    // position converts and stores this KV head's slice of the new K and V rows before anything reads them.  The
    // stores are complete (vmcnt == 0) and the workgroup has met at the barrier before the first load is issued;
    // the lines were not touched by this workgroup before, so the loads fetch them from L2, where the stores went.
    bool owns_new_row = false;
    if (a.k_new != nullptr)
        owns_new_row = il ? ((((a.append_pos - tile_base) / RUN - first_run) / NP) % a.n_tiles == jl)
                          : (a.append_pos >= tile_base && a.append_pos < tile_end);
    if (owns_new_row) {
        constexpr int EPW = 4 / ES;                              // elements per 32-bit word of the cache
        if ((uint32_t)tid < dr / EPW) {
            const size_t src = (size_t)kvh * dr + (size_t)tid * EPW;
            const size_t dst = ((size_t)a.append_pos * a.n_kv_heads + kvh) * dr * ES + (size_t)tid * 4;
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

    // This wavefront's runs are r0, r0 + rs, ...  In a contiguous tile it walks them cyclically from a starting point
    // that depends on the KV head, so that the workgroups reading the same position rows are not all at the same rows
    // at the same time (with separate streams per tile that helps; the interleaved walk is better off without).
    // (No division by a run-time value on the way to the first load: the rotation is taken modulo the largest power
    // of two that fits, and the interleaved walk needs no count of its runs.)
    const uint32_t rs = il ? NP * a.n_tiles : NP;                     // distance between two runs of a wavefront
    const uint32_t r0 = first_run + (il ? jl * NP : 0u) + wp;
    const bool active = lo < tile_end && r0 < n_runs;
    const uint32_t n_cyc = (active && !il) ? (n_runs - r0 + NP - 1) / NP : 0u;   // runs walked cyclically (contiguous tile)
    const uint32_t rot = n_cyc != 0u ? (kvh * 3u) & ((1u << (31 - __builtin_clz(n_cyc))) - 1u) : 0u;
    auto nth_run = [&](uint32_t i) -> uint32_t {   // i-th run of this wavefront; n_runs (= none) past the last
        if (!active) return n_runs;
        if (il) { const uint32_t r = r0 + i * rs; return r < n_runs ? r : n_runs; }
        if (i >= n_cyc) return n_runs;
        uint32_t ii = i + rot;
        if (ii >= n_cyc) ii -= n_cyc;
        return r0 + ii * NP;
    };
    const uint32_t off0 = run_off(nth_run(0));
#pragma unroll
    for (int t = 0; t < RT; ++t) issue_k(0, t, off0);

    // ---- Q^T operands.  The workgroup converts its heads' queries once (coalesced 16-byte loads) into f16 value /
    // remainder planes in LDS; lane (column n16, group kg) then holds q[kg*SEG + c*8 + j], j < 8, per k-step c.
    // The query load sits between the K and the V requests: loads return in order, so the wait for it covers K only.
    constexpr int QLD = (8 * D / 4 + NW * 64 - 1) / (NW * 64);      // 16-byte query loads per thread (<= 8 heads)
    const int nq4 = PAIR ? (int)gcount * (QD / 4) : (int)(gcount * dr) / 4;
    float4 qf[QLD];
#pragma unroll
    for (int i = 0; i < QLD; ++i) {
        const int idx = tid + i * NW * 64;
        qf[i] = *reinterpret_cast<const float4*>(a.q + (size_t)h0 * (PAIR ? (uint32_t)QD : dr) + (idx < nq4 ? idx : 0) * 4);
    }
#pragma unroll
    for (int c = 0; c < VLD; ++c) issue_v(0, c, off0);
#pragma unroll
    for (int b = 1; b < PF; ++b) {
        const uint32_t offb = run_off(nth_run(b));
#pragma unroll
        for (int t = 0; t < RT; ++t) issue_k(b, t, offb);
#pragma unroll
        for (int c = 0; c < VLD; ++c) issue_v(b, c, offb);
    }
    {
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * NW * 64;
            if (idx >= nq4) continue;
            const float4 f = qf[i];
            const int g = PAD ? (int)((uint32_t)(idx * 4) / dr) : (idx * 4) / QD;
            // (PAIR: the heads of the pair's second KV head use the second half of the row)
            const int d = PAD ? idx * 4 - g * (int)dr : (idx * 4) % QD + ((PAIR && hz + (uint32_t)g >= g_all / 2u) ? 64 : 0);
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

    float4_t oacc[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) oacc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = kMasked, l_run = 0.f;
    _Float16* const vb = &vlds[w][0];

    if (active) {
        for (uint32_t it = 0; nth_run(it) < n_runs; it += PF) {
#pragma unroll
          for (int b = 0; b < PF; ++b) {
            const uint32_t rr = nth_run(it + b);
            if (rr >= n_runs) break;                                     // wavefront-uniform
            const uint32_t noff = run_off(nth_run(it + b + PF));
            const uint32_t rb = tile_base + rr * RUN;
            // ---------------- S^T = K Q^T ----------------
            float4_t s[RT];
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                half8_t ka[KS];
#pragma unroll
                for (int c = 0; c < KS; ++c) {
                    if (DT == kF8) {
                        const uint32_t w0 = kraw[b][t][c / 2][(c % 2) * 2], w1 = kraw[b][t][c / 2][(c % 2) * 2 + 1];
                        half2_t p0, p1, p2, p3;
                        e4m3x4_to_h2(w0, p0, p1);
                        e4m3x4_to_h2(w1, p2, p3);
                        ka[c][0] = p0[0]; ka[c][1] = p0[1]; ka[c][2] = p1[0]; ka[c][3] = p1[1];
                        ka[c][4] = p2[0]; ka[c][5] = p2[1]; ka[c][6] = p3[0]; ka[c][7] = p3[1];
                    } else {
                        const u32x4 wv = kraw[b][t][c % KLD];
                        ka[c] = __builtin_bit_cast(half8_t, wv);
                    }
                }
                issue_k(b, t, noff);
                s[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < KS; ++c) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], qb[c], s[t], 0, 0, 0);
            }
            // ---------------- softmax: this lane owns rows rb + t*16 + kg*4 + i of column n16 ----------------
            const bool interior = rb >= lo && rb + RUN <= tile_end;      // wavefront-uniform
            u32x4 pbits[PKS > 0 ? PKS : 1];
            uint32_t pext[2] = {0u, 0u};
            auto softmax = [&](auto masked_tag) {
                constexpr bool MASKED = decltype(masked_tag)::value;
                constexpr bool FOLD = !MASKED && !CAP;                   // scores stay unscaled until the exponent
                float x[RT][4];
                float tmax = kMasked;
#pragma unroll
                for (int t = 0; t < RT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float y = s[t][i];
                        y += dpp_f<kDppRor8>(y);                         // f16(q) part + remainder part
                        if (!FOLD) y *= scale_l2;                        // FOLD: the scale rides in the exponent's FMA
                        if (CAP) y = softcap_l2(y, cap_l2, inv_cap_l2);
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
                // weights as f16 value (columns 0-7) or f16 remainder (columns 8-15), two rows per register
#pragma unroll
                for (int t = 0; t < RT; ++t)
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
                        if (HALF) pext[i2] = is_lo ? pl : ph;
                        else pbits[t / 2][(t % 2) * 2 + i2] = is_lo ? pl : ph;
                    }
            };
            if (interior) softmax(std::false_type{}); else softmax(std::true_type{});
            half8_t pb[PKS > 0 ? PKS : 1];
#pragma unroll
            for (int ks = 0; ks < PKS; ++ks) pb[ks] = __builtin_bit_cast(half8_t, pbits[ks]);
            // ---------------- V run -> f16 row-major in LDS ----------------
#pragma unroll
            for (int c = 0; c < VLD; ++c) {
                _Float16* dst = vb + (c * VROWS + vrow) * VPITCH + vcol * (16 / ES);
                if (DT == kF8) {
                    uint32_t out[8];
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        const uint32_t wd = vraw[b][c][q4];
                        half2_t lo2, hi2;
                        e4m3x4_to_h2(wd, lo2, hi2);
                        out[2 * q4] = __builtin_bit_cast(uint32_t, lo2);
                        out[2 * q4 + 1] = __builtin_bit_cast(uint32_t, hi2);
                    }
                    reinterpret_cast<u32x4*>(dst)[0] = u32x4{out[0], out[1], out[2], out[3]};
                    reinterpret_cast<u32x4*>(dst)[1] = u32x4{out[4], out[5], out[6], out[7]};
                } else {
                    *reinterpret_cast<u32x4*>(dst) = vraw[b][c];
                }
                issue_v(b, c, noff);
            }
            // ---------------- O^T += V^T P ----------------
#pragma unroll
            for (int ks = 0; ks < PKS; ++ks)
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    if (PAD && (uint32_t)dt * 16u >= dr) continue;     // wavefront-uniform
                    // supplier lane s of a 16-lane group points at V[row = ks*32 + 4*kg + s/4 (+16)][d = dt*16 + 4*(s%4)]
                    const _Float16* p0 = vb + (ks * 32 + kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                    const half4_t v0 = lds_read_tr16(p0);
                    const half4_t v1 = lds_read_tr16(p0 + 16 * VPITCH);
                    half8_t va;
                    va[0] = v0[0]; va[1] = v0[1]; va[2] = v0[2]; va[3] = v0[3]; va[4] = v1[0]; va[5] = v1[1]; va[6] = v1[2]; va[7] = v1[3];
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb[ks], oacc[dt], 0, 0, 0);
                }
            if (HALF) {                    // one tile of 16 rows: the 16-deep product on the tile's own weights
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    if (PAD && (uint32_t)dt * 16u >= dr) continue;
                    const _Float16* p0 = vb + (kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
                    const half4_t v0 = lds_read_tr16(p0);
                    const u32x2 pw = u32x2{pext[0], pext[1]};
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x16f16(v0, __builtin_bit_cast(half4_t, pw), oacc[dt], 0, 0, 0);
                }
            }
          }
        }
    }

    // ---------------- wavefront totals, then the workgroup merge through LDS ----------------
    // Every wavefront parks its accumulators in LDS in register order (lane-major: conflict-free 16-byte accesses),
    // then wavefront w merges the d-tiles w, w + NW, ... of all wavefronts and stores them straight from registers
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
    // all LDS reads of the merge are issued before the first use, so their latencies overlap
    // (with output slices: among the NP wavefronts that own the same columns; their statistics are those of the streams)
    constexpr int MT = DTILES / NP;                    // d-tiles merged and stored by each wavefront
    static_assert(DTILES % NP == 0, "d-tiles must divide evenly among the wavefronts");
    float mw[NP], lw[NP];
    float4_t part[MT][NP];
#pragma unroll
    for (int pp = 0; pp < NP; ++pp) { mw[pp] = lds_m[pp * NH + ds][col]; lw[pp] = lds_l[pp * NH + ds][col]; }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int pp = 0; pp < NP; ++pp) part[t][pp] = slot[((pp * NH + ds) * DTILES + t * NP + wp) * 64 + lane];
    float M = mw[0];
#pragma unroll
    for (int pp = 1; pp < NP; ++pp) M = fmaxf(M, mw[pp]);
    float fw[NP];
    float l = 0.f;
#pragma unroll
    for (int pp = 0; pp < NP; ++pp) {
        fw[pp] = __builtin_amdgcn_exp2f(mw[pp] - M);
        l = fmaf(fw[pp], lw[pp], l);
    }
    const bool writer = !is_lo && (uint32_t)col < gcount;
    const size_t pidx = (size_t)(h0 + col) * a.n_tiles + jl;
    // a single tile covers every visible key (the reference's single-workgroup shader for seq <= 64,
    // forward/runs.rs:776-821): the merge is a plain normalisation, done here, and no merge launch follows
    const bool direct = a.o_direct != nullptr;
    const float inv_l = direct ? __builtin_amdgcn_rcpf(l) : 1.0f;
    float* const obase = (direct ? a.o_direct + (size_t)(h0 + col) * (PAIR ? (uint32_t)QD : dr) : a.so + pidx * (PAIR ? (uint32_t)QD : dr)) + ds * DV;
    const bool second_half = PAIR && (hz + (uint32_t)col) >= g_all / 2u;     // PAIR: this column's head belongs to the pair's second KV head
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        float4_t o = fw[0] * part[t][0];
#pragma unroll
        for (int pp = 1; pp < NP; ++pp) o += fw[pp] * part[t][pp];
        if (direct) {                                  // one Newton step brings the reciprocal to f32 accuracy
            const float r = inv_l * (2.0f - l * inv_l);
            o *= r;
        }
        if (PAIR) {                                    // d-tiles 0-3 are the first KV head's V columns, 4-7 the second's
            const int dt = t * NP + wp;
            if (writer && (dt >= 4) == second_half) *reinterpret_cast<float4_t*>(obase + (dt & 3) * 16 + kg * 4) = o;
        } else
        if (writer && (!PAD || (uint32_t)(t * NP + wp) * 16u < dr)) *reinterpret_cast<float4_t*>(obase + (t * NP + wp) * 16 + kg * 4) = o;
    }
    if (writer && w == 0 && kg == 0 && a.o_direct == nullptr) {
        a.sm[pidx] = M > -1e29f ? M * 0.693147180559945f : kMasked;
        a.ss[pidx] = l;
    }
}

}  // namespace vfkv
