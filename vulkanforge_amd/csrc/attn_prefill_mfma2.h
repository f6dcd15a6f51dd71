// Matrix-core kernel of the chunked-prefill attention (flash_attn_batch.comp:105-208) for gfx950, second
// generation; included by attn_prefill.hip.
//
// Workgroup = one KV head x 16 consecutive queries.  Its wavefronts are (head slice hp, key split sp): a
// wavefront serves NCB query heads of the GQA group (NCB column blocks of 16 queries each) over the key tiles
// sp, sp + NS, ... of 32 keys.  Nothing is shared between wavefronts inside the loop -- each one converts its own
// K rows, stages its own V tile in a private LDS area and walks at its own pace -- so there is no workgroup
// barrier until the key splits are merged at the end.  Per tile, with v_mfma_f32_16x16x32_f16:
//
//   S^T[key, query] = K[key, :] . Q[query, :]      A = K rows straight from global memory (a lane owns a contiguous
//                                                  quarter row; FP8 widens to f16 exactly), converted once and
//                                                  reused for the NCB heads; B = Q^T, resident in registers
//   softmax (online) in the accumulator layout: a lane owns 8 scores of ONE query, so max / sum need two
//                                                  lane swaps per tile and head; tiles that every query of the
//                                                  block sees completely take a path without any compare
//   O^T[d, query]  += V^T[d, key] . P^T[key, query]  A = V^T through a row-major f16 copy of the tile in LDS and
//                                                  the transposing LDS read, read once for the NCB heads;
//                                                  B = P^T as f16(p) and f16(p - f16(p)) (two products)
//
// Q is used as f16(q); when some q of the workgroup is not exactly representable the first product is
// repeated with f16(q - f16(q)) kept in LDS, which restores f32-level accuracy.
#pragma once
#include <type_traits>

namespace vfkv {

// wavefronts per workgroup when a wavefront serves one head at head_dim <= 128 (fewer registers: three per SIMD)
constexpr int kPrefillOneHeadWaves = 12;

// NH > 1 (head_dim 512): NH = 2 wavefronts share a head.  Each computes the scores of one of the tile's two 16-key halves
// over the whole head_dim (so each loads and widens half of the K tile), the two swap their halves through LDS behind one
// workgroup barrier per tile, and each then
// accumulates, merges and stores its own slice of D / NH output elements: the accumulators of a 512-wide head do not fit
// one wavefront.  HP then counts (head, slice) units.
//
// PAD (NH == 1): the heads are a.head_dim < D elements wide (a multiple of 16: 80 / 96 / 112 on the kernel for 128, 160 /
// 192 / 224 on the one for 256).  The kernel works on rows of D elements whose tail does not exist: the query planes hold
// zeros there, a lane whose 16-byte piece of a K or V row would lie past the head reads the head's first piece again
// (finite values that meet query zeros, or output columns nobody stores), and the d-tiles past head_dim are neither
// multiplied nor stored.  Rows, queries, outputs, partials and the gate keep their real stride of head_dim.
//
// QB2 (NCB == 2, NH == 1; groups of one head): the two column blocks of a wavefront are two blocks of 16 queries of the SAME
// head instead of two heads, so a workgroup covers 32 consecutive queries and a K / V tile is still widened and staged once
// for two column blocks.  Head slot s of the workgroup's query planes then holds queries q0 + 16 (s % 2) .. of head s / 2.
template <int DT, int D, int NCB, int PFD, bool CAP, int NH = 1, bool F16W = false, bool PAD = false, bool QB2 = false>
__global__ __launch_bounds__((NCB == 1 && D <= 128) ? kPrefillOneHeadWaves * 64 : (D == 256 && NH == 2) ? 512 : (NCB * D >= 512 || (DT == kF16 && D == 256)) ? 256 : 512) void batch_mfma2_kernel(BatchArgs a, int HP, int NS) {
    constexpr int DV = D / NH;                   // output elements (V columns) of this wavefront
    constexpr int ES = DT == kF16 ? 2 : 1;
    constexpr int KT = 32;                       // keys per tile
    constexpr int KS = D / 32;                   // MFMA k-steps of the first product
    constexpr int DTILES = DV / 16;
    constexpr int SEG = D / 4, SEGB = SEG * ES;  // a lane group's quarter of a key row
    constexpr int KLD = SEGB / 16;
    constexpr int VPITCH = DV + 16;              // halves per V row (this wavefront's columns) in LDS
    constexpr int VCHUNK_ROW = DV * ES / 16;     // 16-byte chunks per V row
    constexpr int VLD = KT * VCHUNK_ROW / 64;    // V loads per lane per tile
    constexpr int VROWS = 64 / VCHUNK_ROW;
    constexpr float kMaxSlack = 8.0f;            // log2 units by which a score may exceed the running reference maximum
    constexpr uint32_t kNoTile = 0x80000000u;    // byte offset past any slab: the load returns zeros, no memory access
    // the two wavefronts of a head score one 16-key half of a tile each and swap (not with two heads per wavefront over
    // FP8 rows, where a K tile is already widened once for both heads and the barrier per tile costs more than it saves:
    // 16 / 2 / 512, 512 x 4 608: 218 us without, 245 us with)
    constexpr bool XCH = NH == 2 && !(DT == kF8 && NCB == 2);
    constexpr int NKT = XCH ? 1 : 2;             // 16-key halves of a tile this wavefront loads and scores
    static_assert(NH == 1 || NH == 2, "one or two wavefronts per head");
    static_assert(D % 32 == 0 && SEGB % 16 == 0 && VLD >= 1, "unsupported head_dim");
    static_assert(!PAD || NH == 1, "padded heads: one wavefront per head");
    static_assert(!QB2 || (NCB == 2 && NH == 1), "two query blocks per wavefront");
    constexpr int QW = QB2 ? 32 : 16;            // queries of a workgroup
    const uint32_t dr = PAD ? a.head_dim : (uint32_t)D;                 // elements per head as the buffers hold them

    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];      // [waves][KT][VPITCH] V tiles | [GP][16][D + 8] f16(q) | [GP][16][D + 8] remainders
    __shared__ int lds_haslo;

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = HP * NS;
    const int hp = w % HP, sp = w / HP;
    const int n16 = lane & 15, kg = lane >> 4;
    const int G = a.n_heads / a.n_kv_heads;
    // Workgroups are dispatched to the XCDs round-robin in the order of their linear index.  a.xcd_heads (more than eight KV
    // heads, a multiple of eight): XCD x takes the query blocks of KV head x, then those of head x + 8, and so on, so that
    // the rows of one head at a time occupy its L2.
    uint32_t kvh = blockIdx.x, qblk = blockIdx.y;
    if (a.xcd_heads != 0u) {
        const uint32_t id = blockIdx.x + gridDim.x * blockIdx.y, t = id >> 3;
        kvh = (id & 7u) + 8u * (t / gridDim.y);
        qblk = t % gridDim.y;
    }
    const uint32_t q0 = (gridDim.y - 1u - qblk) * QW;         // later query blocks see more keys: longest workgroups first
    const uint32_t qi = q0 + n16;                               // this lane's query (column of S^T; QB2: of column block 0)
    const bool q_ok = qi < a.m;
    auto qi_of = [&](int cb) -> uint32_t { return QB2 ? qi + (uint32_t)cb * 16u : qi; };
    auto qok_of = [&](int cb) -> bool { return QB2 ? qi + (uint32_t)cb * 16u < a.m : q_ok; };
    const uint32_t row_stride = a.n_kv_heads * dr * ES;
    const uint32_t kc = blockIdx.z % a.nk;                      // key chunk of this workgroup (a.nk == 1: all keys)
    const int gz = (blockIdx.z / a.nk) * (HP / NH) * (QB2 ? 1 : NCB);   // first head (inside the group) of this workgroup
    const int g0 = (hp / NH) * (QB2 ? 1 : NCB);                 // first head (inside the workgroup) of this wavefront
    const int s0 = (hp / NH) * NCB;                             // its first head slot in the query planes
    auto head_of = [&](int cb) -> int { return gz + g0 + (QB2 ? 0 : cb); };   // head (inside the group) of column block cb
    const int dslice = hp % NH;                                 // which D / NH output elements this wavefront owns

    _Float16* const vb = lds + (size_t)w * KT * VPITCH;
    constexpr int QPITCH = D + 8;
    _Float16* const qhi_lds = lds + (size_t)nwaves * KT * VPITCH;   // [GP][16][D + 8] f16(q); the slots past G hold zeros
    const int GP = (HP / NH) * NCB;                                 // head slots of the workgroup: G rounded up to whole wavefronts
    _Float16* const qlo_lds = qhi_lds + (size_t)GP * 16 * QPITCH;   // [GP][16][D + 8] f16(q - f16(q))
    float4_t* const xbuf = reinterpret_cast<float4_t*>(qlo_lds + (size_t)GP * 16 * QPITCH);   // XCH: [2][waves][NCB][64] score halves

    // ---- key range ----
    uint32_t kmax = a.q_start + q0 + QW;                        // one past the last key any of the workgroup's queries sees
    if (kmax > a.n_kv) kmax = a.n_kv;
    const uint32_t my_len = q_ok ? (a.q_start + qi + 1 < a.n_kv ? a.q_start + qi + 1 : a.n_kv) : 0;   // causal_len of this lane's query
    const uint32_t my_len1 = (QB2 && qok_of(1)) ? (a.q_start + qi + 17 < a.n_kv ? a.q_start + qi + 17 : a.n_kv) : 0;   // QB2: of its query in column block 1
    auto len_of = [&](int cb) -> uint32_t { return (QB2 && cb == 1) ? my_len1 : my_len; };
    uint32_t full_len = a.q_start + q0 + 1;                     // keys every query of the block sees
    if (full_len > a.n_kv) full_len = a.n_kv;
    uint32_t t_first = (a.kv_start / KT) * KT;
    if (a.nk > 1u) {                                            // this workgroup's chunk of the keys (multiples of KT)
        t_first += kc * a.chunk;
        const uint32_t hi = t_first + a.chunk;
        if (kmax > hi) kmax = hi;
    }
    const uint32_t fast_end = full_len < kmax ? full_len : kmax;   // tiles below it are seen completely by every query (and are this workgroup's)
    const float scale_l2 = a.scale * 1.44269504088896f;
    const float cap_l2 = a.softcap * 1.44269504088896f;

    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.n_kv * row_stride, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.n_kv * row_stride, 0x00020000);
    const uint32_t head_b = kvh * dr * ES;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * SEGB;
    const int vrow = lane / VCHUNK_ROW, vcol = lane % VCHUNK_ROW;
    const uint32_t lane_voff = vrow * row_stride + head_b + dslice * DV * ES + (PAD && (uint32_t)vcol * 16u >= dr * ES ? 0 : vcol * 16);
    uint32_t kpiece[KLD];                        // PAD: offset of the lane's piece x (the head's first piece where x does not exist)
#pragma unroll
    for (int x = 0; x < KLD; ++x) {
        const uint32_t bo = (uint32_t)(kg * SEGB + x * 16);
        kpiece[x] = n16 * row_stride + head_b + (bo < dr * ES ? bo : 0u);
    }

    const uint32_t kt_own = XCH ? (uint32_t)dslice : 0u;         // XCH: the half this wavefront scores
    u32x4 kraw[PFD][NKT][KLD];
    u32x4 vraw[PFD][VLD];
    auto issue = [&](int slot, uint32_t toff) {
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int x = 0; x < KLD; ++x)
                kraw[slot][kt][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, PAD ? kpiece[x] : lane_koff + x * 16, toff + ((uint32_t)kt + kt_own) * 16u * row_stride, 0);
#pragma unroll
        for (int c = 0; c < VLD; ++c)
            vraw[slot][c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, toff + (uint32_t)(c * VROWS) * row_stride, 0);
    };
    const uint32_t step = KT * NS;
    const uint32_t tb0 = t_first + sp * KT;                     // this wavefront's first tile (may already be past the end)
    // XCH: every tile has a workgroup barrier, so every wavefront walks the same number of tiles; the ones past the last key
    // load nothing (zero-returning offsets) and are masked out entirely
    const uint32_t n_my = kmax > t_first ? ((kmax - t_first + KT - 1) / KT + NS - 1) / NS : 0u;
    const uint32_t kloop = XCH ? tb0 + n_my * step : kmax;      // where this wavefront's walk ends
    int xpar = 0;                                               // XCH: which of the two exchange buffers the next tile uses
    auto tile_off = [&](uint32_t t) -> uint32_t { return t < kmax ? t * row_stride : kNoTile; };
    // ---- Q block of the workgroup: 16 queries x G heads x D floats, loaded once with coalesced 16-byte loads (before the
    // K / V requests, so waiting for it does not wait for them) and kept in LDS as an f16 value plane and a remainder plane
    constexpr int QLD = 4;                                      // query loads per thread and round
    const int nthreads = nwaves * 64;
    const int q4_total = 16 * GP * (D / 4);
    bool has_lo = false;
    if (tid == 0) lds_haslo = 0;
    bool any_lo = false;
    for (int base = 0; base < q4_total; base += QLD * nthreads) {
        float4 qf[QLD];
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = base + tid + i * nthreads;
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            bool ok = idx < q4_total && q0 + qq < a.m && rem < (G - gz) * (D / 4);      // head slots past G read nothing
            if (PAD || QB2) {                                   // slot by slot: the heads are dr floats apart (the tail of a slot reads
                                                                // nothing); QB2: slot s holds queries q0 + 16 (s % 2) + qq of head s / 2
                const int sl = rem / (D / 4), d4 = rem - sl * (D / 4);
                const int gq = QB2 ? sl / 2 : sl;
                const uint32_t qrow = q0 + (uint32_t)qq + (QB2 ? (uint32_t)(sl & 1) * 16u : 0u);
                ok = idx < q4_total && qrow < a.m && gq < G - gz && (uint32_t)d4 * 4u < dr;
                qf[i] = *reinterpret_cast<const float4*>(a.q + ((size_t)(ok ? qrow : 0) * a.n_heads + kvh * G + gz + (ok ? gq : 0)) * dr + (ok ? d4 * 4 : 0));
            } else
            qf[i] = *reinterpret_cast<const float4*>(a.q + ((size_t)(ok ? q0 + qq : 0) * a.n_heads + kvh * G + gz) * D + (ok ? rem * 4 : 0));
            if (!ok) qf[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (base == 0) {
#pragma unroll
            for (int sl = 0; sl < PFD; ++sl) issue(sl, tile_off(tb0 + sl * step));
        }
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = base + tid + i * nthreads;
            if (idx >= q4_total) continue;
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            const int g = rem / (D / 4), d = (rem - g * (D / 4)) * 4;
            const float v[4] = {qf[i].x, qf[i].y, qf[i].z, qf[i].w};
            _Float16 hv[4], lv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) { hv[j] = (_Float16)v[j]; lv[j] = (_Float16)(v[j] - (float)hv[j]); any_lo |= lv[j] != (_Float16)0; }
            *reinterpret_cast<half4_t*>(qhi_lds + ((size_t)g * 16 + qq) * QPITCH + d) = half4_t{hv[0], hv[1], hv[2], hv[3]};
            *reinterpret_cast<half4_t*>(qlo_lds + ((size_t)g * 16 + qq) * QPITCH + d) = half4_t{lv[0], lv[1], lv[2], lv[3]};
        }
    }
    __syncthreads();                                            // lds_haslo cleared, planes written
    if (any_lo && a.q_f16 == 0u) lds_haslo = 1;
    __syncthreads();
    has_lo = __builtin_amdgcn_readfirstlane(lds_haslo) != 0;   // workgroup-uniform

    float4_t oacc[NCB][DTILES];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) oacc[cb][dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run[NCB], l_run[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) { m_run[cb] = kMasked; l_run[cb] = 0.f; }

    // ---- pieces of one tile ----
    float4_t s[NCB][2];
    float x[NCB][8], tmax[NCB];
    // V tile -> f16 row-major in this wavefront's LDS area (first: the writes complete behind the first product and the
    // softmax), the slot's next tile requested, then S^T = K Q^T for the NCB heads (Q operands re-read from LDS every tile)
    auto stage_and_first_product = [&](int sl, uint32_t tcur) {
        const uint32_t noff = tile_off(tcur + PFD * step);
#pragma unroll
        for (int c = 0; c < VLD; ++c) {
            _Float16* dst = vb + (c * VROWS + vrow) * VPITCH + vcol * (16 / ES);
            if (DT == kF8) {
                uint32_t out[8];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const uint32_t wd = vraw[sl][c][q4];
                    half2_t lo2, hi2;
                    e4m3x4_to_h2(wd, lo2, hi2);
                    out[2 * q4] = __builtin_bit_cast(uint32_t, lo2);
                    out[2 * q4 + 1] = __builtin_bit_cast(uint32_t, hi2);
                }
                reinterpret_cast<u32x4*>(dst)[0] = u32x4{out[0], out[1], out[2], out[3]};
                reinterpret_cast<u32x4*>(dst)[1] = u32x4{out[4], out[5], out[6], out[7]};
            } else {
                *reinterpret_cast<u32x4*>(dst) = vraw[sl][c];
            }
            vraw[sl][c] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, noff + (uint32_t)(c * VROWS) * row_stride, 0);
        }
        half8_t qhi[NCB][KS];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int c = 0; c < KS; ++c)
                qhi[cb][c] = *reinterpret_cast<const half8_t*>(qhi_lds + ((size_t)(s0 + cb) * 16 + n16) * QPITCH + kg * SEG + c * 8);
        float4_t sown[NCB];                                     // XCH: this wavefront's half of the scores
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            half8_t ka[KS];
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                if (DT == kF8) {
                    const uint32_t w0 = kraw[sl][kt][c / 2][(c % 2) * 2], w1 = kraw[sl][kt][c / 2][(c % 2) * 2 + 1];
                    half2_t p0, p1, p2, p3;
                    e4m3x4_to_h2(w0, p0, p1);
                    e4m3x4_to_h2(w1, p2, p3);
                    ka[c][0] = p0[0]; ka[c][1] = p0[1]; ka[c][2] = p1[0]; ka[c][3] = p1[1];
                    ka[c][4] = p2[0]; ka[c][5] = p2[1]; ka[c][6] = p3[0]; ka[c][7] = p3[1];
                } else {
                    const u32x4 wv = kraw[sl][kt][c % KLD];
                    ka[c] = __builtin_bit_cast(half8_t, wv);
                }
            }
#pragma unroll
            for (int xx = 0; xx < KLD; ++xx)
                kraw[sl][kt][xx] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, PAD ? kpiece[xx] : lane_koff + xx * 16, noff + ((uint32_t)kt + kt_own) * 16u * row_stride, 0);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < KS; ++c) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], qhi[cb][c], acc, 0, 0, 0);
                if (XCH) sown[cb] = acc; else s[cb][kt] = acc;
            }
            if (has_lo) {
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    const _Float16* lo_row = qlo_lds + ((size_t)(s0 + cb) * 16 + n16) * QPITCH + kg * SEG;
                    float4_t acc = XCH ? sown[cb] : s[cb][kt];
#pragma unroll
                    for (int c = 0; c < KS; ++c) {
                        const half8_t ql = *reinterpret_cast<const half8_t*>(lo_row + c * 8);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], ql, acc, 0, 0, 0);
                    }
                    if (XCH) sown[cb] = acc; else s[cb][kt] = acc;
                }
            }
        }
        if constexpr (XCH) {
            // swap halves with the partner wavefront (the other output slice of the same head and key split: w ^ 1).  Two
            // buffers alternate, so one barrier per tile is enough: a buffer is rewritten two tiles later, after a barrier
            // the partner can only have reached by finishing this tile's read.
            float4_t* const xw = xbuf + ((size_t)(xpar * nwaves + w) * NCB) * 64 + lane;
            const float4_t* const xr = xbuf + ((size_t)(xpar * nwaves + (w ^ 1)) * NCB) * 64 + lane;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) xw[cb * 64] = sown[cb];
            __syncthreads();
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const float4_t other = xr[cb * 64];
                s[cb][0] = kt_own == 0u ? sown[cb] : other;
                s[cb][1] = kt_own == 0u ? other : sown[cb];
            }
            xpar ^= 1;
        }
    };
    // scores of the tile in log2 units (this lane owns keys tcur + kt*16 + kg*4 + i of query n16); returns whether one of
    // them exceeds the lane's reference maximum by more than the slack
    auto scores = [&](auto masked_tag, uint32_t tcur) -> bool {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr bool FOLD = !MASKED && !CAP;                   // scores stay unscaled until the exponent's FMA
        bool moved = false;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            tmax[cb] = kMasked;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = FOLD ? s[cb][kt][i] : s[cb][kt][i] * scale_l2;
                    if (CAP) y = cap_l2 * tanhf(y / cap_l2);
                    if (MASKED) {
                        const uint32_t t = tcur + kt * 16 + kg * 4 + i;
                        y = (t < len_of(cb) && t >= a.kv_start && t < kmax) ? y : kMasked;    // (t >= kmax: padding tiles of a key chunk)
                    }
                    x[cb][kt * 4 + i] = y;
                    tmax[cb] = fmaxf(tmax[cb], y);
                }
            if (FOLD) tmax[cb] *= scale_l2;
            moved |= tmax[cb] > m_run[cb] + kMaxSlack;
        }
        return moved;
    };
    auto move_maximum = [&]() {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            float t = tmax[cb];
            { float y = t; swap16(t, y); t = fmaxf(t, y); y = t; swap32(t, y); t = fmaxf(t, y); }
            const float m_new = fmaxf(m_run[cb], t);
            const float alpha = __builtin_amdgcn_exp2f(m_run[cb] - m_new);
            l_run[cb] *= alpha;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) oacc[cb][dt] *= alpha;
            m_run[cb] = m_new;
        }
    };
    // weights as f16 value + f16 remainder, then O^T += V^T P^T for the NCB heads
    // TWO: the weights enter the product as f16 value + f16 remainder (two MFMAs per d-tile and head: f32-level accuracy);
    // otherwise as the f16 value alone (the F16W instantiations).
    auto weights_and_second_product = [&](auto masked_tag, auto two_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr bool TWO = decltype(two_tag)::value;
        constexpr bool FOLD = !MASKED && !CAP;
        u32x4 phi[NCB], plo[NCB];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int j2 = 0; j2 < 4; ++j2) {
                float2_t pp;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float xe = x[cb][2 * j2 + e];
                    float pv = __builtin_amdgcn_exp2f(FOLD ? __builtin_fmaf(xe, scale_l2, -m_run[cb]) : xe - m_run[cb]);
                    if (MASKED) pv = xe > -1e29f ? pv : 0.f;
                    pp[e] = pv;
                }
                l_run[cb] += pp[0] + pp[1];
                phi[cb][j2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pp, half2_t));
                if (TWO) plo[cb][j2] = pack_f16_remainder(pp[0], pp[1], phi[cb][j2]);
            }
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
            if (PAD && (uint32_t)dt * 16u >= dr) continue;          // wavefront-uniform
            // supplier lane s of a 16-lane group points at V[key = 4*kg + s/4 (+16)][d = dt*16 + 4*(s%4)]
            const _Float16* p0 = vb + (kg * 4 + n16 / 4) * VPITCH + dt * 16 + 4 * (n16 % 4);
            const half4_t v0 = lds_read_tr16(p0);
            const half4_t v1 = lds_read_tr16(p0 + 16 * VPITCH);
            half8_t va;
            va[0] = v0[0]; va[1] = v0[1]; va[2] = v0[2]; va[3] = v0[3]; va[4] = v1[0]; va[5] = v1[1]; va[6] = v1[2]; va[7] = v1[3];
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
                oacc[cb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, phi[cb]), oacc[cb][dt], 0, 0, 0);
            if (TWO) {
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb)
                    oacc[cb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, plo[cb]), oacc[cb][dt], 0, 0, 0);
            }
        }
    };

    // ---- the wavefront's tiles.  The reference maximum m of a query only moves when some score of a tile exceeds it by more
    // than 2^kMaxSlack: until then the weights are exp2(x - m) <= 2^kMaxSlack (exact in the f16 value + remainder pair, far
    // from f32 overflow in the sums), the division by l at the end cancels the common factor, and the accumulators are
    // spared a multiplication per tile.  The four lanes of a query share m, so the test needs no reduction: the ballot sees
    // the lane that holds the query's largest score.  Tiles are processed in groups of PFD (one per prefetch slot) by
    // two loops: the inner one only takes tiles that every query of the block sees completely and leaves as soon as a
    // maximum has to move, so that its accumulators have a single definition per tile and stay in place; the outer one
    // handles whatever the inner one left (first tiles, moved maxima, tiles on the causal diagonal or the window edge).
    uint32_t tb = tb0;
    int first_slot = 0;          // slots of the group at tb that the inner loop has already finished
    bool s_ready = false;        // s[] of slot first_slot is already computed
    while (tb < kloop) {
#pragma unroll
        for (int sl = 0; sl < PFD; ++sl) {
            const uint32_t tcur = tb + sl * step;
            if (tcur >= kloop) break;                           // wavefront-uniform
            if (sl < first_slot) continue;
            if (!(s_ready && sl == first_slot)) stage_and_first_product(sl, tcur);
            if (tcur >= a.kv_start && tcur + KT <= fast_end) {  // every query of the block sees the whole tile (and it is this workgroup's)
                if (__builtin_amdgcn_ballot_w64(scores(std::false_type{}, tcur)) != 0ull) move_maximum();
                weights_and_second_product(std::false_type{}, std::integral_constant<bool, !F16W>{});
            } else {
                if (__builtin_amdgcn_ballot_w64(scores(std::true_type{}, tcur)) != 0ull) move_maximum();
                weights_and_second_product(std::true_type{}, std::integral_constant<bool, !F16W>{});
            }
        }
        tb += PFD * step;
        first_slot = 0;
        s_ready = false;
        bool left = false;
        while (!left && tb >= a.kv_start && tb + (PFD - 1) * step + KT <= fast_end) {
#pragma unroll
            for (int sl = 0; sl < PFD; ++sl) {
                const uint32_t tcur = tb + sl * step;
                stage_and_first_product(sl, tcur);
                if (__builtin_amdgcn_ballot_w64(scores(std::false_type{}, tcur)) != 0ull) {
                    first_slot = sl; s_ready = true; left = true;
                    break;
                }
                weights_and_second_product(std::false_type{}, std::integral_constant<bool, !F16W>{});
            }
            if (!left) tb += PFD * step;
        }
    }
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) l_run[cb] = xor32_sum(xor16_sum(l_run[cb]));   // every lane of a query column has its wavefront's sum

    // ---- gated output (vk_shaders/sigmoid_mul.comp:44-52 in this kernel's store): the wavefronts that will store request
    // their gate values and turn them into factors before the merge, so that the round trip overlaps it.  A head's D
    // elements lie in one gate chunk.
    float4_t gfac[NCB][DTILES];
    if (a.gate != nullptr && sp == 0 && q_ok) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            if (head_of(cb) >= G) continue;
            if (QB2 && !qok_of(cb)) continue;
            const uint32_t i0 = (qi_of(cb) * a.n_heads + kvh * G + head_of(cb)) * dr;
            const uint32_t token = i0 / a.gchunk;
            const float* gp = a.gate + (size_t)token * a.gstride + a.goff + (i0 - token * a.gchunk) + dslice * DV + kg * 4;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                if (PAD && (uint32_t)dt * 16u >= dr) continue;
                const float4 gv = *reinterpret_cast<const float4*>(gp + dt * 16);
                gfac[cb][dt] = float4_t{sigmoid_gate(1.0f, gv.x), sigmoid_gate(1.0f, gv.y), sigmoid_gate(1.0f, gv.z), sigmoid_gate(1.0f, gv.w)};
            }
        }
    }

    // ---- merge the key splits through LDS, normalise and store.  Where the launcher found room for it (a.merge_all) and
    // the split count is 2, 4 or 8, every wavefront leaves its (o, m, l) in LDS -- o as [wavefront][cb][dt][lane] float4:
    // 16-byte accesses of consecutive lanes, no bank conflicts -- and the NS wavefronts of a head unit each merge and store
    // the d-tiles dt = sp, sp + NS, ... of the unit's NCB heads, compiled per split count so that the LDS reads of a head
    // are independent instructions.  Otherwise split 0 collects the records of the others one after the other.
    constexpr int REC = DTILES * 4 + 2;
    // (not compiled into the F16 head_dim 256 form: with it that instantiation's tile loop spills twice as many registers, 109 -> 137 us)
    constexpr bool MERGE_ALL = NH == 1 && !(DT == kF16 && D == 256);
    if (MERGE_ALL && NS > 1 && a.merge_all != 0u && (NS == 2 || NS == 4 || NS == 8)) {
        __syncthreads();                                        // every wavefront is done with its V area
        float4_t* obuf = reinterpret_cast<float4_t*>(lds);
        float* mlbuf = reinterpret_cast<float*>(lds) + (size_t)nwaves * NCB * DTILES * 64 * 4;
        const int slot = sp * HP + hp;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) obuf[((size_t)(slot * NCB + cb) * DTILES + dt) * 64 + lane] = oacc[cb][dt];
            mlbuf[((size_t)(slot * NCB + cb) * 2 + 0) * 64 + lane] = m_run[cb];
            mlbuf[((size_t)(slot * NCB + cb) * 2 + 1) * 64 + lane] = l_run[cb];
        }
        __syncthreads();
        if (!q_ok) return;
        auto merge_and_store = [&](auto ns_tag) {
            constexpr int NSC = decltype(ns_tag)::value;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                if (head_of(cb) >= G) continue;                 // padding slot of an odd group
                if (QB2 && !qok_of(cb)) continue;
                float f[NSC], lv[NSC];
#pragma unroll
                for (int s2 = 0; s2 < NSC; ++s2) {
                    const float* ml = mlbuf + ((size_t)((s2 * HP + hp) * NCB + cb) * 2) * 64 + lane;
                    f[s2] = ml[0]; lv[s2] = ml[64];
                }
                float mm = f[0];
#pragma unroll
                for (int s2 = 1; s2 < NSC; ++s2) mm = fmaxf(mm, f[s2]);
                float lsum = 0.f;
#pragma unroll
                for (int s2 = 0; s2 < NSC; ++s2) { f[s2] = __builtin_amdgcn_exp2f(f[s2] - mm); lsum += lv[s2] * f[s2]; }
                const uint32_t h = kvh * G + head_of(cb), qc = qi_of(cb);
                const size_t pidx = ((size_t)qc * a.n_heads + h) * a.nk + kc;      // (key chunks: the partial of this chunk)
                const float inv = a.so != nullptr ? 1.0f : 1.0f / lsum;
                float* op = a.so != nullptr ? a.so + pidx * dr + kg * 4 : a.o + ((size_t)qc * a.n_heads + h) * dr + kg * 4;
                const float* gp = nullptr;
                if (a.gate != nullptr) {
                    const uint32_t i0 = (qc * a.n_heads + h) * dr;
                    const uint32_t token = i0 / a.gchunk;
                    gp = a.gate + (size_t)token * a.gstride + a.goff + (i0 - token * a.gchunk) + kg * 4;
                }
#pragma unroll
                for (int j = 0; j < (DTILES + NSC - 1) / NSC; ++j) {   // lane (query n16) holds d = dt*16 + kg*4 + i
                    const int dt = sp + j * NSC;
                    if (DTILES % NSC != 0 && dt >= DTILES) break;
                    if (PAD && (uint32_t)dt * 16u >= dr) break;
                    float4_t r = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s2 = 0; s2 < NSC; ++s2)
                        r += obuf[((size_t)((s2 * HP + hp) * NCB + cb) * DTILES + dt) * 64 + lane] * f[s2];
                    r *= inv;
                    if (gp != nullptr) {
                        const float4 gv = *reinterpret_cast<const float4*>(gp + dt * 16);
                        r *= float4_t{sigmoid_gate(1.0f, gv.x), sigmoid_gate(1.0f, gv.y), sigmoid_gate(1.0f, gv.z), sigmoid_gate(1.0f, gv.w)};
                    }
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                if (a.so != nullptr && sp == 0 && kg == 0) {
                    a.sm[pidx] = mm > -1e29f ? mm * 0.693147180559945f : kMasked;
                    a.ss[pidx] = lsum;
                }
            }
        };
        if (NS == 4) merge_and_store(std::integral_constant<int, 4>{});
        else if (NS == 2) merge_and_store(std::integral_constant<int, 2>{});
        else merge_and_store(std::integral_constant<int, 8>{});
        return;
    }
    if (NS > 1) {
        __syncthreads();                                        // every wavefront is done with its V area
        float* mbuf = reinterpret_cast<float*>(lds);            // [NS-1][HP][NCB][64][REC]
        if (sp > 0) {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                float* rec = mbuf + ((size_t)(((sp - 1) * HP + hp) * NCB + cb) * 64 + lane) * REC;
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) rec[dt * 4 + i] = oacc[cb][dt][i];
                rec[DTILES * 4] = m_run[cb];
                rec[DTILES * 4 + 1] = l_run[cb];
            }
        }
        __syncthreads();
        if (sp > 0) return;
#pragma unroll 1
        for (int s2 = 1; s2 < NS; ++s2) {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const float* rec = mbuf + ((size_t)(((s2 - 1) * HP + hp) * NCB + cb) * 64 + lane) * REC;
                const float m2 = rec[DTILES * 4], l2 = rec[DTILES * 4 + 1];
                const float mm = fmaxf(m_run[cb], m2);
                const float f1 = __builtin_amdgcn_exp2f(m_run[cb] - mm), f2 = __builtin_amdgcn_exp2f(m2 - mm);
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) oacc[cb][dt][i] = oacc[cb][dt][i] * f1 + rec[dt * 4 + i] * f2;
                l_run[cb] = l_run[cb] * f1 + l2 * f2;
                m_run[cb] = mm;
            }
        }
    }
    if (q_ok) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            if (head_of(cb) >= G) continue;                                   // padding slot of an odd group
            if (QB2 && !qok_of(cb)) continue;
            const uint32_t h = kvh * G + head_of(cb), qc = qi_of(cb);
            if (a.so != nullptr) {
                // key chunks: the unnormalised partial of this chunk in the layout of the decode merge ([row][chunk][D], the
                // maximum in natural-log units); a query that sees no key of the chunk leaves (0, "minus infinity", 0)
                const size_t pidx = ((size_t)qc * a.n_heads + h) * a.nk + kc;
                float* op = a.so + pidx * dr + dslice * DV + kg * 4;
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    if (PAD && (uint32_t)dt * 16u >= dr) continue;
                    const float4_t r = oacc[cb][dt];
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                if (kg == 0 && dslice == 0) {
                    a.sm[pidx] = m_run[cb] > -1e29f ? m_run[cb] * 0.693147180559945f : kMasked;
                    a.ss[pidx] = l_run[cb];
                }
                continue;
            }
            const float inv = 1.0f / l_run[cb];
            float* op = a.o + ((size_t)qc * a.n_heads + h) * dr + dslice * DV + kg * 4;   // lane (query n16) holds d = dslice*DV + dt*16 + kg*4 + i
            if (a.gate != nullptr) {
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    if (PAD && (uint32_t)dt * 16u >= dr) continue;
                    const float4_t r = oacc[cb][dt] * inv * gfac[cb][dt];
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                continue;
            }
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                if (PAD && (uint32_t)dt * 16u >= dr) continue;
                const float4_t r = oacc[cb][dt] * inv;
                *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
            }
        }
    }
}

}  // namespace vfkv
