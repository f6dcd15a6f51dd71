// Chunked-prefill attention (flash_attn_batch.comp:105-208) over FP8 rows of 128 elements, two query heads per wavefront:
// the form of batch_mfma2_kernel (attn_prefill_mfma2.h: workgroup = one KV head x 16 queries, wavefronts = head pair x key
// split, S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_16x16x32_f16, lazy running maximum, Q planes in LDS) with two
// differences.
//
//   V through LDS without registers.  A V tile goes from global memory straight into LDS as the cache holds it (buffer
//   loads with the LDS bit; three tiles per wavefront in rotation: the one being read and the next two under way), the
//   second product's operand comes from the byte-transposing LDS read and is widened to f16 in registers.  The wavefront
//   holds no V registers and writes no f16 copy.
//
//   Two tiles per pass.  The registers V no longer needs hold a second tile's scores: the fast loop issues the first
//   products of two tiles, then both softmaxes and second products, in one basic block, so that matrix instructions of one
//   tile stand between the vector instructions of the other.  (With general f32 queries the remainder product of Q leaves
//   no room for it and the loop takes one tile per pass.)
//
// and three measures that even out the work inside a workgroup of eight wavefronts (two per SIMD): the key splits of the
// older wavefront of a SIMD take three tiles for every two of the younger one's (the older one issues first whenever both
// are ready); the head pairs of a workgroup take mirrored query blocks, so that every workgroup and every SIMD walks the
// same number of tiles whatever the causal mask leaves each block; and every wavefront merges and stores a share of the
// output tiles.
//
// Included by attn_prefill.hip after attn_prefill_mfma2.h.
#pragma once
#include <type_traits>

namespace vfkv {

template <bool CAP, bool F16W, bool F8S>
__global__ __launch_bounds__(512) void batch_dma_kernel(BatchArgs a, int HP, int NS, int DEAL_A, int DEAL_B) {
    constexpr int D = 128, NCB = 2, PFD = 2;     // head_dim, heads per wavefront, K tiles in flight
    constexpr int KT = 32;                       // keys per tile
    constexpr int KS = D / 32;                   // MFMA k-steps of the first product
    constexpr int DTILES = D / 16;
    constexpr int SEG = D / 4;                   // a lane group's quarter of a key row (bytes = elements)
    constexpr int KLD = SEG / 16;
    constexpr int VBUF = KT * D;                 // bytes of a raw V tile
    constexpr float kMaxSlack = 8.0f;            // log2 units by which a score may exceed the running reference maximum
    constexpr uint32_t kNoTile = 0x80000000u;    // byte offset past any slab: the load returns zeros, no memory access

    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];      // [waves][3][KT * D] bytes: V tiles | [GP][16][D + 8] f16(q) | [GP][16][D + 8] remainders
    __shared__ int lds_haslo;
    __shared__ uint32_t lds_qmax;                                // F8S: bits of the largest |q| of the workgroup's Q block

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = HP * NS;
    // Wavefront w: key split w / HP of head pair (w % HP) -- in a workgroup of eight the second four are turned by one
    // head pair, so that the two wavefronts of a SIMD (w and w + 4) belong to different head pairs.
    const int sp = w / HP;
    const int hp = (nwaves == 8 && HP <= 4 && w >= 4 ? w + 1 : w) % HP;
    const int n16 = lane & 15, kg = lane >> 4;
    const int G = a.n_heads / a.n_kv_heads;
    const uint32_t kvh = blockIdx.x;
    // Later query blocks see more keys.  The even head pairs of workgroup y take query block (last - y), the odd ones block
    // y: every workgroup then has the same number of tiles, and with the turn above so has every SIMD (to within a tenth of
    // the difference of the two blocks).  With an odd number of head pairs every wavefront takes block (last - y), the
    // longest workgroups first.
    const bool mirrored = HP % 2 == 0 && (hp & 1) != 0;
    const uint32_t q0_even = (gridDim.y - 1u - blockIdx.y) * 16, q0_odd = HP % 2 == 0 ? blockIdx.y * 16 : q0_even;
    const uint32_t q0 = mirrored ? q0_odd : q0_even;
    const uint32_t qi = q0 + n16;                               // this lane's query (column of S^T)
    const bool q_ok = qi < a.m;
    const uint32_t row_stride = a.n_kv_heads * D;
    const uint32_t kc = blockIdx.z % a.nk;                      // key chunk of this workgroup (a.nk == 1: all keys)
    const int gz = (blockIdx.z / a.nk) * HP * NCB;              // first head (inside the group) of this workgroup
    const int g0 = hp * NCB;                                    // first head slot (inside the workgroup) of this wavefront

    uint8_t* const v8 = reinterpret_cast<uint8_t*>(lds) + (size_t)w * 3 * VBUF;   // [3][KT * D] raw V tiles of this wavefront
    constexpr int QPITCH = D + 8;
    _Float16* const qhi_lds = lds + (size_t)nwaves * 3 * VBUF / 2;  // [GP][16][D + 8] f16(q); the slots past G hold zeros
    const int GP = HP * NCB;                                        // head slots of the workgroup: G rounded up to whole wavefronts
    _Float16* const qlo_lds = qhi_lds + (size_t)GP * 16 * QPITCH;   // [GP][16][D + 8] f16(q - f16(q))
    uint8_t* const qlo8_lds = reinterpret_cast<uint8_t*>(qlo_lds + (size_t)GP * 16 * QPITCH);   // [GP][16][D + 16] the remainders as E4M3 codes

    // ---- key range ----
    uint32_t kmax = a.q_start + q0 + 16;                        // one past the last key any of the 16 queries sees
    if (kmax > a.n_kv) kmax = a.n_kv;
    const uint32_t my_len = q_ok ? (a.q_start + qi + 1 < a.n_kv ? a.q_start + qi + 1 : a.n_kv) : 0;   // causal_len of this lane's query
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
    const uint32_t head_b = kvh * D;
    const uint32_t lane_koff = n16 * row_stride + head_b + kg * SEG;

    u32x4 kraw[PFD][2][KLD];
    // A buffer load with the LDS bit writes lane L's 16 bytes at (LDS base) + 16 L, so one load lays down eight rows of
    // 128 bytes; which 16-byte chunk of its row a lane fetches is free.  Lane L of the load for rows 8 b .. 8 b + 7 fetches
    // chunk (L % 8) ^ rot(row) of row 8 b + L / 8, rot(row) = (row % 8) ^ (row >= 16 ? 4 : 0): the transposing read of the
    // second product then takes one chunk index from eight rows (four consecutive ones and the four 16 rows further) and
    // finds them in eight different bank groups.
    const uint32_t lane_vdma = (uint32_t)(lane / 8) * row_stride + head_b;
    const uint32_t vdma_lo = lane_vdma + (uint32_t)(((lane % 8) ^ (lane / 8)) * 16);          // rows 0..15 of a tile
    const uint32_t vdma_hi = lane_vdma + (uint32_t)(((lane % 8) ^ (lane / 8) ^ 4) * 16);      // rows 16..31
    const int vrow_rd = (n16 < 8 ? 0 : 16) + kg * 4 + (n16 / 2) % 4;        // the row this lane supplies to the transposing read
    const uint32_t vdma_rd = (uint32_t)((vrow_rd >> 3) * 1024 + (vrow_rd & 7) * 128 + (n16 & 1) * 8 +
                                        (((vrow_rd & 7) ^ (vrow_rd >= 16 ? 4 : 0)) << 4));   // chunk index dt enters by XOR
    int vcur = 0;                                               // buffer (0..2) of the tile the second product reads next
    // The loads are written as assembly: the compiler would otherwise wait, before every LDS read, for the newest load that
    // writes LDS -- the prefetch of the tile after next -- because it cannot tell the three buffers apart.  Here the wait in
    // front of the transposing reads counts the loads issued since the tile they read: vmcnt(8), two tiles of four loads
    // (loads into registers that the compiler places between them only make the count more patient than necessary).
    const u32x4 vdesc = u32x4{(uint32_t)(uintptr_t)a.v, (uint32_t)((uintptr_t)a.v >> 32) & 0xFFFFu, a.n_kv * row_stride, 0x00020000u};
    const uint32_t v8_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)v8;
    auto v_dma = [&](int buf, uint32_t toff) {
#pragma unroll
        for (int b = 0; b < 4; ++b)
            // (m0 is listed as clobbered, so the compiler sets it again in front of any instruction of its own that reads it)
            asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(v8_addr + (uint32_t)(buf * VBUF + b * 1024)), "v"(b < 2 ? vdma_lo : vdma_hi), "s"(vdesc),
                            "s"(toff + (uint32_t)(b * 8) * row_stride) : "memory", "m0");
    };
    auto issue = [&](int slot, uint32_t toff) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int x = 0; x < KLD; ++x)
                kraw[slot][kt][x] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + x * 16, toff + (uint32_t)kt * 16u * row_stride, 0);
        v_dma(slot, toff);
    };
    // rows past the end of the cache are outside the buffer: whatever such a lane leaves in LDS only ever meets weights of
    // zero, so it must be a finite number -- the buffers start as zeros
#pragma unroll
    for (int i = 0; i < 3 * VBUF / (64 * 16); ++i) *reinterpret_cast<u32x4*>(v8 + (i * 64 + lane) * 16) = u32x4{0u, 0u, 0u, 0u};
    __builtin_amdgcn_s_waitcnt(0xC07F);                         // lgkmcnt(0): the zeros are in place before a load can overwrite them
    // Which tiles a wavefront takes.  The key splits deal the tiles round-robin, but not evenly: of two wavefronts on one
    // SIMD the older one issues first whenever both are ready, so it advances about 1.5 times as fast, and an even deal
    // leaves the younger one to finish alone at the single-wavefront rate.  Per period the splits of the older half of the
    // workgroup take DEAL_A tiles each and the others DEAL_B (DEAL_A >= DEAL_B >= 1; equal: the even deal): DEAL_B rows of
    // NS tiles, then DEAL_A - DEAL_B rows of NS / 2 tiles for the older half.  tp[] holds the positions of the wavefront's
    // next four tiles (slot sl works on tp[sl]; its next one, already requested, is tp[sl + PFD]).
    const uint32_t step = KT * NS;
    const bool older = sp * 2 < NS;
    const uint32_t deal_n = older ? (uint32_t)DEAL_A : (uint32_t)DEAL_B;
    const uint32_t deal_period = (uint32_t)DEAL_B * step + (uint32_t)(DEAL_A - DEAL_B) * (step / 2);
    uint32_t deal_base = t_first + sp * KT, deal_r = 0;         // (a wavefront's first tile may already be past the end)
    auto next_tile = [&]() -> uint32_t {
        const uint32_t p = deal_base + (deal_r < (uint32_t)DEAL_B ? deal_r * step : (uint32_t)DEAL_B * step + (deal_r - (uint32_t)DEAL_B) * (step / 2));
        if (++deal_r == deal_n) { deal_r = 0; deal_base += deal_period; }
        return p;
    };
    uint32_t tp[2 * PFD];
#pragma unroll
    for (int i = 0; i < 2 * PFD; ++i) tp[i] = next_tile();
    auto advance = [&]() {
#pragma unroll
        for (int i = 0; i < PFD; ++i) tp[i] = tp[i + PFD];
#pragma unroll
        for (int i = 0; i < PFD; ++i) tp[PFD + i] = next_tile();
    };
    const uint32_t kloop = kmax;                                // where this wavefront's walk ends
    auto tile_off = [&](uint32_t t) -> uint32_t { return t < kmax ? t * row_stride : kNoTile; };
    // ---- Q block of the workgroup: 16 queries x G heads x D floats, loaded once with coalesced 16-byte loads (before the
    // K / V requests, so waiting for it does not wait for them) and kept in LDS as an f16 value plane and a remainder plane
    constexpr int QLD = 4;                                      // query loads per thread and round
    const int nthreads = nwaves * 64;
    const int q4_total = 16 * GP * (D / 4);
    // F8S: Q as three E4M3 planes q ~ 2^e (t1 + t2 / 16 + t3 / 256), every term the E4M3 rounding of what the terms before it
    // left (12 significant bits: exact for f16-representable q; e keeps the largest |q| of the block below 256).  The first
    // product then runs on the FP8 matrix instruction with the cache rows as they are.
    constexpr int Q8PITCH = D + 16;                             // bytes per (head slot, query) row of a term plane
    uint8_t* const q8_lds = reinterpret_cast<uint8_t*>(qhi_lds);    // [3][GP][16][Q8PITCH]
    int q_exp = 0;
    bool has_lo = false;
    if constexpr (F8S) {
        if (tid == 0) lds_qmax = 0u;
        float4 qf[QLD];                                         // the launcher guarantees q4_total <= QLD * nthreads
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * nthreads;
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            const uint32_t qrow = (((rem / (D / 4)) / NCB) & 1 ? q0_odd : q0_even) + qq;     // the head slot's query block
            const bool ok = idx < q4_total && qrow < a.m && rem < (G - gz) * (D / 4);
            qf[i] = *reinterpret_cast<const float4*>(a.q + ((size_t)(ok ? qrow : 0) * a.n_heads + kvh * G + gz) * D + (ok ? rem * 4 : 0));
            if (!ok) qf[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            amax = fmaxf(fmaxf(amax, fmaxf(fabsf(qf[i].x), fabsf(qf[i].y))), fmaxf(fabsf(qf[i].z), fabsf(qf[i].w)));
        }
#pragma unroll
        for (int sl = 0; sl < PFD; ++sl) issue(sl, tile_off(tp[sl]));
        __syncthreads();                                        // lds_qmax cleared
        amax = wave_max_uniform(amax);
        if (lane == 0) atomicMax(&lds_qmax, __builtin_bit_cast(uint32_t, amax));   // non-negative floats order like their bits
        __syncthreads();
        const uint32_t mb = lds_qmax;
        q_exp = (int)((mb >> 23) & 0xFFu) - 127 - 7;            // floor(log2(max|q|)) - 7: max|q| * 2^-e < 256
        q_exp = q_exp < -100 ? -100 : q_exp > 100 ? 100 : q_exp;
        const float down = __builtin_bit_cast(float, (uint32_t)(127 - q_exp) << 23);
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = tid + i * nthreads;
            if (idx >= q4_total) continue;
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            const int g = rem / (D / 4), d = (rem - g * (D / 4)) * 4;
            float r[4] = {qf[i].x * down, qf[i].y * down, qf[i].z * down, qf[i].w * down};
#pragma unroll
            for (int t = 0; t < 3; ++t) {
                int w8 = __builtin_amdgcn_cvt_pk_fp8_f32(r[0], r[1], 0, false);
                w8 = __builtin_amdgcn_cvt_pk_fp8_f32(r[2], r[3], w8, true);
                *reinterpret_cast<uint32_t*>(q8_lds + ((size_t)(t * GP + g) * 16 + qq) * Q8PITCH + d) = (uint32_t)w8;
                const float2_t d01 = __builtin_amdgcn_cvt_pk_f32_fp8(w8, false), d23 = __builtin_amdgcn_cvt_pk_f32_fp8(w8, true);
                r[0] = (r[0] - d01[0]) * 16.f; r[1] = (r[1] - d01[1]) * 16.f;
                r[2] = (r[2] - d23[0]) * 16.f; r[3] = (r[3] - d23[1]) * 16.f;
            }
        }
        __syncthreads();                                        // planes written
    } else {
    if (tid == 0) { lds_haslo = 0; lds_qmax = 0u; }
    bool any_lo = false;
    float lo_max = 0.f;                                         // largest |q - f16(q)| this thread has seen
    for (int base = 0; base < q4_total; base += QLD * nthreads) {
        float4 qf[QLD];
#pragma unroll
        for (int i = 0; i < QLD; ++i) {
            const int idx = base + tid + i * nthreads;
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            const uint32_t qrow = (((rem / (D / 4)) / NCB) & 1 ? q0_odd : q0_even) + qq;     // the head slot's query block
            const bool ok = idx < q4_total && qrow < a.m && rem < (G - gz) * (D / 4);      // head slots past G read nothing
            qf[i] = *reinterpret_cast<const float4*>(a.q + ((size_t)(ok ? qrow : 0) * a.n_heads + kvh * G + gz) * D + (ok ? rem * 4 : 0));
            if (!ok) qf[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (base == 0) {
#pragma unroll
            for (int sl = 0; sl < PFD; ++sl) issue(sl, tile_off(tp[sl]));
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
            for (int j = 0; j < 4; ++j) {
                hv[j] = (_Float16)v[j]; lv[j] = (_Float16)(v[j] - (float)hv[j]); any_lo |= lv[j] != (_Float16)0;
                lo_max = fmaxf(lo_max, fabsf((float)lv[j]));
            }
            *reinterpret_cast<half4_t*>(qhi_lds + ((size_t)g * 16 + qq) * QPITCH + d) = half4_t{hv[0], hv[1], hv[2], hv[3]};
            *reinterpret_cast<half4_t*>(qlo_lds + ((size_t)g * 16 + qq) * QPITCH + d) = half4_t{lv[0], lv[1], lv[2], lv[3]};
        }
    }
    __syncthreads();                                            // lds_haslo cleared, planes written
    if (any_lo && a.q_f16 == 0u) lds_haslo = 1;
    lo_max = wave_max_uniform(lo_max);
    if (lane == 0) atomicMax(&lds_qmax, __builtin_bit_cast(uint32_t, lo_max));   // non-negative floats order like their bits
    __syncthreads();
    has_lo = __builtin_amdgcn_readfirstlane(lds_haslo) != 0;   // workgroup-uniform
    if (has_lo) {
        // General f32 queries.  The cache rows are E4M3 codes, so K (q - f16(q))^T can run on the FP8 matrix instruction with
        // the rows as loaded: one instruction spans the whole row where the f16 one needs four, and the remainders only
        // need the few bits E4M3 gives them (q is then carried with 15 significant bits).  Every thread turns the remainders
        // it wrote above into codes 2^-e (q - f16(q)), e keeping the largest of the block below 256; 2^e rides in the
        // instruction's block-scale operand.
        const uint32_t mb = lds_qmax;
        q_exp = (int)((mb >> 23) & 0xFFu) - 127 - 7;
        q_exp = q_exp < -100 ? -100 : q_exp > 100 ? 100 : q_exp;
        const float down = __builtin_bit_cast(float, (uint32_t)(127 - q_exp) << 23);
        for (int idx = tid; idx < q4_total; idx += nthreads) {
            const int qq = idx / (GP * (D / 4)), rem = idx - qq * (GP * (D / 4));
            const int g = rem / (D / 4), d = (rem - g * (D / 4)) * 4;
            const half4_t lv = *reinterpret_cast<const half4_t*>(qlo_lds + ((size_t)g * 16 + qq) * QPITCH + d);
            int w8 = __builtin_amdgcn_cvt_pk_fp8_f32((float)lv[0] * down, (float)lv[1] * down, 0, false);
            w8 = __builtin_amdgcn_cvt_pk_fp8_f32((float)lv[2] * down, (float)lv[3] * down, w8, true);
            *reinterpret_cast<uint32_t*>(qlo8_lds + ((size_t)g * 16 + qq) * Q8PITCH + d) = (uint32_t)w8;
        }
        __syncthreads();
    }
    }

    float4_t oacc[NCB][DTILES];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) oacc[cb][dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run[NCB], l_run[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) { m_run[cb] = kMasked; l_run[cb] = 0.f; }

    // ---- pieces of one tile ----
    float4_t s[PFD][NCB][2];
    float x[PFD][NCB][8], tmax[PFD][NCB];
    // the request for the V tile after next: it goes where the tile before the current one was
    auto stage_v = [&](int sl) {
        const int nb = vcur + 2 >= 3 ? vcur - 1 : vcur + 2;
        v_dma(nb, tile_off(tp[sl + PFD]));
    };
    // S^T = K Q^T for the NCB heads (Q operands re-read from LDS every tile); lo_tag: whether the remainder plane of Q takes
    // part (a bool, or a type where the walk is compiled once per case)
    auto first_product = [&](int sl, uint32_t tcur, auto lo_tag) {
        bool with_lo;
        if constexpr (std::is_same_v<decltype(lo_tag), bool>) with_lo = lo_tag; else with_lo = decltype(lo_tag)::value;
        const uint32_t noff = tile_off(tp[sl + PFD]);
        if constexpr (F8S) {
            // S^T = K Q^T on the FP8 matrix instruction: A = the lane's quarter row of K as loaded (32 codes), B = the same
            // quarter of the query's three term planes, each with its power-of-two weight as the instruction's block scale
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) s[sl][cb][kt] = float4_t{0.f, 0.f, 0.f, 0.f};
            typedef int v8i_t __attribute__((ext_vector_type(8)));
            v8i_t ka8[2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int j = 0; j < 8; ++j) ka8[kt][j] = (int)kraw[sl][kt][j / 4][j % 4];
#pragma unroll
            for (int t = 0; t < 3; ++t) {
                const int sb = 127 + q_exp - 4 * t;             // E8M0 code of 2^(e - 4t)
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    const uint8_t* qrow = q8_lds + ((size_t)(t * GP + g0 + cb) * 16 + n16) * Q8PITCH + kg * 32;
                    const u32x4 b0 = *reinterpret_cast<const u32x4*>(qrow), b1 = *reinterpret_cast<const u32x4*>(qrow + 16);
                    v8i_t qb8;
#pragma unroll
                    for (int j = 0; j < 4; ++j) { qb8[j] = (int)b0[j]; qb8[4 + j] = (int)b1[j]; }
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
                        s[sl][cb][kt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka8[kt], qb8, s[sl][cb][kt], 0, 0, 0, 127, 0, sb);
                }
            }
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int xx = 0; xx < KLD; ++xx)
                    kraw[sl][kt][xx] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + xx * 16, noff + (uint32_t)(kt * 16) * row_stride, 0);
            return;
        }
        half8_t qhi[NCB][KS];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int c = 0; c < KS; ++c)
                qhi[cb][c] = *reinterpret_cast<const half8_t*>(qhi_lds + ((size_t)(g0 + cb) * 16 + n16) * QPITCH + kg * SEG + c * 8);
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            if (with_lo) {
                // K (q - f16(q))^T first: A = the lane's quarter row of K as loaded (32 codes), B = the same quarter of the
                // query's remainder codes, their power of two as the block scale; the f16 products below add to it
                typedef int v8i_t __attribute__((ext_vector_type(8)));
                v8i_t ka8;
#pragma unroll
                for (int j = 0; j < 8; ++j) ka8[j] = (int)kraw[sl][kt][j / 4][j % 4];
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    const uint8_t* qrow = qlo8_lds + ((size_t)(g0 + cb) * 16 + n16) * Q8PITCH + kg * 32;
                    const u32x4 b0 = *reinterpret_cast<const u32x4*>(qrow), b1 = *reinterpret_cast<const u32x4*>(qrow + 16);
                    v8i_t qb8;
#pragma unroll
                    for (int j = 0; j < 4; ++j) { qb8[j] = (int)b0[j]; qb8[4 + j] = (int)b1[j]; }
                    s[sl][cb][kt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka8, qb8, float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 127, 0, 127 + q_exp);
                }
            }
            half8_t ka[KS];
#pragma unroll
            for (int c = 0; c < KS; ++c) {
                const uint32_t w0 = kraw[sl][kt][c / 2][(c % 2) * 2], w1 = kraw[sl][kt][c / 2][(c % 2) * 2 + 1];
                half2_t p0, p1, p2, p3;
                e4m3x4_to_h2(w0, p0, p1);
                e4m3x4_to_h2(w1, p2, p3);
                ka[c][0] = p0[0]; ka[c][1] = p0[1]; ka[c][2] = p1[0]; ka[c][3] = p1[1];
                ka[c][4] = p2[0]; ka[c][5] = p2[1]; ka[c][6] = p3[0]; ka[c][7] = p3[1];
            }
#pragma unroll
            for (int xx = 0; xx < KLD; ++xx)
                kraw[sl][kt][xx] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff + xx * 16, noff + (uint32_t)kt * 16u * row_stride, 0);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                float4_t acc = with_lo ? s[sl][cb][kt] : float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < KS; ++c) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[c], qhi[cb][c], acc, 0, 0, 0);
                s[sl][cb][kt] = acc;
            }
        }
    };
    // scores of the tile in log2 units (this lane owns keys tcur + kt*16 + kg*4 + i of query n16); returns whether one of
    // them exceeds the lane's reference maximum by more than the slack
    auto scores = [&](auto masked_tag, int sl, uint32_t tcur) -> bool {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr bool FOLD = !MASKED && !CAP;                   // scores stay unscaled until the exponent's FMA
        bool moved = false;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            tmax[sl][cb] = kMasked;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float y = FOLD ? s[sl][cb][kt][i] : s[sl][cb][kt][i] * scale_l2;
                    if (CAP) y = cap_l2 * tanhf(y / cap_l2);
                    if (MASKED) {
                        const uint32_t t = tcur + kt * 16 + kg * 4 + i;
                        y = (t < my_len && t >= a.kv_start && t < kmax) ? y : kMasked;    // (t >= kmax: padding tiles of a key chunk)
                    }
                    x[sl][cb][kt * 4 + i] = y;
                    tmax[sl][cb] = fmaxf(tmax[sl][cb], y);
                }
            if (FOLD) tmax[sl][cb] *= scale_l2;
            moved |= tmax[sl][cb] > m_run[cb] + kMaxSlack;
        }
        return moved;
    };
    auto move_maximum = [&](int sl) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            float t = tmax[sl][cb];
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
    // Between the two: the request for the tile after next and the wait for this tile's rows.
    auto weights_and_second_product = [&](auto masked_tag, auto two_tag, int sl, uint32_t tcur) {
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
                    const float xe = x[sl][cb][2 * j2 + e];
                    float pv = __builtin_amdgcn_exp2f(FOLD ? __builtin_fmaf(xe, scale_l2, -m_run[cb]) : xe - m_run[cb]);
                    if (MASKED) pv = xe > -1e29f ? pv : 0.f;
                    pp[e] = pv;
                }
                l_run[cb] += pp[0] + pp[1];
                phi[cb][j2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pp, half2_t));
                if (TWO) plo[cb][j2] = pack_f16_remainder(pp[0], pp[1], phi[cb][j2]);
            }
        stage_v(sl);
        // supplier lane s of a 16-lane group points at the 8 bytes V[key][dt*16 + 8*(s%2) ..], key = 4*kg + s/2 for s < 8
        // and 16 + 4*kg + (s/2 - 4) above; the read hands lane n the bytes of the eight keys at d = dt*16 + n
        const uint32_t vrd = vdma_rd + (uint32_t)(vcur * VBUF);
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");       // this tile's V rows are in LDS
        typedef int v2i_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) {
            const v2i_t raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i_t*)(v8 + (vrd ^ (uint32_t)(dt << 4))));
            half2_t p0, p1, p2, p3;
            e4m3x4_to_h2((uint32_t)raw[0], p0, p1);
            e4m3x4_to_h2((uint32_t)raw[1], p2, p3);
            half8_t va;
            va[0] = p0[0]; va[1] = p0[1]; va[2] = p1[0]; va[3] = p1[1]; va[4] = p2[0]; va[5] = p2[1]; va[6] = p3[0]; va[7] = p3[1];
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
                oacc[cb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, phi[cb]), oacc[cb][dt], 0, 0, 0);
            if (TWO) {
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb)
                    oacc[cb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, __builtin_bit_cast(half8_t, plo[cb]), oacc[cb][dt], 0, 0, 0);
            }
        }
        vcur = vcur == 2 ? 0 : vcur + 1;
    };

    // ---- the wavefront's tiles: the lazy reference maximum and the two loops of batch_mfma2_kernel (an inner one for tiles
    // that every query of the block sees completely, left as soon as a maximum has to move; an outer one for everything
    // else).  The walk is compiled once with and once without the remainder product of Q: without it the first products
    // are straight-line code and the inner loop is the grouped one.
    auto walk = [&](auto lo_tag) {
    constexpr bool GROUP = std::is_same_v<decltype(lo_tag), std::false_type>;   // (with the remainder product in it the two-tile loop spills in both walks)
    int first_slot = 0;          // slots of the group at tb that the inner loop has already finished
    bool s_ready = false;        // the inner loop left the group at tb with scores computed: those of slot first_slot; GROUP:
                                 // those of every slot
    constexpr auto two_tag = std::integral_constant<bool, !F16W>{};
    while (tp[0] < kloop) {
#pragma unroll
        for (int sl = 0; sl < PFD; ++sl) {
            const uint32_t tcur = tp[sl];
            if (tcur >= kloop) break;                           // wavefront-uniform
            if (sl < first_slot) continue;
            if (!(s_ready && (GROUP || sl == first_slot))) first_product(sl, tcur, lo_tag);
            if (tcur >= a.kv_start && tcur + KT <= fast_end) {  // every query of the block sees the whole tile (and it is this workgroup's)
                if (__builtin_amdgcn_ballot_w64(scores(std::false_type{}, sl, tcur)) != 0ull) move_maximum(sl);
                weights_and_second_product(std::false_type{}, two_tag, sl, tcur);
            } else {
                if (__builtin_amdgcn_ballot_w64(scores(std::true_type{}, sl, tcur)) != 0ull) move_maximum(sl);
                weights_and_second_product(std::true_type{}, two_tag, sl, tcur);
            }
        }
        advance();
        first_slot = 0;
        s_ready = false;
        if constexpr (GROUP) {
            // a whole group per pass: the first products of its tiles do not depend on the softmax and the second product of
            // the tiles before them, so the matrix pipe and the vector ALU have work from different tiles side by side
            while (tp[0] >= a.kv_start && tp[PFD - 1] + KT <= fast_end) {
                bool moved = false;
                // the first products issue ahead of the other wavefront's vector work (measured: 2 % of a 32-layer step; the
                // same around the second products, or around the softmax instead, gains nothing, and the FP8 first product
                // loses 1 % with it)
                if constexpr (!F8S) __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int sl = 0; sl < PFD; ++sl) first_product(sl, tp[sl], lo_tag);
                if constexpr (!F8S) __builtin_amdgcn_s_setprio(0);
#pragma unroll
                for (int sl = 0; sl < PFD; ++sl) moved |= scores(std::false_type{}, sl, tp[sl]);
                if (__builtin_amdgcn_ballot_w64(moved) != 0ull) { s_ready = true; break; }
#pragma unroll
                for (int sl = 0; sl < PFD; ++sl) weights_and_second_product(std::false_type{}, two_tag, sl, tp[sl]);
                advance();
            }
        } else {
            bool left = false;
            while (!left && tp[0] >= a.kv_start && tp[PFD - 1] + KT <= fast_end) {
#pragma unroll
                for (int sl = 0; sl < PFD; ++sl) {
                    const uint32_t tcur = tp[sl];
                    first_product(sl, tcur, lo_tag);
                    if (__builtin_amdgcn_ballot_w64(scores(std::false_type{}, sl, tcur)) != 0ull) {
                        first_slot = sl; s_ready = true; left = true;
                        break;
                    }
                    weights_and_second_product(std::false_type{}, two_tag, sl, tcur);
                }
                if (!left) advance();
            }
        }
    }
    };
    if (has_lo) walk(std::true_type{}); else walk(std::false_type{});
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) l_run[cb] = xor32_sum(xor16_sum(l_run[cb]));   // every lane of a query column has its wavefront's sum

    // ---- merge the key splits through LDS, normalise and store: every wavefront leaves its (o, m, l) in LDS, then the NS
    // wavefronts of a head pair each merge and store the d-tiles dt = sp, sp + NS, ... of the pair's NCB heads (gated
    // output, vk_shaders/sigmoid_mul.comp:44-52, applied in that store: a head's D elements lie in one gate chunk).
    // Layout: o as [wavefront slot][cb][dt][lane] float4 (16-byte accesses, consecutive lanes: no bank conflicts), then
    // m and l as [wavefront slot][cb][2][lane].
    if (NS > 1) {
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
        // the gate values of the tiles this wavefront will store are requested here, so that their round trip overlaps the
        // barrier and the merge (tile j of its share is dt = sp + j NS)
        float4 gpre[NCB][DTILES / 2];
        if (a.gate != nullptr && q_ok) {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                if (gz + g0 + cb >= G) continue;
                const uint32_t i0 = (qi * a.n_heads + kvh * G + gz + g0 + cb) * D;
                const uint32_t token = i0 / a.gchunk;
                const float* gp = a.gate + (size_t)token * a.gstride + a.goff + (i0 - token * a.gchunk) + kg * 4;
#pragma unroll
                for (int j = 0; j < DTILES / 2; ++j)
                    if (sp + j * NS < DTILES) gpre[cb][j] = *reinterpret_cast<const float4*>(gp + (sp + j * NS) * 16);
            }
        }
        __syncthreads();
        if (!q_ok) return;
        // (compiled per split count so that the LDS reads of a head are independent instructions, not a chain of round trips)
        auto merge_and_store = [&](auto ns_tag) {
            constexpr int NSC = decltype(ns_tag)::value;
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                if (gz + g0 + cb >= G) continue;                // padding slot of an odd group
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
                const uint32_t h = kvh * G + gz + g0 + cb;
                const size_t pidx = ((size_t)qi * a.n_heads + h) * a.nk + kc;      // (key chunks: the partial of this chunk)
                const float inv = a.so != nullptr ? 1.0f : 1.0f / lsum;
                float* op = a.so != nullptr ? a.so + pidx * D + kg * 4 : a.o + ((size_t)qi * a.n_heads + h) * D + kg * 4;
#pragma unroll
                for (int j = 0; j < DTILES / NSC; ++j) {        // lane (query n16) holds d = dt*16 + kg*4 + i
                    const int dt = sp + j * NSC;
                    float4_t r = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s2 = 0; s2 < NSC; ++s2)
                        r += obuf[((size_t)((s2 * HP + hp) * NCB + cb) * DTILES + dt) * 64 + lane] * f[s2];
                    r *= inv;
                    if (a.gate != nullptr) {
                        const float4 gv = gpre[cb][j];
                        r *= float4_t{sigmoid_gate(1.0f, gv.x), sigmoid_gate(1.0f, gv.y), sigmoid_gate(1.0f, gv.z), sigmoid_gate(1.0f, gv.w)};
                    }
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                if (a.so != nullptr && sp == 0 && kg == 0) {
                    // key chunks: the unnormalised partial in the layout of the decode merge ([row][chunk][D], the maximum
                    // in natural-log units); a query that sees no key of the chunk leaves (0, "minus infinity", 0)
                    a.sm[pidx] = mm > -1e29f ? mm * 0.693147180559945f : kMasked;
                    a.ss[pidx] = lsum;
                }
            }
        };
        if (NS == 4) merge_and_store(std::integral_constant<int, 4>{});
        else if (NS == 2) merge_and_store(std::integral_constant<int, 2>{});
        else merge_and_store(std::integral_constant<int, 8>{});  // (the launcher gives 2, 4 or 8 splits)
        return;
    }
    float4_t gfac[NCB][DTILES];
    if (a.gate != nullptr && q_ok) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            if (gz + g0 + cb >= G) continue;
            const uint32_t i0 = (qi * a.n_heads + kvh * G + gz + g0 + cb) * D;
            const uint32_t token = i0 / a.gchunk;
            const float* gp = a.gate + (size_t)token * a.gstride + a.goff + (i0 - token * a.gchunk) + kg * 4;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const float4 gv = *reinterpret_cast<const float4*>(gp + dt * 16);
                gfac[cb][dt] = float4_t{sigmoid_gate(1.0f, gv.x), sigmoid_gate(1.0f, gv.y), sigmoid_gate(1.0f, gv.z), sigmoid_gate(1.0f, gv.w)};
            }
        }
    }
    if (q_ok) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            if (gz + g0 + cb >= G) continue;                                  // padding slot of an odd group
            const uint32_t h = kvh * G + gz + g0 + cb;
            if (a.so != nullptr) {
                // key chunks: the unnormalised partial of this chunk in the layout of the decode merge ([row][chunk][D], the
                // maximum in natural-log units); a query that sees no key of the chunk leaves (0, "minus infinity", 0)
                const size_t pidx = ((size_t)qi * a.n_heads + h) * a.nk + kc;
                float* op = a.so + pidx * D + kg * 4;
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    const float4_t r = oacc[cb][dt];
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                if (kg == 0) {
                    a.sm[pidx] = m_run[cb] > -1e29f ? m_run[cb] * 0.693147180559945f : kMasked;
                    a.ss[pidx] = l_run[cb];
                }
                continue;
            }
            const float inv = 1.0f / l_run[cb];
            float* op = a.o + ((size_t)qi * a.n_heads + h) * D + kg * 4;   // lane (query n16) holds d = dt*16 + kg*4 + i
            if (a.gate != nullptr) {
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    const float4_t r = oacc[cb][dt] * inv * gfac[cb][dt];
                    *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
                }
                continue;
            }
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                const float4_t r = oacc[cb][dt] * inv;
                *reinterpret_cast<float4*>(op + dt * 16) = make_float4(r[0], r[1], r[2], r[3]);
            }
        }
    }
}


}  // namespace vfkv
