// Chunked-prefill causal attention over the cache (flash_attn_batch.comp:105-208) for gfx950.
//
// batch_mfma2_kernel   (attn_prefill_mfma2.h) f16 matrix-core tiles, private K / V tiles per wavefront: FP8 / F16 caches,
//                      head_dim 64 / 128 / 256 / 512, any GQA group.
// batch_mfma_f32_kernel (attn_prefill_f32.h) f32 matrix-core tiles: F32 caches (head_dim 64 / 128 / 256 / 512 and the multiples of
//                      16 in between); FP8 / F16 caches of those in-between widths run on batch_mfma2_kernel's padded form.
// batch_generic_kernel one wavefront per (query, head); covers every dtype and head_dim <= 512.
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
    // key chunks over workgroups (f16 matrix-core kernel only): workgroup z handles keys [kc * chunk, (kc + 1) * chunk) and
    // stores an unnormalised partial (o, m, l) per (query, head, chunk) for the decode merge kernel; so == NULL: off
    float* so;
    float* sm;
    float* ss;
    uint32_t nk, chunk;
    // gated output (f16 matrix-core kernel only, and only when it stores final values): o *= sigmoid(gate[...]) in the
    // kernel's own store; gate == NULL: off.  The launcher guarantees gchunk % head_dim == 0, gchunk, gstride and goff
    // multiples of 4, a 16-byte aligned gate and fewer than 2^32 output elements.
    const float* gate;
    uint32_t gchunk, gstride, goff;
    uint32_t q_f16;          // f16 matrix-core kernels: use f16(q) alone, whatever the queries hold
    uint32_t merge_all;      // batch_mfma2_kernel: the LDS area holds the (o, m, l) of every wavefront, and every wavefront merges a share
    uint32_t xcd_heads;      // batch_mfma2_kernel: deal the (KV head, query block) pairs so that an XCD works on one KV head at a time
};

}  // namespace vfkv
#include "attn_prefill_mfma2.h"
#include "attn_prefill_dma.h"
#include "attn_prefill_f32.h"
namespace vfkv {

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

// Launches the attention kernel(s) for L.  *gate_applied tells whether L.gate went into their stores.
static hipError_t launch_batch_kernels(const BatchLaunch& L, hipStream_t stream, bool* gate_applied, bool* generic_used) {
    *gate_applied = false;
    BatchArgs a;
    a.q = L.q; a.k = (const uint8_t*)L.k; a.v = (const uint8_t*)L.v; a.o = L.o;
    a.n_heads = L.n_heads; a.n_kv_heads = L.n_kv_heads; a.head_dim = L.head_dim;
    a.m = L.m; a.n_kv = L.n_kv; a.q_start = L.q_start; a.kv_start = L.kv_start;
    a.scale = L.scale; a.softcap = L.softcap; a.dtype = L.dtype;
    a.so = nullptr; a.sm = nullptr; a.ss = nullptr; a.nk = 1u; a.chunk = 0u;
    a.gate = nullptr; a.gchunk = 1u; a.gstride = 0u; a.goff = 0u;
    a.q_f16 = L.f16_queries ? 1u : 0u;
    a.merge_all = 0u;
    a.xcd_heads = 0u;
    const uint32_t g = L.n_heads / L.n_kv_heads;
    const uint64_t slab_bytes = (uint64_t)L.n_kv * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.o)) & 15u) == 0u;
    // Head widths between the tiled ones (80 / 96 / 112, 160 / 192 / 224) run on the next wider instantiation of the f16
    // kernel with its tail masked off (PAD): hd is the width of the kernel, L.head_dim what the buffers hold.
    const uint32_t dpad = split_padded_dim(L.dtype, L.head_dim);
    const uint32_t hd = dpad != 0u ? dpad : L.head_dim;
    const bool mfma_ok = (L.dtype == kF8 || L.dtype == kF16) && aligned && slab_bytes < 0x7FFF0000ull &&
                         (hd == 64u || hd == 128u || hd == 256u || hd == 512u);
    // f16 matrix-core kernel: NCB heads per wavefront, private tiles per wavefront, no barrier in the loop
    if (mfma_ok) {
        // head_dim 512: one head per wavefront, and two wavefronts share a head (each owns half of the output columns)
        // (also FP8 rows of 256 elements without grouping: 8 / 8 / 256, 512 queries over 4 608 keys, 76.3 us with two query
        // blocks per wavefront, 56.4 us with two wavefronts per head; every grouped shape and F16 rows measured slower so:
        // 16 / 8 / 256 FP8 87 -> 100 us, F16 105 -> 120 us)
        const uint32_t nh = hd == 512u ? 2u : (hd == 256u && dpad == 0u && L.dtype == kF8 && g == 1u) ? 2u : 1u;
        // Heads per wavefront.  Two where the registers allow it (a K / V tile is then converted once for both); odd groups
        // of three and more heads round up, the spare slot computes on zeros and stores nothing.  Where the rows are wide
        // (F16 at head_dim 128, everything at head_dim 256) the traffic between L2 and the CUs is what binds: four / two heads
        // per wavefront in workgroups of four wavefronts (one per SIMD, up to 512 registers), so that a K / V tile is loaded
        // by one wavefront of the workgroup only.
        uint32_t ncb = 1u;
        // Groups of one head (no grouping): two blocks of 16 queries of the same head per wavefront instead of two heads, so
        // that a K / V tile is still widened and staged once for two column blocks; a workgroup then covers 32 queries.
        const bool qb2 = g == 1u && nh == 1u && L.m > 16u;
        if (qb2) ncb = 2u;
        if (g >= 2u) {
            // head_dim 512: a second head per wavefront only for FP8 rows (F16 rows leave no registers for it) and only while
            // head pairs still give every compute unit a workgroup
            if (nh == 2u) ncb = (L.dtype == kF8 && (uint64_t)((L.m + 15u) / 16u) * L.n_kv_heads * ((g + 1u) / 2u) >= 256u) ? 2u : 1u;
            else if (hd == 128u && L.dtype == kF16 && g >= 3u && dpad == 0u) ncb = 4u;   // (the padded form of it crashes the compiler's AGPR rewriting pass)
            else ncb = 2u;
        }
        const uint32_t dv = hd / nh;
        const uint32_t hp_group = qb2 ? 1u : (g + ncb - 1u) / ncb * nh;     // (head slice, output slice) units of a whole GQA group
        const uint32_t qblocks = qb2 ? (L.m + 31u) / 32u : (L.m + 15u) / 16u;   // query blocks = workgroups per (KV head, head slice)
        // wavefronts per workgroup the registers allow: one head per wavefront at head_dim <= 128 needs few (three wavefronts
        // per SIMD), 512 accumulator columns per wavefront need the whole register file of a SIMD (one wavefront per SIMD)
        const uint32_t reg_waves = (ncb == 1u && hd <= 128u) ? (uint32_t)kPrefillOneHeadWaves : (hd == 256u && nh == 2u) ? 8u
                                 : (ncb * hd >= 512u || (L.dtype == kF16 && hd == 256u)) ? 4u : 8u;   // (always 4 at head_dim 512)
        // FP8 rows of 128 elements, two heads per wavefront: three raw V tiles per wavefront (filled by loads that write LDS)
        // instead of one f16 copy
        const bool vdma = L.dtype == kF8 && L.head_dim == 128u && ncb == 2u && !qb2;      // (not the padded widths)
        // the private V tiles and the two Q planes have to fit in 160 KiB of LDS
        auto waves_for = [&](uint32_t slices) -> uint32_t {
            const size_t qbytes = (size_t)2 * (slices / nh) * ncb * 16 * (hd + 8) * sizeof(_Float16) +
                                  (vdma ? (size_t)slices * ncb * 16 * (hd + 16) : 0u);   // (that kernel: a third plane of one byte per element)
            // private V tile, and with two wavefronts per head the two buffers through which they swap score halves
            const size_t per_wave = (vdma ? (size_t)3 * 32 * 128 : (size_t)32 * (dv + 16) * sizeof(_Float16)) +
                                    (nh == 2u ? (size_t)2 * ncb * 64 * 16 : 0u);   // (unused by the two-heads FP8 form)
            const size_t fit = qbytes < 160u * 1024u ? (160u * 1024u - qbytes) / per_wave : 0u;
            return fit < reg_waves ? (uint32_t)fit : reg_waves;
        };
        // Head slices per workgroup: the whole group where it fits; launches that would leave compute units without a
        // workgroup, and groups whose Q planes or wavefronts do not fit one workgroup, spread the slices of a group over
        // several workgroups (each then splits the keys further: same work per workgroup, more of them).
        uint32_t hp = hp_group;
        {
            const uint64_t wgs = (uint64_t)qblocks * L.n_kv_heads;
            if (wgs < 256u) {
                uint32_t want = (uint32_t)((256u + wgs - 1u) / wgs);
                if (want > hp_group / nh) want = hp_group / nh;
                hp = (hp_group / nh + want - 1u) / want * nh;    // the output slices of a head stay in one workgroup
            }
            while (hp > nh && waves_for(hp) < hp) hp -= nh;      // one head always fits
            // the V-through-LDS kernel runs best as two head pairs x four key splits (two wavefronts per SIMD, mirrored query
            // blocks, the uneven deal): a group of four head pairs becomes two such workgroups instead of one workgroup of
            // four wavefronts that each walk every key (512 queries over 4 608 keys, 64 / 8 / 128: 133.7 -> 120.0 us; 128 / 8 / 128: 352 -> 233 us)
            if (vdma && hp > 2u && hp_group % 2u == 0u) hp = 2u;
        }
        const uint32_t nz = (hp_group + hp - 1u) / hp;
        const uint32_t max_waves = waves_for(hp);
        if (max_waves >= hp && nz <= 65535u && qblocks <= 65535u) {
            uint32_t ns = max_waves / hp;                     // key splits: fill the workgroup
            if (vdma) while (ns & (ns - 1u)) --ns;            // (that kernel's merge deals the 8 output tiles of a head to the splits)
            const uint32_t nwaves = hp * ns;
            // Short chunks over long histories (the suffix of a request that reuses its prefix) still leave most compute
            // units idle: with a workspace the keys are also cut into chunks over workgroups, every workgroup stores a
            // partial per (query, head, chunk), and the decode merge kernel combines them.
            uint32_t nk = 1u;
            if (L.scratch_out != nullptr && L.n_heads != 0u) {
                const uint64_t wgs = (uint64_t)qblocks * L.n_kv_heads * nz;
                const uint32_t t0 = (L.kv_start / 32u) * 32u;
                const uint32_t kend = L.q_start + L.m < L.n_kv ? L.q_start + L.m : L.n_kv;
                const uint32_t span = kend > t0 ? kend - t0 : 0u;
                if (wgs < 192u && span >= 1024u) {
                    nk = (uint32_t)((256u + wgs - 1u) / wgs);
                    if (nk > span / 512u) nk = span / 512u;   // at least 512 keys per chunk
                    if (nk > 32u) nk = 32u;
                    const uint64_t rows = (uint64_t)L.m * L.n_heads;
                    while (nk > 1u && (rows * nk * L.head_dim > L.scratch_out_floats || rows * nk > L.scratch_ml_floats)) --nk;
                    if (rows > 65535u) nk = 1u;               // rows are a grid dimension of the merge launch
                }
                if (nk > 1u) {
                    a.so = L.scratch_out; a.sm = L.scratch_max; a.ss = L.scratch_sum; a.nk = nk;
                    a.chunk = ((span + nk - 1u) / nk + 31u) / 32u * 32u;
                }
            }
            // the gate goes into the kernel's store when a lane's four output elements share a chunk and a 16-byte gate
            // load, and a head's elements share a chunk; with key chunks the merge applies it instead
            const bool gate_in_store = L.gate != nullptr && nk == 1u && L.gate->chunk % L.head_dim == 0u &&
                                       ((L.gate->chunk | L.gate->stride | L.gate->gate_offset) % 4u) == 0u &&
                                       (((uintptr_t)L.gate->gate) & 15u) == 0u;
            if (gate_in_store) { a.gate = L.gate->gate; a.gchunk = L.gate->chunk; a.gstride = L.gate->stride; a.goff = L.gate->gate_offset; }
            // the KV head is the fastest grid index: consecutive workgroups go to consecutive XCDs, so with eight KV heads all
            // query blocks of a head share one XCD's L2 and its K / V rows come from memory once, not once per XCD
            // With more than eight KV heads that order gives every XCD several heads at once, whose K / V rows then compete
            // for its L2 (32 KV heads of 2.4 MB each: 320 MB fetched per launch for 57 MB of rows); the kernel then renumbers
            // its workgroups so that an XCD takes all query blocks of one head before the next head.  512 queries over 4 608
            // keys, 32 / 32 heads: FP8 rows of 96 / 128 elements 141.7 -> 129.1 / 119.0 -> 117.9 us; F16 rows did not gain
            // (96: 190.9 -> 191.7, 128: 199.5 -> 211.4 us) and keep the plain order.
            a.xcd_heads = (L.dtype == kF8 && L.n_kv_heads > 8u && L.n_kv_heads % 8u == 0u) ? 1u : 0u;
            const dim3 grid(L.n_kv_heads, qblocks, nz * nk), block(nwaves * kWave);
            const size_t vbytes = (size_t)nwaves * (vdma ? (size_t)3 * 32 * 128 : (size_t)32 * (dv + 16) * sizeof(_Float16)) +
                                  (size_t)2 * (hp / nh) * ncb * 16 * (hd + 8) * sizeof(_Float16) +
                                  (vdma ? (size_t)hp * ncb * 16 * (hd + 16) : 0u) +
                                  (nh == 2u ? (size_t)2 * nwaves * ncb * 64 * 16 : 0u);
            // merge area: the general kernel keeps the records of all splits but the first; the V-through-LDS kernel the
            // output tiles and (m, l) of every wavefront
            const size_t mbytes_all = (size_t)nwaves * ncb * 64 * (dv / 4 + 2) * sizeof(float);
            a.merge_all = (!vdma && nh == 1u && mbytes_all + 64u <= 160u * 1024u) ? 1u : 0u;
            const size_t mbytes = (vdma || a.merge_all) ? mbytes_all : (size_t)(ns - 1) * hp * ncb * 64 * (dv / 4 + 2) * sizeof(float);
            const size_t lds = vbytes > mbytes ? vbytes : mbytes;
            const bool cap = L.softcap > 0.f;
            bool launched = true;
#define VFKV_P2(DT, DD, NCBV, PFDV)                                                                         \
    if (L.dtype == DT && L.head_dim == DD && ncb == NCBV) {                                                 \
        if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, NCBV, PFDV, true>), grid, block, lds, stream, a, (int)hp, (int)ns);  \
        else hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, NCBV, PFDV, false>), grid, block, lds, stream, a, (int)hp, (int)ns);      \
    } else
#define VFKV_P2PAD(DT, DD, NCBV, PFDV)                                                                      \
    if (L.dtype == DT && dpad == DD && ncb == NCBV) {                                                       \
        if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, NCBV, PFDV, true, 1, false, true>), grid, block, lds, stream, a, (int)hp, (int)ns);  \
        else hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, NCBV, PFDV, false, 1, false, true>), grid, block, lds, stream, a, (int)hp, (int)ns);      \
    } else
            // FP8 rows of 128 elements, two heads per wavefront: the kernel that loads V straight into LDS.  Its options --
            // f16_weights: one product with the weights instead of value + remainder; fp8_scores: the first product on the
            // FP8 matrix instruction (needs the Q block staged in one round: four key splits).  Over F16 rows (four heads per
            // wavefront) f16_weights is an instantiation of the general kernel; other shapes keep the default arithmetic.
            const bool f8s = L.fp8_scores && vdma && ns >= 4u;
            // eight wavefronts (two per SIMD) and an even number of key splits: the older wavefront of a SIMD gets 3 tiles
            // for every 2 of the younger one
            int deal_a = 1, deal_b = 1;
            if (nwaves == 8u && ns % 2u == 0u) { deal_a = 3; deal_b = 2; }
#define VFKV_PDMA(F16WV, F8SV)                                                                                         \
    { if (cap) hipLaunchKernelGGL((batch_dma_kernel<true, F16WV, F8SV>), grid, block, lds, stream, a, (int)hp, (int)ns, deal_a, deal_b);  \
      else hipLaunchKernelGGL((batch_dma_kernel<false, F16WV, F8SV>), grid, block, lds, stream, a, (int)hp, (int)ns, deal_a, deal_b); }
            if (vdma && f8s && L.f16_weights) VFKV_PDMA(true, true)
            else if (vdma && f8s) VFKV_PDMA(false, true)
            else if (vdma && L.f16_weights) VFKV_PDMA(true, false)
            else if (vdma) VFKV_PDMA(false, false)
#undef VFKV_PDMA
            else
#define VFKV_P2QB(DT, DD, PFDV, PADV)                                                                       \
    if (qb2 && L.dtype == DT && hd == DD && (dpad != 0u) == PADV) {                                         \
        if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, 2, PFDV, true, 1, false, PADV, true>), grid, block, lds, stream, a, (int)hp, (int)ns);  \
        else hipLaunchKernelGGL((batch_mfma2_kernel<DT, DD, 2, PFDV, false, 1, false, PADV, true>), grid, block, lds, stream, a, (int)hp, (int)ns);      \
    } else
            VFKV_P2QB(kF8, 64, 2, false) VFKV_P2QB(kF16, 64, 2, false) VFKV_P2QB(kF8, 128, 2, false) VFKV_P2QB(kF16, 128, 1, false)
            VFKV_P2QB(kF8, 256, 1, false) VFKV_P2QB(kF16, 256, 1, false)
            VFKV_P2QB(kF8, 128, 2, true) VFKV_P2QB(kF16, 128, 1, true) VFKV_P2QB(kF8, 256, 1, true) VFKV_P2QB(kF16, 256, 1, true)
#undef VFKV_P2QB
            if (hd == 256u && nh == 2u) {
                if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 256, 1, 1, true, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
                else hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 256, 1, 1, false, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
            } else
            if (L.f16_weights && L.dtype == kF16 && L.head_dim == 128u && ncb == 4u) {
                if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<kF16, 128, 4, 1, true, 1, true>), grid, block, lds, stream, a, (int)hp, (int)ns);
                else hipLaunchKernelGGL((batch_mfma2_kernel<kF16, 128, 4, 1, false, 1, true>), grid, block, lds, stream, a, (int)hp, (int)ns);
            } else
            VFKV_P2(kF8, 64, 2, 2) VFKV_P2(kF8, 64, 1, 2) VFKV_P2(kF8, 128, 1, 2)
            VFKV_P2(kF16, 64, 2, 2) VFKV_P2(kF16, 64, 1, 2) VFKV_P2(kF16, 128, 1, 1) VFKV_P2(kF16, 128, 2, 1)
            VFKV_P2(kF8, 256, 1, 1) VFKV_P2(kF16, 256, 1, 1)
            VFKV_P2(kF16, 128, 4, 1) VFKV_P2(kF8, 256, 2, 1) VFKV_P2(kF16, 256, 2, 1)
            VFKV_P2PAD(kF8, 128, 1, 2) VFKV_P2PAD(kF8, 128, 2, 2) VFKV_P2PAD(kF16, 128, 1, 1) VFKV_P2PAD(kF16, 128, 2, 1)
            VFKV_P2PAD(kF8, 256, 1, 1) VFKV_P2PAD(kF8, 256, 2, 1) VFKV_P2PAD(kF16, 256, 1, 1) VFKV_P2PAD(kF16, 256, 2, 1)
            if (L.head_dim == 512u && L.dtype == kF8 && ncb == 2u) {
                if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 512, 2, 1, true, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
                else hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 512, 2, 1, false, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
            } else if (L.head_dim == 512u && L.dtype == kF8) {
                if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 512, 1, 1, true, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
                else hipLaunchKernelGGL((batch_mfma2_kernel<kF8, 512, 1, 1, false, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
            } else if (L.head_dim == 512u && L.dtype == kF16) {
                if (cap) hipLaunchKernelGGL((batch_mfma2_kernel<kF16, 512, 1, 1, true, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
                else hipLaunchKernelGGL((batch_mfma2_kernel<kF16, 512, 1, 1, false, 2>), grid, block, lds, stream, a, (int)hp, (int)ns);
            } else
            { launched = false; }
#undef VFKV_P2
#undef VFKV_P2PAD
            if (launched) {
                hipError_t e = hipGetLastError();
                if (e == hipSuccess && nk > 1u)
                    e = launch_reduce(a.so, a.sm, a.ss, L.o, L.m * L.n_heads, L.head_dim, nk, stream, L.gate, gate_applied);
                else
                    *gate_applied = gate_in_store;
                return e;
            }
            a.so = nullptr; a.nk = 1u; a.gate = nullptr;
        }
    }
    // f32 matrix-core kernel: F32 caches, and the head sizes the f16 kernels above do not cover
    if (aligned && slab_bytes < 0x7FFF0000ull && L.n_kv_heads <= 65535u && (g + 3u) / 4u * 2u <= 65535u) {
        const bool cap = L.softcap > 0.f;
#define VFKV_PF32(DTV, DD, NHV)                                                                                        \
    if (L.dtype == DTV && L.head_dim == DD) {                                                                          \
        const dim3 grid((L.m + 15u) / 16u, L.n_kv_heads, (g + 3u) / 4u * NHV), block(256);                             \
        if (cap) hipLaunchKernelGGL((batch_mfma_f32_kernel<DTV, DD, NHV, true>), grid, block, 0, stream, a);           \
        else hipLaunchKernelGGL((batch_mfma_f32_kernel<DTV, DD, NHV, false>), grid, block, 0, stream, a);              \
        return hipGetLastError();                                                                                      \
    }
        VFKV_PF32(kF32, 64, 1) VFKV_PF32(kF32, 128, 1) VFKV_PF32(kF32, 256, 1) VFKV_PF32(kF32, 96, 1)
        VFKV_PF32(kF16, 96, 1) VFKV_PF32(kF8, 96, 1) VFKV_PF32(kF32, 512, 2)
        // the other head widths between the tiled ones over F32 caches (FP8 / F16 caches take the f16 kernel's padded form)
        VFKV_PF32(kF32, 80, 1) VFKV_PF32(kF32, 112, 1) VFKV_PF32(kF32, 160, 1) VFKV_PF32(kF32, 192, 1) VFKV_PF32(kF32, 224, 1)
#undef VFKV_PF32
    }
    if (generic_used) *generic_used = true;
    hipLaunchKernelGGL(batch_generic_kernel, dim3(L.n_heads, L.m), dim3(kWave), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_batch(const BatchLaunch& L, hipStream_t stream, bool* generic_used) {
    if (generic_used) *generic_used = false;
    if (L.dtype > kF8 || L.head_dim == 0u || L.head_dim > 512u) return hipErrorInvalidValue;
    if (L.m == 0u) return hipSuccess;
    const uint64_t ne = (uint64_t)L.m * L.n_heads * L.head_dim;
    if (L.gate != nullptr && (L.gate->gate == nullptr || L.gate->chunk == 0u || ne > 0xFFFFFFFFull)) return hipErrorInvalidValue;
    bool gate_applied = false;
    hipError_t e = launch_batch_kernels(L, stream, &gate_applied, generic_used);
    if (e == hipSuccess && L.gate != nullptr && !gate_applied) e = launch_sigmoid_mul(L.o, (uint32_t)ne, *L.gate, stream);
    return e;
}

}  // namespace vfkv
