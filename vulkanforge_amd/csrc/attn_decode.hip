// Split-K decode attention for gfx950: worker (flash_attn_split.comp:82-162) and log-sum-exp
// merge (flash_attn_reduce.comp:35-81), re-designed around the HBM stream.
//
//   split_mfma_kernel    (attn_decode_mfma.h) matrix-core worker: FP8 / F16 caches, head_dim 64 / 128 / 256 / 512, and the
//                        multiples of 16 in between on the next wider instantiation with its tail masked off
//   split_mfma_il_kernel (attn_decode_il.h) the same arithmetic with the runs of the whole span dealt to the workgroups:
//                        head_dim 64 / 128 / 256, the kernel every benchmark configuration runs on
//   split_kernel         vector-ALU worker described below: F32 caches (and every shape under VFKV_DECODE_WORKER=valu)
//   split_generic_kernel one wavefront per (head, tile), any dtype, head_dim <= 512
//   reduce_direct_kernel merge of up to 64 partials per head without LDS; reduce_kernel / reduce_generic_kernel beyond
//
// Vector-ALU worker.  One workgroup (NW wavefronts) owns one (tile of keys, KV head, group of GT query heads);
// every K / V byte of the tile is requested from memory once and serves all GT heads of the GQA
// group.  Each wavefront walks its share of the tile in runs of 64 rows:
//
//   K phase   LPRK lanes x 16 B cover a row, so one load instruction fetches 64/LPRK whole rows.
//             Each lane keeps its 16-byte slice of Q for the GT heads in registers as f16 pairs,
//             multiplies with v_dot2_f32_f16 (products of two f16 values are exact in f32) and the
//             lanes of a row combine their partial sums with DPP butterflies.  The row's GT scores
//             go to LDS.  When Q is not exactly representable in f16 the run is swept a second time
//             with the rounding remainders of Q, which restores f32 accuracy.
//   softmax   one lane per row: scale, optional soft-cap, mask, wavefront maximum through DPP row
//             broadcasts, one exp2 per score; the weights go back to LDS.
//   V phase   LPRV lanes x VB bytes cover a row; every lane accumulates GT x VE outputs in f32.
//
// K and V rows travel through two small register rings that are refilled immediately after use
// with the rows needed one ring-length later (of this run or of the wavefront's next run), so the
// loads of one phase are in flight during the other.  Loads are raw buffer loads whose descriptor
// ends at the last populated row: rows past it read as zero without touching memory, which is also
// how the ring is "refilled" when there is no next run.
#include <cstdio>
#include <cstdlib>
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
    float* o_direct;      // optional, single-tile launches of the matrix-core worker: final output [n_heads][D], no partials
    const float* k_new;   // optional: one token row [n_kv_heads * D] f32 to append at row `append_pos` first (matrix-core worker)
    const float* v_new;
    uint32_t append_pos;
    uint32_t n_heads, n_kv_heads;
    uint32_t seq_len, kv_start;
    uint32_t tile, tile_first, n_tiles;
    uint32_t group;          // n_heads / n_kv_heads
    uint32_t interleave;     // matrix-core worker: deal the runs of the launched span round-robin instead of by tile
    float scale, softcap;
};

template <int DT>
struct ElemBytes { static constexpr int value = DT == kF32 ? 4 : DT == kF16 ? 2 : 1; };

template <int GT> struct RowVec;
template <> struct RowVec<4> { typedef float4_t T; };
template <> struct RowVec<2> { typedef float2_t T; };
template <> struct RowVec<1> { typedef float T; };
template <int GT> __device__ __forceinline__ float rv_get(const typename RowVec<GT>::T& v, int g) { return v[g]; }
template <> __device__ __forceinline__ float rv_get<1>(const float& v, int) { return v; }
template <int GT> __device__ __forceinline__ void rv_set(typename RowVec<GT>::T& v, int g, float x) { v[g] = x; }
template <> __device__ __forceinline__ void rv_set<1>(float& v, int, float x) { v = x; }

constexpr uint32_t kOOB = 0x80000000u;   // byte offset beyond any slab (slabs are < 2 GiB): the buffer load returns zeros, no memory access
constexpr int kRun = 64;                 // rows per run: one softmax row per lane

template <int DT, int D, int GT, int NW, bool CAP>
__global__ __launch_bounds__(NW * 64) void split_kernel(SplitArgs a) {
  constexpr int ES = ElemBytes<DT>::value;
  constexpr int KE = 16 / ES;
  constexpr int QR = DT == kF32 ? KE : KE / 2;
  constexpr int LPRK = D / KE, RPK = 64 / LPRK, KI = kRun / RPK;     // K loads per run
  constexpr int VB0 = (ES == 1 && GT > 2) ? 8 : 16;          // keeps GT x VE accumulators at <= 32 registers
  constexpr int VB = (D * ES / VB0 < 8) ? D * ES / 8 : VB0;    // at least 8 lanes per V row
  constexpr int VE = VB / ES;
  constexpr int LPRV = D * ES / VB, RPV = 64 / LPRV, VI = kRun / RPV;  // V loads per run
  constexpr int PFK = KI < 8 ? KI : 8;                                // registers in the K ring
  constexpr int PFV = VB == 8 ? (VI < 16 ? VI : 16) : (VI < 8 ? VI : 8);
  constexpr bool SPLITQ = DT != kF32;
  static_assert(LPRK >= 4 && LPRK <= 64 && LPRV >= 8 && LPRV <= 64, "unsupported row shape");
  static_assert(KI % PFK == 0 && VI % PFV == 0, "rings must tile a run");
  typedef typename RowVec<GT>::T rowvec_t;

  __shared__ rowvec_t lds_s[NW][kRun];
  constexpr int QN = SPLITQ ? D / 2 : D;
  __shared__ uint32_t lds_q[2][GT][QN];
  __shared__ float lds_o[NW][GT][D];
  __shared__ float lds_m[NW][GT], lds_l[NW][GT];
  __shared__ int lds_haslo;

  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ck = lane % LPRK, rk = lane / LPRK;
  const int cv = lane % LPRV, rv = lane / LPRV;
  const uint32_t jl = blockIdx.x, kvh = blockIdx.y;
  const uint32_t h0 = kvh * (a.n_heads / a.n_kv_heads) + blockIdx.z * GT;
  const uint32_t tile_base = (a.tile_first + jl) * a.tile;
  uint32_t tile_end = tile_base + a.tile; if (tile_end > a.seq_len) tile_end = a.seq_len;
  const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;

  float m_run[GT], l_run[GT], acc[GT][VE];
#pragma unroll
  for (int g = 0; g < GT; ++g) { m_run[g] = kMasked; l_run[g] = 0.f;
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[g][e] = 0.f; }

  const uint32_t row_stride = a.n_kv_heads * D * ES;
  const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.k, 0, a.seq_len * row_stride, 0x00020000);
  const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)a.v, 0, a.seq_len * row_stride, 0x00020000);
  const uint32_t lane_koff = rk * row_stride + kvh * D * ES + ck * 16;
  const uint32_t lane_voff = rv * row_stride + kvh * D * ES + cv * VB;
  const float scale_l2 = a.scale * 1.44269504088896f;
  const float cap_l2 = a.softcap * 1.44269504088896f;

  // runs of this wavefront: w, w + NW, ... counted from the first run that reaches the window
  const uint32_t first_run = (lo - tile_base) / kRun;
  const uint32_t n_runs = tile_end > tile_base ? (tile_end - tile_base + kRun - 1) / kRun : 0;
  auto run_off = [&](uint32_t r) -> uint32_t {   // byte offset of a run's first row, or out of bounds when there is none
    return r < n_runs ? (tile_base + r * kRun) * row_stride : kOOB;
  };

  u32x4 kreg[PFK];
  u32x4 vreg4[VB == 16 ? PFV : 1];
  u32x2 vreg2[VB == 8 ? PFV : 1];
  // lane part in the VGPR offset, uniform part in the scalar offset; the range check covers their sum
  auto issue_k = [&](int j, uint32_t off) { kreg[j] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, lane_koff, off, 0); };
  auto issue_v = [&](int j, uint32_t off) {
    if (VB == 16) vreg4[j] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, lane_voff, off, 0);
    else vreg2[j] = __builtin_amdgcn_raw_buffer_load_b64(vrsrc, lane_voff, off, 0);
  };

  uint32_t r = first_run + w;
  const bool active = lo < tile_end && r < n_runs;
  {   // fill both rings first: these loads do not depend on Q and fly while Q is staged
    const uint32_t off = active ? run_off(r) : kOOB;
#pragma unroll
    for (int j = 0; j < PFK; ++j) issue_k(j, off + (uint32_t)(j * RPK) * row_stride);
#pragma unroll
    for (int j = 0; j < PFV; ++j) issue_v(j, off + (uint32_t)(j * RPV) * row_stride);
  }

  // ---- Q -> LDS once per workgroup ----
  if (tid == 0) lds_haslo = 0;
  __syncthreads();
  {
    bool any_lo = false;
    if (SPLITQ) {
      for (int idx = tid; idx < GT * D / 2; idx += NW * 64) {
        const int g = idx / (D / 2), pr = idx % (D / 2);
        const float2 f = *reinterpret_cast<const float2*>(a.q + (size_t)(h0 + g) * D + 2 * pr);
        const _Float16 hx = (_Float16)f.x, hy = (_Float16)f.y;
        const _Float16 lx = (_Float16)(f.x - (float)hx), ly = (_Float16)(f.y - (float)hy);
        lds_q[0][g][pr] = __builtin_bit_cast(uint32_t, half2_t{hx, hy});
        lds_q[1][g][pr] = __builtin_bit_cast(uint32_t, half2_t{lx, ly});
        any_lo |= (lx != (_Float16)0) | (ly != (_Float16)0);
      }
      if (any_lo) lds_haslo = 1;
    } else {
      for (int idx = tid; idx < GT * D; idx += NW * 64) {
        const int g = idx / D, d = idx % D;
        lds_q[0][g][d] = __builtin_bit_cast(uint32_t, a.q[(size_t)(h0 + g) * D + d]);
      }
    }
  }
  __syncthreads();
  const int npass = (SPLITQ && __builtin_amdgcn_readfirstlane(lds_haslo) != 0) ? 2 : 1;
  uint32_t qh[GT][QR];
  auto load_q = [&](int part) {
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
      for (int j = 0; j < QR; ++j) qh[g][j] = lds_q[part][g][ck * QR + j];
  };
  load_q(0);

  if (active) {
    for (; r < n_runs; r += NW) {
      const uint32_t off = run_off(r), noff = run_off(r + NW);
      const uint32_t rb = tile_base + r * kRun;
      // ---------------- K phase ----------------
      // (vector elements are copied to scalars before __builtin_bit_cast: bit-casting the element
      // expression directly was observed to read element 0)
      auto dot = [&](int j, float (&s)[GT]) {
        if (DT == kF8) {
          half2_t kh[8];
#pragma unroll
          for (int x = 0; x < 4; ++x) e4m3x4_to_h2(kreg[j][x], kh[2 * x], kh[2 * x + 1]);
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            float d2 = 0.f;
#pragma unroll
            for (int x = 0; x < 8; ++x) d2 = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, qh[g][x % QR]), kh[x], d2, false);
            s[g] = d2;
          }
        } else if (DT == kF16) {
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            float d2 = 0.f;
#pragma unroll
            for (int x = 0; x < 4; ++x) { const uint32_t kw = kreg[j][x]; d2 = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, qh[g][x % QR]), __builtin_bit_cast(half2_t, kw), d2, false); }
            s[g] = d2;
          }
        } else {
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            float d2 = 0.f;
#pragma unroll
            for (int x = 0; x < 4; ++x) { const uint32_t kw = kreg[j][x]; d2 = fmaf(__builtin_bit_cast(float, qh[g][x % QR]), __builtin_bit_cast(float, kw), d2); }
            s[g] = d2;
          }
        }
      };
      auto put_scores = [&](int i, float (&s)[GT], bool accumulate) {
        rowvec_t sv;
#pragma unroll
        for (int g = 0; g < GT; ++g) rv_set<GT>(sv, g, group_sum<LPRK>(s[g]));
        if (ck == 0) {
          if (accumulate) { rowvec_t old = lds_s[w][i * RPK + rk]; lds_s[w][i * RPK + rk] = old + sv; }
          else lds_s[w][i * RPK + rk] = sv;
        }
      };
      // Q = hi + lo (only when some lo != 0): the run is swept once per part, Q swapped through LDS; the
      // second sweep re-reads the same K rows (cache hits) through the same ring.
#pragma unroll 1
      for (int pass = 0; pass < npass; ++pass) {
        if (npass == 2) load_q(pass);
        const uint32_t wrap = (pass + 1 < npass) ? off : noff;
#pragma unroll
        for (int i = 0; i < KI; ++i) {
          float s[GT];
          dot(i % PFK, s);
          issue_k(i % PFK, i + PFK < KI ? off + (uint32_t)((i + PFK) * RPK) * row_stride : wrap + (uint32_t)((i + PFK - KI) * RPK) * row_stride);
          put_scores(i, s, pass > 0);
        }
      }
      if (npass == 2) load_q(0);
      __builtin_amdgcn_wave_barrier();
      // ---------------- softmax: lane = row ----------------
      {
        const uint32_t t = rb + lane;
        const bool valid = t < tile_end && t >= lo;
        rowvec_t sv = lds_s[w][lane];
        float x[GT];
        bool changed = false;
        float mnew[GT];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          float y = rv_get<GT>(sv, g) * scale_l2;
          if (CAP) y = cap_l2 * tanhf(y / cap_l2);
          y = valid ? y : kMasked;
          x[g] = y;
          mnew[g] = fmaxf(m_run[g], wave_max_uniform(y));
          changed |= mnew[g] > m_run[g];
        }
        if (changed) {
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            const float alpha = exp2f(m_run[g] - mnew[g]);
            l_run[g] *= alpha;
#pragma unroll
            for (int e = 0; e < VE; ++e) acc[g][e] *= alpha;
            m_run[g] = mnew[g];
          }
        }
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          const float p = valid ? exp2f(x[g] - m_run[g]) : 0.f;
          l_run[g] += p;
          rv_set<GT>(sv, g, p);
        }
        lds_s[w][lane] = sv;
      }
      __builtin_amdgcn_wave_barrier();
      // ---------------- V phase ----------------
#pragma unroll
      for (int i = 0; i < VI; ++i) {
        const int j = i % PFV;
        float vf[VE];
        if (DT == kF8) {
          if (VB == 8) { e4m3x4_to_f32(vreg2[j].x, vf); e4m3x4_to_f32(vreg2[j].y, vf + 4 % VE); }
          else {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) e4m3x4_to_f32(vreg4[j][q4], vf + (4 * q4) % VE);
          }
        } else if (DT == kF16) {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) { vf[(2 * q4) % VE] = h16_bits_to_f32(vreg4[j][q4] & 0xFFFFu); vf[(2 * q4 + 1) % VE] = h16_bits_to_f32(vreg4[j][q4] >> 16); }
        } else {
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) { const uint32_t vw = vreg4[j][q4]; vf[q4 % VE] = __builtin_bit_cast(float, vw); }
        }
        issue_v(j, (i + PFV < VI ? off + (uint32_t)((i + PFV) * RPV) * row_stride : noff + (uint32_t)((i + PFV - VI) * RPV) * row_stride));
        const rowvec_t pv = lds_s[w][i * RPV + rv];
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          const float p = rv_get<GT>(pv, g);
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[g][e] = fmaf(p, vf[e], acc[g][e]);
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }

  // ---------------- wave-level merge of the RPV row groups, then workgroup merge ----------------
#pragma unroll
  for (int g = 0; g < GT; ++g) l_run[g] = wave_sum_uniform(l_run[g]);
  constexpr int G1 = (LPRV <= 32 && GT >= 2) ? GT / 2 : GT;
  float r1[G1][VE];
  int head_off = 0;
  if (LPRV <= 32) {
    if (GT >= 2) {
#pragma unroll
      for (int g = 0; g < G1; ++g)
#pragma unroll
        for (int e = 0; e < VE; ++e) { float x = acc[g][e], y = acc[g + G1][e]; swap32(x, y); r1[g][e] = x + y; }
      head_off += (lane >> 5) * G1;
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e) r1[0][e] = xor32_sum(acc[0][e]);
    }
  } else {
#pragma unroll
    for (int g = 0; g < G1; ++g)
#pragma unroll
      for (int e = 0; e < VE; ++e) r1[g][e] = acc[g][e];
  }
  constexpr int G2 = (LPRV <= 16 && G1 >= 2) ? G1 / 2 : G1;
  float r2[G2][VE];
  if (LPRV <= 16) {
    if (G1 >= 2) {
#pragma unroll
      for (int g = 0; g < G2; ++g)
#pragma unroll
        for (int e = 0; e < VE; ++e) { float x = r1[g][e], y = r1[g + G2][e]; swap16(x, y); r2[g][e] = x + y; }
      head_off += ((lane >> 4) & 1) * G2;
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e) r2[0][e] = xor16_sum(r1[0][e]);
    }
  } else {
#pragma unroll
    for (int g = 0; g < G2; ++g)
#pragma unroll
      for (int e = 0; e < VE; ++e) r2[g][e] = r1[g][e];
  }
  if (LPRV <= 8) {
#pragma unroll
    for (int g = 0; g < G2; ++g)
#pragma unroll
      for (int e = 0; e < VE; ++e) r2[g][e] += dpp_f<kDppRor8>(r2[g][e]);
  }
  bool writer = true;
  if (LPRV <= 8) writer = writer && ((lane & 8) == 0);
  if (LPRV <= 16 && G1 < 2) writer = writer && ((lane & 16) == 0);
  if (LPRV <= 32 && GT < 2) writer = writer && ((lane & 32) == 0);
  if (writer) {
#pragma unroll
    for (int g = 0; g < G2; ++g)
#pragma unroll
      for (int e = 0; e < VE; ++e) lds_o[w][head_off + g][cv * VE + e] = r2[g][e];
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < GT; ++g) { lds_m[w][g] = m_run[g]; lds_l[w][g] = l_run[g]; }
  }
  __syncthreads();
  for (int idx = tid; idx < GT * D; idx += NW * 64) {
    const int g = idx / D, d = idx - g * D;
    float M = lds_m[0][g];
#pragma unroll
    for (int ww = 1; ww < NW; ++ww) M = fmaxf(M, lds_m[ww][g]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) { const float f = exp2f(lds_m[ww][g] - M); o = fmaf(f, lds_o[ww][g][d], o); l = fmaf(f, lds_l[ww][g], l); }
    const size_t pidx = (size_t)(h0 + g) * a.n_tiles + jl;
    a.so[pidx * D + d] = o;
    if (d == 0) { a.sm[pidx] = M > -1e29f ? M * 0.693147180559945f : kMasked; a.ss[pidx] = l; }
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
        const float bm = wave_max_all(sc);
        const float m_new = fmaxf(m_run, bm);
        const float alpha = __expf(m_run - m_new);
        const float p = valid ? __expf(sc - m_new) : 0.f;
        l_run = l_run * alpha + wave_sum_all(p);
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
// have no serial dependency; mathematically this is the reference's running merge.  Every load a
// thread needs (its tiles' max / sum and its slice of the partial outputs) is issued before the
// first reduction, so the kernel costs about one memory round trip.
constexpr int kReduceThreads = 256;
constexpr int kReduceChunk = 8;      // partial-output rows a thread holds in registers at a time
__global__ __launch_bounds__(kReduceThreads) void reduce_kernel(const float* __restrict__ so,
                                                                const float* __restrict__ sm,
                                                                const float* __restrict__ ss,
                                                                float* __restrict__ o, uint32_t D,
                                                                uint32_t n_tiles) {
    extern __shared__ float lds[];   // [n_tiles] weights, then [parts][D] partial sums
    __shared__ float red[2][kReduceThreads / kWave];
    const uint32_t h = blockIdx.x;
    const int tid = threadIdx.x;
    const float* hm = sm + (size_t)h * n_tiles;
    const float* hs = ss + (size_t)h * n_tiles;
    const float* ho = so + (size_t)h * n_tiles * D;
    float* wts = lds;
    float* psum = lds + n_tiles;

    const uint32_t d4n = D / 4u;                       // D is a multiple of 4 on this path
    const uint32_t parts = kReduceThreads / d4n;       // >= 1 because D <= 1024
    const uint32_t part = tid / d4n, d4 = tid % d4n;
    const bool has_slice = part < parts;

    // first chunk of partial outputs, in flight during the max / sum reductions
    float4 x[kReduceChunk];
#pragma unroll
    for (int c = 0; c < kReduceChunk; ++c) {
        const uint32_t j = part + c * parts;
        x[c] = (has_slice && j < n_tiles) ? *reinterpret_cast<const float4*>(ho + (size_t)j * D + 4u * d4)
                                          : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float M = kMasked;
    for (uint32_t j = tid; j < n_tiles; j += kReduceThreads) M = fmaxf(M, hm[j]);
    M = wave_max_uniform(M);
    if ((tid & (kWave - 1)) == 0) red[0][tid >> 6] = M;
    __syncthreads();
    M = red[0][0];
#pragma unroll
    for (int i = 1; i < kReduceThreads / kWave; ++i) M = fmaxf(M, red[0][i]);

    float L = 0.f;
    for (uint32_t j = tid; j < n_tiles; j += kReduceThreads) {
        const float wj = __expf(hm[j] - M);
        wts[j] = wj;
        L = fmaf(wj, hs[j], L);
    }
    L = wave_sum_uniform(L);
    if ((tid & (kWave - 1)) == 0) red[1][tid >> 6] = L;
    __syncthreads();
    L = 0.f;
#pragma unroll
    for (int i = 0; i < kReduceThreads / kWave; ++i) L += red[1][i];

    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (has_slice) {
        for (uint32_t j0 = part; j0 < n_tiles; j0 += kReduceChunk * parts) {
            if (j0 != part) {
#pragma unroll
                for (int c = 0; c < kReduceChunk; ++c) {
                    const uint32_t j = j0 + c * parts;
                    x[c] = j < n_tiles ? *reinterpret_cast<const float4*>(ho + (size_t)j * D + 4u * d4)
                                       : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
#pragma unroll
            for (int c = 0; c < kReduceChunk; ++c) {
                const uint32_t j = j0 + c * parts;
                const float wj = j < n_tiles ? wts[j] : 0.f;
                acc.x = fmaf(wj, x[c].x, acc.x); acc.y = fmaf(wj, x[c].y, acc.y);
                acc.z = fmaf(wj, x[c].z, acc.z); acc.w = fmaf(wj, x[c].w, acc.w);
            }
        }
        float* dst = psum + (size_t)part * D + 4u * d4;
        dst[0] = acc.x; dst[1] = acc.y; dst[2] = acc.z; dst[3] = acc.w;
    }
    __syncthreads();
    const float inv = 1.0f / L;
    for (uint32_t d = tid; d < D; d += kReduceThreads) {
        float sum = 0.f;
        for (uint32_t p = 0; p < parts; ++p) sum += psum[(size_t)p * D + d];
        o[(size_t)h * D + d] = sum * inv;
    }
}

// Few tiles (<= MAXT <= 64): one wavefront per (head, 64 output dimensions), no LDS and no barrier.  Lane j owns tile
// j's max / sum and turns them into its merge weight; every lane also owns one output dimension and loads that
// dimension of all partial outputs before the first reduction, so the kernel costs one memory round trip.
// GATED: the output element is multiplied by sigmoid(gate) in the same store (the reference's separate sigmoid_mul dispatch,
// executor/attention.rs:632-680); the gate value is requested with the partials.
// RAGGED: head_dim is no multiple of 64; the lanes past the last output dimension follow it and store nothing.
template <int MAXT, bool GATED, bool RAGGED = false>
__global__ __launch_bounds__(kWave) void reduce_direct_kernel(const float* __restrict__ so, const float* __restrict__ sm,
                                                              const float* __restrict__ ss, float* __restrict__ o,
                                                              uint32_t D, uint32_t n_tiles, GateArgs gate) {
    const uint32_t h = blockIdx.y, lane = threadIdx.x;
    const uint32_t d_lane = blockIdx.x * kWave + lane;
    const uint32_t d = RAGGED && d_lane >= D ? D - 1u : d_lane;
    const float* ho = so + (size_t)h * n_tiles * D + d;
    float x[MAXT];
#pragma unroll
    for (int j = 0; j < MAXT; ++j) x[j] = ho[(size_t)((uint32_t)j < n_tiles ? j : 0) * D];
    const float mj = lane < n_tiles ? sm[(size_t)h * n_tiles + lane] : kMasked;
    const float sj = lane < n_tiles ? ss[(size_t)h * n_tiles + lane] : 0.f;
    float gv = 0.f;
    if (GATED) {   // the index arithmetic (one 32-bit division: n_heads * D < 2^32) runs while the partials are in flight
        const uint32_t i = h * D + d, token = i / gate.chunk;
        gv = gate.gate[(uint64_t)token * gate.stride + gate.gate_offset + (i - token * gate.chunk)];
    }
    const float M = wave_max_uniform(mj);
    const float wj = lane < n_tiles ? __expf(mj - M) : 0.f;
    const float L = wave_sum_uniform(wj * sj);
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < MAXT; ++j)
        acc = fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), x[j], acc);
    const float r = acc * (1.0f / L);
    if (!RAGGED || d_lane < D) o[(size_t)h * D + d] = GATED ? sigmoid_gate(r, gv) : r;
}

// 65 to 2 048 tiles (few KV heads over long contexts: one tile per compute unit then means many per head; the reference's
// 64-key tiles at long contexts): the same scheme with four wavefronts per (head, 64 output dimensions).  Wavefront w
// merges tiles [64 w, 64 w + 64) into a partial (maximum, sum, 64 outputs) exactly as above, then the tiles 256 further
// on into another that it folds into the first, and so on; the four partials are combined through LDS.  One memory
// round trip per 256 tiles, where the generic kernel below walks the tiles of a head in a loop of one workgroup.
template <bool GATED>
__global__ __launch_bounds__(4 * kWave) void reduce_direct4_kernel(const float* __restrict__ so, const float* __restrict__ sm,
                                                                  const float* __restrict__ ss, float* __restrict__ o,
                                                                  uint32_t D, uint32_t n_tiles, GateArgs gate) {
    __shared__ float pacc[4][kWave];
    __shared__ float pm[4], pl[4];
    const uint32_t h = blockIdx.y, lane = threadIdx.x & (kWave - 1), w = threadIdx.x >> 6;
    const uint32_t d = blockIdx.x * kWave + lane;
    float gv = 0.f;
    if (GATED && w == 0u) {
        const uint32_t i = h * D + d, token = i / gate.chunk;
        gv = gate.gate[(uint64_t)token * gate.stride + gate.gate_offset + (i - token * gate.chunk)];
    }
    float Mr = kMasked, Lr = 0.f, ar = 0.f;                       // this wavefront's partial so far
    for (uint32_t base = w * kWave; base < n_tiles; base += 4u * kWave) {   // wavefront-uniform
        const uint32_t cnt = n_tiles - base < (uint32_t)kWave ? n_tiles - base : (uint32_t)kWave;
        const float* ho = so + ((size_t)h * n_tiles + base) * D + d;
        float x[kWave];
#pragma unroll
        for (int j = 0; j < kWave; ++j) x[j] = ho[(size_t)((uint32_t)j < cnt ? j : 0) * D];
        const float mj = lane < cnt ? sm[(size_t)h * n_tiles + base + lane] : kMasked;
        const float sj = lane < cnt ? ss[(size_t)h * n_tiles + base + lane] : 0.f;
        const float M = wave_max_uniform(mj);
        const float wj = lane < cnt ? __expf(mj - M) : 0.f;
        const float L = wave_sum_uniform(wj * sj);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < kWave; ++j)
            acc = fmaf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), j)), x[j], acc);
        const float Mn = fmaxf(Mr, M);
        const float fr = __expf(Mr - Mn), fc = __expf(M - Mn);   // first round: fr scales zeros
        ar = ar * fr + acc * fc;
        Lr = Lr * fr + L * fc;
        Mr = Mn;
    }
    pacc[w][lane] = ar;
    if (lane == 0u) { pm[w] = Mr; pl[w] = Lr; }
    __syncthreads();
    if (w != 0u) return;
    const float Mt = fmaxf(fmaxf(pm[0], pm[1]), fmaxf(pm[2], pm[3]));
    float Lt = 0.f, r = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float f = __expf(pm[i] - Mt);      // a wavefront without tiles holds the "minus infinity": factor 0
        Lt = fmaf(f, pl[i], Lt);
        r = fmaf(f, pacc[i][lane], r);
    }
    r *= 1.0f / Lt;
    o[(size_t)h * D + d] = GATED ? sigmoid_gate(r, gv) : r;
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

}  // namespace vfkv
#include "attn_decode_mfma.h"
#include "attn_decode_il.h"
#include "attn_decode_f32.h"
namespace vfkv {

// ---- dispatch -----------------------------------------------------------------------------------
constexpr int kSplitWaves = 4;

// Shape of the matrix-core worker: four wavefronts per workgroup (one per SIMD), runs of 32 rows (64 at head_dim 64), one
// run in flight ahead of the one being computed.  Two runs in flight, runs of 64 rows, and eight wavefronts per workgroup
// were each measured slower on the 32 k and 8 k FP8 workloads.
constexpr int kMfmaWaves = 4;

template <int DT, int D, int RUN, int PF, int NH = 1, bool PAD = false, bool PAIR = false>
static hipError_t launch_split_mfma(const SplitArgs& a, uint32_t g, hipStream_t stream, uint32_t head_dim = (uint32_t)D) {
    constexpr int NW = kMfmaWaves;
    const uint32_t gt = g < 8u ? g : 8u;
    dim3 grid(a.n_kv_heads, a.n_tiles, (g + gt - 1u) / gt);
    if (PAD && (head_dim >= (uint32_t)D || head_dim % 16u != 0u)) return hipErrorInvalidValue;
    if (PAIR && (g > 8u || g % 2u != 0u)) return hipErrorInvalidValue;
    if (a.softcap > 0.f)
        hipLaunchKernelGGL((split_mfma_kernel<DT, D, RUN, PF, NW, true, NH, PAD, PAIR>), grid, dim3(NW * kWave), 0, stream, a, gt, head_dim);
    else
        hipLaunchKernelGGL((split_mfma_kernel<DT, D, RUN, PF, NW, false, NH, PAD, PAIR>), grid, dim3(NW * kWave), 0, stream, a, gt, head_dim);
    return hipGetLastError();
}

template <int DT, int D, int RUN>
static hipError_t launch_split_il(const SplitArgs& a_in, uint32_t g, const RopeFold* rope, hipStream_t stream) {
    constexpr int NW = kMfmaWaves;
    SplitArgs a = a_in;
    {   // A ragged last run of at most 16 rows rides with the run before it when that saves the launch a round: when, without
        // it as a unit of its own, the units divide evenly among the run streams of a KV head.
        const uint32_t tile_base = a.tile_first * a.tile, span = a.seq_len > tile_base ? a.seq_len - tile_base : 0u;
        const uint32_t lo = tile_base > a.kv_start ? tile_base : a.kv_start;
        const uint32_t n_runs = (span + RUN - 1u) / RUN, first_run = (lo - tile_base) / RUN, r_tail = span % RUN;
        const uint32_t S = NW * a.n_tiles;
        if (r_tail != 0u && r_tail <= 16u && n_runs >= first_run + 2u && (n_runs - first_run - 1u) % S == 0u) a.interleave |= 2u;
    }
    const uint32_t gt = g < 8u ? g : 8u;
    dim3 grid(a.n_kv_heads, a.n_tiles, (g + gt - 1u) / gt);
    if (rope != nullptr) {
        RopeFoldArgs rf;
        rf.q_weight = rope->q_weight; rf.k_weight = rope->k_weight; rf.freq_factors = rope->freq_factors;
        rf.q_out = rope->q_out; rf.k_out = rope->k_out; rf.rotary_dim = rope->rotary_dim; rf.mode = rope->mode;
        rf.theta_scale = rope->theta_scale; rf.freq_scale = rope->freq_scale; rf.attn_factor = rope->attn_factor; rf.eps = rope->eps;
        if (a.softcap > 0.f) hipLaunchKernelGGL((split_mfma_il_rope_kernel<DT, D, RUN, NW, true>), grid, dim3(NW * kWave), 0, stream, a, gt, rf);
        else hipLaunchKernelGGL((split_mfma_il_rope_kernel<DT, D, RUN, NW, false>), grid, dim3(NW * kWave), 0, stream, a, gt, rf);
    } else {
        if (a.softcap > 0.f) hipLaunchKernelGGL((split_mfma_il_kernel<DT, D, RUN, NW, true>), grid, dim3(NW * kWave), 0, stream, a, gt);
        else hipLaunchKernelGGL((split_mfma_il_kernel<DT, D, RUN, NW, false>), grid, dim3(NW * kWave), 0, stream, a, gt);
    }
    return hipGetLastError();
}

// Head widths between the tiled ones (Phi-style 80 / 96, 112, 160, 192, 224): the width of the worker that serves them with
// its tail masked off (the PAD forms of split_mfma_kernel and split_mfma_f32_kernel), 0 for every other width.
uint32_t split_padded_dim(uint32_t dtype, uint32_t D) {
    if (dtype > kF8 || D % 16u != 0u) return 0u;
    return (D > 64u && D < 128u) ? 128u : (D > 128u && D < 256u) ? 256u : 0u;
}

// F32 caches on the f32 matrix instruction (attn_decode_f32.h)
static bool f32_mfma_shape(uint32_t dtype, uint32_t D) {
    return dtype == kF32 && (D == 64u || D == 128u || D == 256u || split_padded_dim(dtype, D) != 0u);
}

// Rows per run of the interleaved worker.  The full run is 32 rows (64 at head_dim 64): 8 KiB of K and V per wavefront in
// flight over FP8 rows of 64 / 128 elements, 16 KiB over F16 rows of 64 / 128 and FP8 rows of 256, 32 KiB over F16 rows of 256.
// Every shape also has a worker with runs of half that, and a launch takes whichever measured faster for its shape and its
// number of full runs per run stream (us per layer inside graphs that stream at least 768 MB per replay, so that nothing is
// left in the memory-side cache; 32 / 8 heads, 16 / 8 at head_dim 256; S = run streams of a KV head):
//   * where a stream has at most one and a half full runs (300 to 6 144 keys with 128 streams) half runs win on every shape,
//     4-12 % per layer: the launch is a latency chain there and a smaller unit shortens it;
//   * 32 KiB in flight per wavefront is too much at every length (F16 256: 13.8 -> 11.7 us at 4 096 keys, 28.9 -> 26.9 at 16 384);
//   * the 8 KiB shapes lose with half runs from two full runs per stream on (FP8 128: 8.8 -> 9.3 us at 8 192 keys, 10.0 -> 11.2
//     at 12 288, 16.4 -> 18.6 at 32 768), and so do F16 rows of 128 (15.6 -> 16.0 us at 16 384 keys, 25.9 -> 26.8 at 32 768,
//     47.2 -> 48.5 at 65 536); F16 rows of 64 and FP8 rows of 256 are level there.
static uint32_t il_full_run(uint32_t D) { return D == 64u ? 64u : 32u; }

static bool il_half_runs(uint32_t dtype, uint32_t D, uint32_t span_rows, uint32_t n_tiles) {
    static const bool off = [] { const char* e = getenv("VFKV_DECODE_HALF_RUNS"); return e && e[0] == '0'; }();   // for comparisons (the shapes that have both)
    if (off) return false;
    const uint32_t full = il_full_run(D), units = (span_rows + full - 1u) / full, S = (uint32_t)kMfmaWaves * n_tiles;
    if ((dtype == kF8 && D != 256u) || (dtype == kF16 && D == 128u)) return 2u * units <= 3u * S;
    return true;                     // F16 rows of 64 and of 256 elements, FP8 rows of 256
}

// The shortest run the worker may take for this shape: what the caller sizes its workgroup count by.
uint32_t split_run_rows(uint32_t dtype, uint32_t D) {
    if (f32_mfma_shape(dtype, D)) return 16u;                                   // the F32 worker: one tile per run
    if (const uint32_t dp = split_padded_dim(dtype, D)) return dp == 256u && dtype == kF16 ? 16u : 32u;   // as launch_split deals them
    if ((dtype != kF8 && dtype != kF16) || (D != 64u && D != 128u && D != 256u && D != 512u)) return 0u;
    return il_full_run(D) / 2u;      // (head_dim 512: 16 rows as well)
}

template <int D, bool PAD = false>
static hipError_t launch_split_f32(const SplitArgs& a, uint32_t g, hipStream_t stream, uint32_t head_dim = (uint32_t)D) {
    constexpr int NW = kMfmaWaves;
    const uint32_t gt = g < 16u ? g : 16u;          // up to 16 heads of a group share a workgroup's K / V stream
    dim3 grid(a.n_kv_heads, a.n_tiles, (g + gt - 1u) / gt);
    if (PAD && (head_dim >= (uint32_t)D || head_dim % 16u != 0u)) return hipErrorInvalidValue;
    if (a.softcap > 0.f) hipLaunchKernelGGL((split_mfma_f32_kernel<D, NW, true, PAD>), grid, dim3(NW * kWave), 0, stream, a, gt, head_dim);
    else hipLaunchKernelGGL((split_mfma_f32_kernel<D, NW, false, PAD>), grid, dim3(NW * kWave), 0, stream, a, gt, head_dim);
    return hipGetLastError();
}

// Shapes the matrix-core worker is built for (head_dim 512: two wavefronts per run, each half of the output columns).
static bool mfma_worker_shape(uint32_t dtype, uint32_t D) {
    return (dtype == kF8 || dtype == kF16) && (D == 64u || D == 128u || D == 256u || D == 512u || split_padded_dim(dtype, D) != 0u);
}

// VFKV_DECODE_WORKER=valu keeps the vector-ALU worker for every shape (for comparisons).
static bool mfma_worker_enabled() {
    static const bool on = [] { const char* e = getenv("VFKV_DECODE_WORKER"); return !(e && e[0] == 'v'); }();
    return on;
}

// FP8 heads of 64 elements are half a 128-byte memory line each: taken as separate KV heads (whose workgroups may sit on
// different XCDs) every line of the cache is fetched twice.  Over long spans a launch that deals runs takes two neighbouring
// KV heads as one row of 128 bytes instead (split_mfma_kernel's PAIR form), when the pair's query heads fit one workgroup
// (2 G <= 8).  Us per layer, worker + merge, separate heads -> pairs: 32 / 8 / 64 at 65 536 rows 23.1 -> 17.1, 32 768 rows
// 14.1 -> 11.6, 16 384 rows 9.7 -> 9.4, 12 288 rows 8.4 -> 9.0; 16 / 16 / 64 at 16 384 rows 14.7 -> 11.6, 8 192 rows 9.5 -> 8.4,
// 4 096 rows 7.2 -> 7.5; 32 / 32 / 64 at 8 192 rows 14.3 -> 11.1, 4 096 rows 9.7 -> 8.6, 2 048 rows level: pairs pay from about
// 131 072 / n_kv_heads visible rows on.
bool split_pairs_heads(const SplitLaunch& L) {
    static const bool off = [] { const char* e = getenv("VFKV_DECODE_PAIRS"); return e && e[0] == '0'; }();   // for comparisons
    if (off || !L.interleave || L.rope != nullptr || L.dtype != kF8 || L.head_dim != 64u || L.n_kv_heads == 0u || L.n_kv_heads % 2u != 0u)
        return false;
    const uint32_t g = L.n_heads / L.n_kv_heads;
    const uint32_t min_rows = 131072u / L.n_kv_heads;      // 16 384 visible rows with 8 KV heads, 8 192 with 16, 4 096 with 32
    if (g == 0u || g > 4u || L.n_heads % L.n_kv_heads != 0u || L.seq_len < L.kv_start + min_rows) return false;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.scratch_out) | ((uintptr_t)L.o_direct)) & 15u) == 0u;
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim;
    return aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled();
}

// Run streams per workgroup of a launch that deals the runs of the whole span to its workgroups whatever the tile length
// says (0: the launch keeps partial j = tile j): four for the interleaved worker and the F32 worker, two at head_dim 512,
// where two wavefronts share a run.  *heads_per_wg: query heads of a GQA group that one workgroup serves.
uint32_t split_run_streams(const SplitLaunch& L, uint32_t* heads_per_wg) {
    if (heads_per_wg) *heads_per_wg = 8u;
    if (split_pairs_heads(L) || split_interleaves(L)) return (uint32_t)kMfmaWaves;
    if (!L.interleave || L.n_kv_heads == 0u) return 0u;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.scratch_out) | ((uintptr_t)L.o_direct)) & 15u) == 0u;
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    if (!aligned || slab_bytes >= 0x7FFF0000ull || !mfma_worker_enabled()) return 0u;
    if (L.head_dim == 512u && (L.dtype == kF8 || L.dtype == kF16)) return (uint32_t)kMfmaWaves / 2u;
    if (f32_mfma_shape(L.dtype, L.head_dim)) { if (heads_per_wg) *heads_per_wg = 16u; return (uint32_t)kMfmaWaves; }
    if (split_padded_dim(L.dtype, L.head_dim) != 0u) return (uint32_t)kMfmaWaves;
    return 0u;
}

template <int DT, int D, int GT>
static hipError_t launch_split_t(const SplitArgs& a, uint32_t groups, hipStream_t stream) {
    dim3 grid(a.n_tiles, a.n_kv_heads, groups);
    if (a.softcap > 0.f)
        hipLaunchKernelGGL((split_kernel<DT, D, GT, kSplitWaves, true>), grid, dim3(kSplitWaves * kWave), 0, stream, a);
    else
        hipLaunchKernelGGL((split_kernel<DT, D, GT, kSplitWaves, false>), grid, dim3(kSplitWaves * kWave), 0, stream, a);
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
    return (uint32_t)kRun;
}

// True when launch_split would write the token row (k_new, v_new) itself.  The interleaved worker (attn_decode_il.h) does
// so for the last row of the span (the wavefront that reads the row converts it into its own registers and stores it);
// split_mfma_kernel with a single head slice, where one workgroup per KV head owns the new row and can store it before
// anything reads it.
bool split_appends(const SplitLaunch& L) {
    if (!L.k_new || !L.v_new || L.n_kv_heads == 0u) return false;
    const uint32_t g = L.n_heads / L.n_kv_heads;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.k_new) | ((uintptr_t)L.v_new) |
                           ((uintptr_t)L.scratch_out)) & 15u) == 0u;
    if (split_pairs_heads(L)) return aligned && L.append_pos < L.seq_len && L.append_pos >= L.kv_start;   // (split_mfma_kernel, one head slice)
    if (split_interleaves(L)) return aligned && L.append_pos + 1u == L.seq_len && L.append_pos >= L.kv_start;
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    const bool mfma_shape = mfma_worker_shape(L.dtype, L.head_dim);
    return aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled() && mfma_shape && g <= 8u &&
           L.append_pos < L.seq_len && L.append_pos >= L.kv_start;
}

// True when a launch of one tile can write the normalised output itself (matrix-core worker shapes).
bool split_writes_output(const SplitLaunch& L) {
    if (L.n_tiles != 1u || L.n_kv_heads == 0u) return false;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.scratch_out)) & 15u) == 0u;
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    const bool mfma_shape = mfma_worker_shape(L.dtype, L.head_dim) || f32_mfma_shape(L.dtype, L.head_dim);
    return aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled() && mfma_shape;
}

bool split_interleaves(const SplitLaunch& L) {
    static const bool off = [] { const char* e = getenv("VFKV_DECODE_IL"); return e && e[0] == '0'; }();
    if (off || !L.interleave || L.n_kv_heads == 0u || L.n_tiles == 0u || split_pairs_heads(L)) return false;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q) | ((uintptr_t)L.scratch_out) | ((uintptr_t)L.o_direct)) & 15u) == 0u;
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    return aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled() && (L.dtype == kF8 || L.dtype == kF16) &&
           (L.head_dim == 64u || L.head_dim == 128u || L.head_dim == 256u);
}

bool split_folds_rope(const SplitLaunch& L) {
    if (!L.rope || !split_interleaves(L) || !split_appends(L)) return false;
    {   // FP8 heads of 64 elements over very long spans: the rotation as a launch of its own in front of paired KV heads beats
        // the fold into the worker for separate heads (32 / 8 / 64, us per 8-layer step, fold -> rotation launch + pairs:
        // 16 385 keys 90.7 -> 111.9, 32 769 keys 121.8 -> 128.4, 65 537 keys 194.1 -> 171.6): no fold from three times the
        // span at which pairs start to pay
        SplitLaunch P = L;
        P.rope = nullptr; P.k_new = nullptr; P.v_new = nullptr;
        if (split_pairs_heads(P) && L.seq_len >= L.kv_start + 3u * (131072u / L.n_kv_heads)) return false;
    }
    const RopeFold& r = *L.rope;
    const bool aligned = ((((uintptr_t)r.q_out) | ((uintptr_t)r.k_out)) & 3u) == 0u;
    return aligned && r.rotary_dim % 2u == 0u && r.rotary_dim <= L.head_dim && (r.mode == 0u || r.mode == 2u);
}

hipError_t launch_split(const SplitLaunch& L, hipStream_t stream, bool* generic_used) {
    if (generic_used) *generic_used = false;
    if (L.dtype > kF8 || L.head_dim == 0u || L.head_dim > 512u) return hipErrorInvalidValue;
    if (L.n_tiles == 0u) return hipSuccess;
    SplitArgs a;
    a.q = L.q; a.k = (const uint8_t*)L.k; a.v = (const uint8_t*)L.v;
    a.so = L.scratch_out; a.sm = L.scratch_max; a.ss = L.scratch_sum;
    a.n_heads = L.n_heads; a.n_kv_heads = L.n_kv_heads; a.group = L.n_heads / L.n_kv_heads;
    a.seq_len = L.seq_len; a.kv_start = L.kv_start;
    a.tile = L.tile; a.tile_first = L.tile_first; a.n_tiles = L.n_tiles;
    a.scale = L.scale; a.softcap = L.softcap;
    a.k_new = nullptr; a.v_new = nullptr; a.append_pos = 0u; a.o_direct = nullptr;
    a.interleave = L.interleave ? 1u : 0u;
    if (L.o_direct) {
        if (!split_writes_output(L) || ((uintptr_t)L.o_direct & 15u) != 0u) return hipErrorInvalidValue;
        a.o_direct = L.o_direct;
    }
    const uint32_t g = L.n_heads / L.n_kv_heads;
    const bool aligned = ((((uintptr_t)L.k) | ((uintptr_t)L.v) | ((uintptr_t)L.q)) & 15u) == 0u;
    // the register-tiled worker addresses the slab with 32-bit byte offsets below 2 GiB
    const uint64_t slab_bytes = (uint64_t)L.seq_len * L.n_kv_heads * L.head_dim * elem_size(L.dtype);
    if (L.k_new && L.v_new) {
        if (!split_appends(L)) return hipErrorInvalidValue;      // the caller asked for a fused append this worker cannot do
        a.k_new = L.k_new; a.v_new = L.v_new; a.append_pos = L.append_pos;
    }
    // the matrix-core worker also stores its partials (or the output) 16 bytes at a time
    const bool out_aligned = ((((uintptr_t)L.scratch_out) | ((uintptr_t)L.o_direct)) & 15u) == 0u;
    if (L.rope != nullptr && !split_folds_rope(L)) return hipErrorInvalidValue;      // the caller rotates in a launch of its own then
    if (split_pairs_heads(L) && out_aligned) {     // two 64-wide FP8 heads as one row of 128: half as many KV heads, twice the group
        SplitArgs ap = a;
        ap.n_kv_heads = a.n_kv_heads / 2u; ap.group = a.group * 2u;
        return launch_split_mfma<kF8, 128, 32, 1, 1, false, true>(ap, ap.group, stream);
    }
    if (split_interleaves(L) && out_aligned) {
        const uint32_t base_row = a.tile_first * a.tile;
        const bool half = il_half_runs(L.dtype, L.head_dim, a.seq_len > base_row ? a.seq_len - base_row : 0u, a.n_tiles);
#define VFKV_IL(DT, DD, FULL) \
    if (L.dtype == DT && L.head_dim == DD) \
        return half ? launch_split_il<DT, DD, FULL / 2>(a, g, L.rope, stream) : launch_split_il<DT, DD, FULL>(a, g, L.rope, stream);
        VFKV_IL(kF8, 64u, 64) VFKV_IL(kF8, 128u, 32) VFKV_IL(kF16, 128u, 32)
#undef VFKV_IL
        // (these three take half runs at every length)
        if (L.dtype == kF16 && L.head_dim == 64u) return launch_split_il<kF16, 64, 32>(a, g, L.rope, stream);
        if (L.dtype == kF8 && L.head_dim == 256u) return launch_split_il<kF8, 256, 16>(a, g, L.rope, stream);
        if (L.dtype == kF16 && L.head_dim == 256u) return launch_split_il<kF16, 256, 16>(a, g, L.rope, stream);
    }
    if (aligned && out_aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled()) {
        // Tiles with fewer full runs than the workgroup has run streams (the reference's 64-key tiles: two runs of 32 rows for
        // four wavefronts) take runs of half the rows, so that every wavefront has one; a launch that deals the runs of the
        // whole span (interleave) keeps full runs.
        const bool short_tiles = !a.interleave && a.tile < (uint32_t)kMfmaWaves * il_full_run(L.head_dim);
#define VFKV_TM(DT, DD, FULL) \
    if (L.dtype == DT && L.head_dim == DD) \
        return short_tiles ? launch_split_mfma<DT, DD, FULL / 2, 1>(a, g, stream) : launch_split_mfma<DT, DD, FULL, 1>(a, g, stream);
        VFKV_TM(kF8, 64u, 64) VFKV_TM(kF16, 64u, 64) VFKV_TM(kF8, 128u, 32) VFKV_TM(kF16, 128u, 32) VFKV_TM(kF8, 256u, 32)
#undef VFKV_TM
        if (L.dtype == kF16 && L.head_dim == 256u) return launch_split_mfma<kF16, 256, 16, 1>(a, g, stream);      // (32 rows of 512 bytes: 32 KiB per wavefront in flight)
        // (runs of 16 rows: with 32 a wavefront has 48 KiB of F16 rows in flight; 9-10 % per layer at every length, FP8 and F16)
        if (L.dtype == kF8 && L.head_dim == 512u) return launch_split_mfma<kF8, 512, 16, 1, 2>(a, g, stream);
        if (L.dtype == kF16 && L.head_dim == 512u) return launch_split_mfma<kF16, 512, 16, 1, 2>(a, g, stream);
        // head widths between the tiled ones: the next wider worker with its tail masked off
        if (const uint32_t dp = split_padded_dim(L.dtype, L.head_dim)) {
            const bool short_pad = !a.interleave && a.tile < (uint32_t)kMfmaWaves * 32u;
#define VFKV_TP(DT, DD, FULL) \
    if (L.dtype == DT && dp == DD) \
        return short_pad ? launch_split_mfma<DT, DD, 16, 1, 1, true>(a, g, stream, L.head_dim) : launch_split_mfma<DT, DD, FULL, 1, 1, true>(a, g, stream, L.head_dim);
            VFKV_TP(kF8, 128u, 32) VFKV_TP(kF16, 128u, 32) VFKV_TP(kF8, 256u, 32) VFKV_TP(kF16, 256u, 16)
#undef VFKV_TP
        }
    }
    if (aligned && out_aligned && slab_bytes < 0x7FFF0000ull && mfma_worker_enabled() && f32_mfma_shape(L.dtype, L.head_dim)) {
        if (L.head_dim == 64u) return launch_split_f32<64>(a, g, stream);
        if (L.head_dim == 128u) return launch_split_f32<128>(a, g, stream);
        if (L.head_dim == 256u) return launch_split_f32<256>(a, g, stream);
        if (L.head_dim < 128u) return launch_split_f32<128, true>(a, g, stream, L.head_dim);
        return launch_split_f32<256, true>(a, g, stream, L.head_dim);
    }
    if (fast_shape(L.dtype, L.head_dim) && aligned && slab_bytes < 0x7FFF0000ull) {
#define VFKV_CASE(DT, DD) \
    if (L.dtype == DT && L.head_dim == DD) return launch_split_d<DT, DD>(a, g, stream);
        VFKV_CASE(kF8, 64) VFKV_CASE(kF8, 128) VFKV_CASE(kF8, 256) VFKV_CASE(kF8, 512)
        VFKV_CASE(kF16, 64) VFKV_CASE(kF16, 128) VFKV_CASE(kF16, 256) VFKV_CASE(kF16, 512)
        VFKV_CASE(kF32, 64) VFKV_CASE(kF32, 128) VFKV_CASE(kF32, 256)
#undef VFKV_CASE
    }
    if (generic_used) *generic_used = true;
    dim3 grid(L.n_tiles, L.n_heads, 1);
    hipLaunchKernelGGL(split_generic_kernel, grid, dim3(kWave), 0, stream, a, L.dtype, L.head_dim);
    return hipGetLastError();
}

hipError_t launch_reduce(const float* so, const float* sm, const float* ss, float* o, uint32_t n_heads,
                         uint32_t D, uint32_t n_tiles, hipStream_t stream, const GateArgs* gate, bool* gate_applied) {
    if (n_heads == 0u || D == 0u || n_tiles == 0u) return hipErrorInvalidValue;
    if (gate_applied) *gate_applied = false;
    const bool gated = gate != nullptr && gate->gate != nullptr;
    if (gated && gate->chunk == 0u) return hipErrorInvalidValue;
    const bool vec = (D % 4u == 0u) && (D / 4u <= (uint32_t)kReduceThreads) && n_tiles <= 8192u &&
                     ((((uintptr_t)so) & 15u) == 0u);
    if (n_tiles <= 64u && D % (uint32_t)kWave == 0u) {
        const dim3 grid(D / kWave, n_heads);
        const GateArgs g = gated ? *gate : GateArgs();
        if (gated) {
            if (n_tiles <= 32u) hipLaunchKernelGGL((reduce_direct_kernel<32, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            else hipLaunchKernelGGL((reduce_direct_kernel<64, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            if (gate_applied) *gate_applied = true;
        } else {
            if (n_tiles <= 32u) hipLaunchKernelGGL((reduce_direct_kernel<32, false>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            else hipLaunchKernelGGL((reduce_direct_kernel<64, false>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
        }
    } else if (n_tiles <= 64u) {                       // head sizes that are no multiple of 64
        const dim3 grid((D + kWave - 1u) / kWave, n_heads);
        const GateArgs g = gated ? *gate : GateArgs();
        if (gated) {
            if (n_tiles <= 32u) hipLaunchKernelGGL((reduce_direct_kernel<32, true, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            else hipLaunchKernelGGL((reduce_direct_kernel<64, true, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            if (gate_applied) *gate_applied = true;
        } else {
            if (n_tiles <= 32u) hipLaunchKernelGGL((reduce_direct_kernel<32, false, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            else hipLaunchKernelGGL((reduce_direct_kernel<64, false, true>), grid, dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
        }
    } else if (n_tiles <= 2048u && D % (uint32_t)kWave == 0u) {
        const dim3 grid(D / kWave, n_heads);
        const GateArgs g = gated ? *gate : GateArgs();
        if (gated) {
            hipLaunchKernelGGL((reduce_direct4_kernel<true>), grid, dim3(4 * kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
            if (gate_applied) *gate_applied = true;
        } else {
            hipLaunchKernelGGL((reduce_direct4_kernel<false>), grid, dim3(4 * kWave), 0, stream, so, sm, ss, o, D, n_tiles, g);
        }
    } else if (vec) {
        const uint32_t d4n = D / 4u;
        const uint32_t parts = kReduceThreads / d4n;
        const size_t lds = ((size_t)parts * D + n_tiles) * sizeof(float);
        hipLaunchKernelGGL(reduce_kernel, dim3(n_heads), dim3(kReduceThreads), lds, stream, so, sm, ss, o, D, n_tiles);
    } else {
        hipLaunchKernelGGL(reduce_generic_kernel, dim3(n_heads), dim3(kWave), 0, stream, so, sm, ss, o, D, n_tiles);
    }
    return hipGetLastError();
}

}  // namespace vfkv
