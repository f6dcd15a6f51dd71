// RMS-norm * weight and RoPE of one (token, head) row by one wavefront, shared by rope_append_kernel and the decode worker
// that folds the decode token's Q / K norm + RoPE into its own prologue: both must produce the same bits for the same
// row, so the arithmetic lives here once (every multiply-add that could be contracted either way is spelled as an fma).
//   rms_norm.comp:61-112 (scale * x * w in f32), rope_funcs.glsl:39-112 (NORM pairs (2p, 2p + 1), NEOX pairs (p, p + n_dims / 2)),
//   rope_funcs.glsl:63-67,97-101 (theta = pos * theta_scale^p / freq_factor[p] * freq_scale, results scaled by attn_factor).
#pragma once
#include "device_utils.h"

namespace vfkv {

// cos / sin of the `half` rotation angles of one position into LDS, by `nthreads` threads (accurate powf / sincosf: the
// arguments reach tens of thousands of radians).  The caller separates this from the rows' use by a barrier.
__device__ __forceinline__ void rope_table(float* cs_lds, float* sn_lds, uint32_t half, float pos, float theta_scale, float freq_scale,
                                           float attn_factor, const float* freq_factors, uint32_t tid, uint32_t nthreads) {
    for (uint32_t p = tid; p < half; p += nthreads) {
        const float theta_base = pos * powf(theta_scale, (float)p);
        const float ff = freq_factors ? freq_factors[p] : 1.0f;
        const float theta = freq_scale * (theta_base / ff);
        float sn, cs;
        sincosf(theta, &sn, &cs);
        cs_lds[p] = cs * attn_factor;
        sn_lds[p] = sn * attn_factor;
    }
}

// One row of D elements held as x[j] = element lane + 64 j (zeros past D), MAXJ >= ceil(D / 64).  normed: RMS-norm times
// wt[] first.  The row is left in `row` (LDS, private to the wavefront until the caller's next barrier), rotated when
// `rotate` is set.  LDS operations of a wavefront execute in order; the fences only keep the compiler from moving
// accesses across them.
template <int MAXJ>
__device__ __forceinline__ void rope_row(float (&x)[MAXJ], const float (&wt)[MAXJ], bool normed, float eps, uint32_t D, uint32_t half,
                                         uint32_t mode, bool rotate, const float* cs_lds, const float* sn_lds, float* row, int lane) {
    if (normed) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) ss = __builtin_fmaf(x[j], x[j], ss);
        ss = wave_sum_all(ss);
        const float scale = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) x[j] = (scale * x[j]) * wt[j];
    }
#pragma unroll
    for (int j = 0; j < MAXJ; ++j) {
        const uint32_t d = lane + j * kWave;
        if (d < D) row[d] = x[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    if (rotate) {
        for (uint32_t p = lane; p < half; p += kWave) {
            const float cs = cs_lds[p], sn = sn_lds[p];
            const uint32_t i0 = mode == 2u ? p : 2u * p, i1 = mode == 2u ? p + half : 2u * p + 1u;
            const float x0 = row[i0], x1 = row[i1];
            row[i0] = __builtin_fmaf(x0, cs, -(x1 * sn));
            row[i1] = __builtin_fmaf(x0, sn, x1 * cs);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
}

}  // namespace vfkv
