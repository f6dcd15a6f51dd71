// K RMS-norm * weight, RoPE and the KV append in one launch for gfx950.
//
// Replaces, per layer, the reference's `KNormRope` / `KRope` step followed by `KvWrite`
// (forward/layer_plan.rs:119-137): rms_norm.comp:36-129 in its RMS_NORM_ROPE_FUSION form (or rope_neox.comp /
// rope_norm.comp alone), rope_funcs.glsl:17-112, then kv_store_fp8.comp / kv_copy_fp16.comp for K and V.  The
// rotated K row never makes the round trip through its f32 buffer (it is still written there when the caller asks
// for it), and K and V go out in one launch.
//
// One wavefront per (token, tensor, KV head) row, four rows of a token per workgroup.  The angles depend on (token,
// pair) only: the workgroup evaluates cos / sin once (accurate powf / sincosf: the arguments reach tens of thousands of
// radians) into LDS while the rows and the norm weight are already in flight.  K: the sum of squares is a wavefront
// reduction, the normalised row is parked in the wavefront's LDS row so that a lane can reach both elements of its
// rotation pairs, rotated, and stored from LDS as whole 32-bit words of the cache dtype; V: plain conversion.
// HBM / launch bound: 4 bytes read and 1, 2 or 4 written per element.
#include "device_utils.h"
#include "kernels.h"
#include "rope_device.h"

namespace vfkv {

struct RopeAppendArgs {
    const float* q_src;       // [n_tokens][n_q_heads][head_dim] or NULL: no Q rows in this launch
    const float* q_weight;    // [head_dim] or NULL
    float* q_out;             // rotated Q (may alias q_src)
    uint32_t n_q_heads;
    const float* k_src;       // [n_tokens][n_kv_heads][head_dim]
    const float* v_src;       // same shape, or NULL: K only
    const float* weight;      // [head_dim] or NULL: no RMS-norm
    const int32_t* positions; // [n_tokens] or NULL: pos0 + token
    const float* freq_factors;// [rotary_dim / 2] or NULL
    float* k_out;             // rotated K as f32 (may alias k_src) or NULL
    uint8_t* k_dst;           // cache row of the first token, K; NULL = no cache store (k_out only)
    uint8_t* v_dst;
    uint32_t n_kv_heads, head_dim, rotary_dim, mode, pos0, dtype;
    uint64_t row_bytes;       // distance between two tokens' rows in the cache
    float theta_scale, freq_scale, attn_factor, eps;
};

constexpr int kRopeMaxPerLane = 8;   // head_dim <= 512
constexpr int kRopeWaves = 4;         // rows per workgroup, one per wavefront

__global__ __launch_bounds__(kRopeWaves * kWave) void rope_append_kernel(RopeAppendArgs a) {
    __shared__ float cs_lds[256], sn_lds[256];             // rotary_dim / 2 <= 256
    __shared__ float rows[kRopeWaves][512];
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t tok = blockIdx.x;
    const uint32_t D = a.head_dim;
    const uint32_t half = a.rotary_dim / 2u;
    // rows of this token: the Q heads (if any), then the K heads, then the V heads (if any)
    const uint32_t nq = a.q_src ? a.n_q_heads : 0u;
    const uint32_t n_units = nq + (a.v_src ? 2u * a.n_kv_heads : a.n_kv_heads);
    const uint32_t u = blockIdx.y * kRopeWaves + w;                         // this wavefront's row
    const bool active = u < n_units;
    const bool is_q = u < nq;
    const bool is_v = u >= nq + a.n_kv_heads;
    const uint32_t head = is_q ? u : (is_v ? u - nq - a.n_kv_heads : u - nq);
    const size_t src_off = ((size_t)tok * (is_q ? nq : a.n_kv_heads) + head) * D;
    float* const row = rows[w];
    // every global load of the wavefront (its row, the norm weight) is requested before the angles are computed, so the
    // latencies overlap
    float x[kRopeMaxPerLane], wt[kRopeMaxPerLane];
    const float* const weight = is_q ? a.q_weight : a.weight;
    const bool normed = active && !is_v && weight != nullptr;
    {
        const float* src = (is_q ? a.q_src : is_v ? a.v_src : a.k_src) + src_off;
#pragma unroll
        for (int j = 0; j < kRopeMaxPerLane; ++j) {
            const uint32_t d = lane + j * kWave;
            x[j] = (active && d < D) ? src[d] : 0.f;
            wt[j] = (normed && d < D) ? weight[d] : 1.f;
        }
    }
    // the token's cos / sin table (rope_device.h)
    if (blockIdx.y * kRopeWaves < nq + a.n_kv_heads) {     // workgroup-uniform: workgroups that only hold V rows skip it
        const float pos = (float)(a.positions ? a.positions[tok] : (int32_t)(a.pos0 + tok));
        rope_table(cs_lds, sn_lds, half, pos, a.theta_scale, a.freq_scale, a.attn_factor, a.freq_factors, (uint32_t)tid, kRopeWaves * kWave);
    }
    __syncthreads();
    if (!active) return;
    rope_row<kRopeMaxPerLane>(x, wt, normed, a.eps, D, half, a.mode, !is_v, cs_lds, sn_lds, row, lane);
    if (!is_v) {
        float* const out = is_q ? a.q_out : a.k_out;
        if (out != nullptr)
            for (uint32_t d = lane; d < D; d += kWave) out[src_off + d] = row[d];
    }
    if (is_q || a.k_dst == nullptr) return;                // norm + RoPE only: no cache row to write
    // ---- the head's slice of the cache row as 32-bit words (kv_store_fp8.comp:42-67, kv_copy_fp16.comp:39-51)
    uint8_t* dst = (is_v ? a.v_dst : a.k_dst) + (uint64_t)tok * a.row_bytes;
    if (a.dtype == kF8) {
        uint32_t* d32 = reinterpret_cast<uint32_t*>(dst + (size_t)head * D);
        for (uint32_t e = lane; e < D / 4u; e += kWave)
            d32[e] = pack4_e4m3(row[4 * e], row[4 * e + 1], row[4 * e + 2], row[4 * e + 3]);
    } else if (a.dtype == kF16) {
        uint32_t* d32 = reinterpret_cast<uint32_t*>(dst + (size_t)head * D * 2u);
        for (uint32_t e = lane; e < D / 2u; e += kWave)
            d32[e] = f32_to_h16_bits(row[2 * e]) | (f32_to_h16_bits(row[2 * e + 1]) << 16);
    } else {
        float* d32 = reinterpret_cast<float*>(dst + (size_t)head * D * 4u);
        for (uint32_t d = lane; d < D; d += kWave) d32[d] = row[d];
    }
}

hipError_t launch_rope_append(const RopeAppendLaunch& L, hipStream_t stream) {
    if (L.n_tokens == 0u) return hipSuccess;
    if (L.head_dim == 0u || L.head_dim > 512u || L.head_dim % 4u != 0u || L.rotary_dim > L.head_dim ||
        L.rotary_dim % 2u != 0u || (L.mode != 0u && L.mode != 2u) || L.dtype > kF8 || L.n_kv_heads == 0u)
        return hipErrorInvalidValue;
    RopeAppendArgs a;
    a.q_src = L.q_src; a.q_weight = L.q_weight; a.q_out = L.q_out; a.n_q_heads = L.n_q_heads;
    a.k_src = L.k_src; a.v_src = L.v_src; a.weight = L.weight; a.positions = L.positions;
    a.freq_factors = L.freq_factors; a.k_out = L.k_out;
    a.k_dst = (uint8_t*)L.k_dst; a.v_dst = (uint8_t*)L.v_dst;
    a.n_kv_heads = L.n_kv_heads; a.head_dim = L.head_dim; a.rotary_dim = L.rotary_dim; a.mode = L.mode;
    a.pos0 = L.pos0; a.dtype = L.dtype; a.row_bytes = L.row_bytes;
    a.theta_scale = L.theta_scale; a.freq_scale = L.freq_scale; a.attn_factor = L.attn_factor; a.eps = L.eps;
    if (L.q_src != nullptr && (L.q_out == nullptr || L.n_q_heads == 0u)) return hipErrorInvalidValue;
    const uint32_t n_units = (L.q_src ? L.n_q_heads : 0u) + (L.v_src ? 2u * L.n_kv_heads : L.n_kv_heads);
    if ((n_units + kRopeWaves - 1u) / kRopeWaves > 65535u) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rope_append_kernel, dim3(L.n_tokens, (n_units + kRopeWaves - 1u) / kRopeWaves), dim3(kRopeWaves * kWave),
                       0, stream, a);
    return hipGetLastError();
}

}  // namespace vfkv
