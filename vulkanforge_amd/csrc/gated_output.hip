// Gated attention output for gfx950: data[i] *= sigmoid(gate[(i / chunk) * stride + gate_offset + i % chunk]).
//
// Replaces the reference's `run_sigmoid_mul` dispatch (forward/runs.rs:2649-2681, vk_shaders/sigmoid_mul.comp:40-53) as
// `step_attn_gated_output` / `b_step_attn_gated_output` issue it (executor/attention.rs:632-680, 2405-2444).  HBM bound:
// 8 bytes read and 4 written per element.  Four consecutive elements per lane as 16-byte accesses when the chunk
// geometry and the pointers allow it, one element per lane otherwise.  The decode merge (attn_decode.hip) and the f16
// matrix-core prefill kernel (attn_prefill_mfma2.h) apply the same gate in their own stores, so a decode step only comes
// here when its span fits one tile and a prefill chunk only for gate geometries or kernels without that store.
#include "device_utils.h"
#include "kernels.h"

namespace vfkv {

__global__ __launch_bounds__(256) void sigmoid_mul_vec4_kernel(const float* __restrict__ gate, float* __restrict__ data,
                                                               uint32_t n4, GateArgs g) {
    const uint32_t i4 = blockIdx.x * 256u + threadIdx.x;
    if (i4 >= n4) return;
    const uint64_t i = (uint64_t)i4 * 4u;
    const float4 gv = *reinterpret_cast<const float4*>(gate + gate_index(g, i));
    float4 x = *reinterpret_cast<float4*>(data + i);
    x.x = sigmoid_gate(x.x, gv.x); x.y = sigmoid_gate(x.y, gv.y); x.z = sigmoid_gate(x.z, gv.z); x.w = sigmoid_gate(x.w, gv.w);
    *reinterpret_cast<float4*>(data + i) = x;
}

__global__ __launch_bounds__(256) void sigmoid_mul_kernel(const float* __restrict__ gate, float* __restrict__ data, uint32_t ne,
                                                          GateArgs g) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= ne) return;
    data[i] = sigmoid_gate(data[i], gate[gate_index(g, i)]);
}

hipError_t launch_sigmoid_mul(float* data, uint32_t ne, const GateArgs& g, hipStream_t stream) {
    if (ne == 0u) return hipSuccess;
    if (g.gate == nullptr || data == nullptr || g.chunk == 0u) return hipErrorInvalidValue;
    const bool vec = ((g.chunk | g.stride | g.gate_offset | ne) % 4u) == 0u &&
                     ((((uintptr_t)g.gate) | ((uintptr_t)data)) & 15u) == 0u;
    if (vec) hipLaunchKernelGGL(sigmoid_mul_vec4_kernel, dim3((ne / 4u + 255u) / 256u), dim3(256), 0, stream, g.gate, data, ne / 4u, g);
    else hipLaunchKernelGGL(sigmoid_mul_kernel, dim3((ne + 255u) / 256u), dim3(256), 0, stream, g.gate, data, ne, g);
    return hipGetLastError();
}

}  // namespace vfkv
