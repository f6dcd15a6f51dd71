// Self-test of the C++ host layer: layout arithmetic without a device, then (with a GPU) one FP8
// append + decode step checked against closed forms that need no reference implementation:
//   * K = 0 makes every weight equal, so O = mean of the decoded V rows;
//   * one key far larger than the rest makes O equal that key's decoded V row;
//   * RoPE with theta_scale = 1 turns every (1, 0) pair into (cos pos, sin pos).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <vector>

#include "vfkv_host.hpp"

#define REQUIRE(c) do { if (!(c)) { std::printf("FAILED: %s (line %d)\n", #c, __LINE__); return 1; } } while (0)

int main() {
    using namespace vfkv;
    {   // kv_cache.rs:553-587
        KvCacheConfig cfg; cfg.n_layers = 36; cfg.n_kv_heads = 8; cfg.head_dim = 128; cfg.max_seq_len = 2048; cfg.dtype = KvDtype::F16;
        KvCache c(cfg, true);
        REQUIRE(2 * c.bytes_per_buffer() == 288ull * 1024 * 1024);
        REQUIRE(c.pos_offset_bytes(3, 5) == c.layer_offset_bytes(3) + 5 * c.row_bytes(3));
        std::vector<uint32_t> hd{256, 256, 512, 512}, kvh{2, 2, 4, 4};
        REQUIRE(kv_bytes_per_token(4, 999, 999, &hd, &kvh, 1) == 10240);
        bool threw = false;
        try { guard_kv_precision(true, KvDtype::F16); } catch (const Error&) { threw = true; }
        REQUIRE(threw);
        KvCacheConfig bad = cfg; bad.n_layers = bad.n_kv_heads = bad.head_dim = bad.max_seq_len = 0xFFFFFFFFu;
        threw = false;
        try { KvCache c2(bad, true); } catch (const Error& e) { threw = e.status == VFKV_ERR_OVERFLOW; }
        REQUIRE(threw);
    }
    {   // gguf.rs:1531-1567 (E2B share pattern), forward/arch/gemma4.rs:27-49, server/state.rs:363-396
        std::vector<uint8_t> sliding(35);
        for (int i = 0; i < 35; ++i) sliding[i] = (i % 5) != 4;
        const std::vector<uint32_t> src = build_kv_sources(sliding, 15, 35);
        REQUIRE(src[13] == VFKV_KV_OWN_PUBLISHES_SLIDING && src[14] == VFKV_KV_OWN_PUBLISHES_FULL && src[12] == VFKV_KV_OWN);
        REQUIRE(gemma4_kv_read_layer(src, 20) == 13 && gemma4_kv_read_layer(src, 34) == 14 && gemma4_kv_read_layer(src, 9) == 9);
        REQUIRE(prefix_reuse_start({10, 11, 12, 13, 14}, {10, 11, 12, 99}) == 3);
        REQUIRE(prefix_reuse_start({1, 2, 3, 4}, {1, 2, 3, 4}) == 3 && prefix_reuse_start({}, {1, 2, 3}) == 0);
    }
    if (vfkv_device_count() == 0) { std::printf("host selftest: layout checks passed (no GPU: compute checks skipped)\n"); return 0; }

    const uint32_t H = 32, Hkv = 8, D = 128, ctx = 1000;
    KvCacheConfig cfg; cfg.n_layers = 2; cfg.n_kv_heads = Hkv; cfg.head_dim = D; cfg.max_seq_len = ctx + 1; cfg.dtype = KvDtype::F8;
    Forward fwd(KvCache(cfg), H);
    fwd.kv_cache.zero_fill();
    const size_t row = Hkv * D;
    std::vector<float> k((ctx + 1) * row, 0.f), v((ctx + 1) * row), q(H * D, 1.0f), o(H * D);
    for (size_t t = 0; t <= ctx; ++t) for (size_t x = 0; x < row; ++x) v[t * row + x] = 0.25f * (float)((t * 7 + x * 3) % 9) - 1.0f;  // exact in E4M3
    float *dk, *dv, *dq, *dout;
    hipMalloc(&dk, k.size() * 4); hipMalloc(&dv, v.size() * 4); hipMalloc(&dq, q.size() * 4); hipMalloc(&dout, o.size() * 4);
    hipMemcpy(dk, k.data(), k.size() * 4, hipMemcpyHostToDevice); hipMemcpy(dv, v.data(), v.size() * 4, hipMemcpyHostToDevice);
    hipMemcpy(dq, q.data(), q.size() * 4, hipMemcpyHostToDevice);
    fwd.b_step_kv_write(1, 0, ctx, dk, dv);
    fwd.step_kv_write(1, ctx, dk + ctx * row, dv + ctx * row);
    fwd.step_attention(1, ctx, dq, dout);
    hipDeviceSynchronize();
    hipMemcpy(o.data(), dout, o.size() * 4, hipMemcpyDeviceToHost);
    double worst = 0;
    for (uint32_t h = 0; h < H; ++h) for (uint32_t d = 0; d < D; ++d) {
        double mean = 0; for (size_t t = 0; t <= ctx; ++t) mean += v[t * row + (h / 4) * D + d]; mean /= (ctx + 1);
        worst = std::fmax(worst, std::fabs(o[h * D + d] - mean));
    }
    std::printf("uniform-weight decode: max |O - mean(V)| = %.3g\n", worst);
    REQUIRE(worst < 1e-5);
    // one dominant key at position 123: K row = 16 on every dim, q = 1 -> score 16*128*scale = 181 above the rest
    std::vector<float> kd(row, 16.0f);
    hipMemcpy(dk, kd.data(), row * 4, hipMemcpyHostToDevice);
    fwd.step_kv_write(1, 123, dk, dv + 123 * row);
    fwd.step_attention(1, ctx, dq, dout);
    hipDeviceSynchronize();
    hipMemcpy(o.data(), dout, o.size() * 4, hipMemcpyDeviceToHost);
    worst = 0;
    for (uint32_t h = 0; h < H; ++h) for (uint32_t d = 0; d < D; ++d) worst = std::fmax(worst, std::fabs(o[h * D + d] - v[123 * row + (h / 4) * D + d]));
    std::printf("dominant-key decode: max |O - V[123]| = %.3g\n", worst);
    REQUIRE(worst < 1e-6);
    // K RoPE + append, closed forms: with theta_scale = 1 every pair turns by `position` radians.  A key whose pairs are
    // (1, 0) scores sum(cos(pos)) * ... against q = 1 on the first halves only: use it through the F8 cache-free check of k_out.
    {
        std::vector<float> kr(row), kout(row);
        for (size_t x = 0; x < row; ++x) kr[x] = (x % D) < D / 2 ? 1.0f : 0.0f;           // every NEOX pair = (1, 0)
        float* dko; hipMalloc(&dko, row * 4);
        hipMemcpy(dk, kr.data(), row * 4, hipMemcpyHostToDevice);
        vfkv_rope_params rp{VFKV_ROPE_NEOX, D, 1.0f, 1.0f, 1.0f, 1e-6f};
        for (uint32_t pos : {0u, 3u}) {
            fwd.step_k_rope_kv_write(0, pos, 1, dk, dv, nullptr, rp, nullptr, nullptr, dko);
            hipDeviceSynchronize();
            hipMemcpy(kout.data(), dko, row * 4, hipMemcpyDeviceToHost);
            double w2 = 0;
            for (size_t x = 0; x < row; ++x) {
                const double want = (x % D) < D / 2 ? std::cos((double)pos) : std::sin((double)pos);
                w2 = std::fmax(w2, std::fabs(kout[x] - want));
            }
            std::printf("rope (1,0) pairs at position %u: max |k - (cos, sin)| = %.3g\n", pos, w2);
            REQUIRE(w2 < 1e-6);
        }
        hipFree(dko);
    }
    // The whole attention block of a decode token in one call (Q / K norm + RoPE, append, attention), closed form: no norm,
    // theta_scale = 1, so every NEOX pair (1, 1) of q turns by `ctx` radians into (cos - sin, sin + cos); the new K row is zero,
    // row 123 still dominates (score 16 * 128 * cos(ctx) * scale, about 100 above the rest), so O = V[123] again.
    {
        float *dqo, *dz; hipMalloc(&dqo, q.size() * 4); hipMalloc(&dz, row * 4);
        hipMemset(dz, 0, row * 4);
        vfkv_rope_params rp{VFKV_ROPE_NEOX, D, 1.0f, 1.0f, 1.0f, 1e-6f};
        fwd.step_qk_rope_kv_write_attention(1, ctx, dq, nullptr, dqo, dz, dv + ctx * row, nullptr, rp, dout);
        hipDeviceSynchronize();
        std::vector<float> qo(q.size());
        hipMemcpy(qo.data(), dqo, qo.size() * 4, hipMemcpyDeviceToHost);
        hipMemcpy(o.data(), dout, o.size() * 4, hipMemcpyDeviceToHost);
        const double c = std::cos((double)ctx), sn = std::sin((double)ctx);
        double wq = 0; worst = 0;
        for (uint32_t h = 0; h < H; ++h) for (uint32_t d = 0; d < D; ++d) {
            wq = std::fmax(wq, std::fabs(qo[h * D + d] - (d < D / 2 ? c - sn : sn + c)));
            worst = std::fmax(worst, std::fabs(o[h * D + d] - v[123 * row + (h / 4) * D + d]));
        }
        std::printf("fused decode block: max |q_rot - closed form| = %.3g, max |O - V[123]| = %.3g\n", wq, worst);
        REQUIRE(wq < 2e-4 && worst < 1e-6);
        hipFree(dqo); hipFree(dz);
    }
    bool threw = false;
    try { fwd.step_attention(1, ctx + 1, dq, dout); } catch (const Error& e) { threw = e.status == VFKV_ERR_INVALID_ARG; }
    REQUIRE(threw);
    hipFree(dk); hipFree(dv); hipFree(dq); hipFree(dout);
    std::printf("host selftest: all checks passed\n");
    return 0;
}
