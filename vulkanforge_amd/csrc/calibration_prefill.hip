// The FP8 prefill kernel of attn_prefill.hip compiled a second time, with wall-clock stamps at seven points of every
// wavefront (VFKV_STAMP in attn_prefill_dma.h), for libvfkv_calib.so: where a launch's time goes outside the tile loop.
// Same sources, same flags; the library proper contains none of this.
#define VFKV_PREFILL_STAMPS 1
#include "attn_prefill.hip"

#pragma GCC visibility push(default)    // the library is built with hidden visibility: only these entry points are exported
extern "C" {

// One launch of the FP8 head_dim-128 prefill kernel (flash_attn_batch.comp:105-208) with stamps: q [m, n_heads, 128] f32, k / v
// FP8 layer slabs of n_kv rows, o [m, n_heads, 128] f32, stamps [n_kv_heads * ceil(m / 16)][8][8] uint64 (device, zeroed by the
// caller; entry i of wavefront w of workgroup (x = KV head, y): 100 MHz wall clock at point i, 0 where a wavefront left before it).
// n_heads / n_kv_heads must be 4 (two head pairs per workgroup) and ceil(m / 16) * n_kv_heads at least 256: below that the launcher
// spreads the head pairs of a KV head over a third grid dimension, which the stamp layout has no room for (-1).  One caller at a time: the stamp buffer reaches the launcher
// through a file-scope pointer.  0 on success.
int vfkv_calib_prefill_stamps(const float* q, const void* k, const void* v, float* o, uint32_t n_heads, uint32_t n_kv_heads,
                              uint32_t m, uint32_t n_kv, uint32_t q_start, float scale, int f16_weights, void* stamps, void* stream) {
    if (!q || !k || !v || !o || !stamps || n_kv_heads == 0 || n_heads != 4u * n_kv_heads || m == 0 || q_start + m > n_kv ||
        (uint64_t)((m + 15u) / 16u) * n_kv_heads < 256u) return -1;
    vfkv::BatchLaunch L{};
    L.q = q; L.k = k; L.v = v; L.o = o;
    L.dtype = vfkv::kF8; L.n_heads = n_heads; L.n_kv_heads = n_kv_heads; L.head_dim = 128;
    L.m = m; L.n_kv = n_kv; L.q_start = q_start; L.kv_start = 0;
    L.scale = scale; L.softcap = 0.f;
    L.f16_weights = f16_weights != 0;
    vfkv::g_prefill_stamps = (unsigned long long*)stamps;
    const hipError_t e = vfkv::launch_batch(L, (hipStream_t)stream);
    vfkv::g_prefill_stamps = nullptr;
    return e == hipSuccess ? 0 : -5;
}

}  // extern "C"
#pragma GCC visibility pop
