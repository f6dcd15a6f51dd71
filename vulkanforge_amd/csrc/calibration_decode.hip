// The decode kernels of attn_decode.hip compiled a second time, with wall-clock stamps at four points of every wavefront of the
// matrix-core worker (VFKV_DSTAMP in attn_decode_mfma.h), for libvfkv_calib.so: where a decode launch's time goes.  Same sources,
// same flags; the library proper contains none of this.
#define VFKV_DECODE_STAMPS 1
#include "attn_decode.hip"

#pragma GCC visibility push(default)
extern "C" {

// One launch of the decode worker as vfkv_decode_attention issues it (flash_attn_split.comp:82-162; rows dealt in interleaved runs)
// (the rows are dealt to the n_tiles workgroups per KV head whatever `tile` says) with stamps: q [n_heads, head_dim] f32, k / v layer slabs of seq_len rows (kv_dtype 1 = F16, 2 = FP8), partials into
// so [n_heads][n_tiles][head_dim] / sm, ss [n_heads][n_tiles]; stamps [n_kv_heads][n_tiles][head slices][4 wavefronts][4] uint64
// (device, zeroed by the caller; head slices = ceil(group / 8)).  One caller at a time: the stamp buffer reaches the launcher through
// a file-scope pointer.  0 on success.
int vfkv_calib_decode_stamps(const float* q, const void* k, const void* v, float* so, float* sm, float* ss, uint32_t kv_dtype,
                             uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t seq_len, uint32_t tile,
                             uint32_t n_tiles, float scale, void* stamps, void* stream) {
    if (!q || !k || !v || !so || !sm || !ss || !stamps || n_kv_heads == 0 || n_heads % n_kv_heads != 0 || seq_len == 0 || tile == 0 ||
        n_tiles == 0 || (kv_dtype != vfkv::kF16 && kv_dtype != vfkv::kF8) ||
        (head_dim != 64 && head_dim != 128 && head_dim != 256))
        return -1;
    vfkv::SplitLaunch L;
    L.q = q; L.k = k; L.v = v;
    L.scratch_out = so; L.scratch_max = sm; L.scratch_sum = ss;
    L.dtype = kv_dtype; L.n_heads = n_heads; L.n_kv_heads = n_kv_heads; L.head_dim = head_dim;
    L.seq_len = seq_len; L.kv_start = 0; L.tile = tile; L.tile_first = 0; L.n_tiles = n_tiles;
    L.scale = scale; L.softcap = 0.f;
    L.interleave = true;
    vfkv::g_decode_stamps = (unsigned long long*)stamps;
    const hipError_t e = vfkv::launch_split(L, (hipStream_t)stream);
    vfkv::g_decode_stamps = nullptr;
    return e == hipSuccess ? 0 : -5;
}

}  // extern "C"
#pragma GCC visibility pop
