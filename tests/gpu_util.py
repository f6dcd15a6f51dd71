"""Shared helpers of the GPU parity tests: seeded inputs, cache encodings through the oracle, and
thin wrappers that drive the library through its C ABI (via the package's ctypes mirror)."""
import ctypes

import numpy as np
import torch

import oracle
import vulkanforge_amd as vf

DEV = "cuda:0"
# tolerances of this path (max-abs vs the CPU oracle): F16 KV 2e-3, FP8 KV 5e-3.  F32 KV follows the
# reference's own test bar of 1e-3 (tests/correctness.rs:2875-2894).
TOL = {vf.KvDtype.F32: 1e-3, vf.KvDtype.F16: 2e-3, vf.KvDtype.F8: 5e-3}
# what f32 arithmetic on identical decoded inputs is expected to reach; a regression guard
TIGHT = 2e-4


def rng(seed):
    return np.random.default_rng(seed)


def fp16_normal(r, shape, scale=1.0):
    """N(0,1)*scale cast to fp16 and back, as the benchmark configurations specify."""
    return (r.standard_normal(shape) * scale).astype(np.float16).astype(np.float32)


def outlier_normal(r, shape, scale=0.5, frac=0.01, mag=40.0):
    """N(0,1)*scale with a seeded `frac` tail at +-mag (exercises E4M3 saturation paths)."""
    x = (r.standard_normal(shape) * scale).astype(np.float32)
    hit = r.random(shape) < frac
    sign = np.where(r.random(shape) < 0.5, -1.0, 1.0).astype(np.float32)
    return np.where(hit, sign * np.float32(mag), x).astype(np.float32)


def encode_np(x, dtype):
    """f32 array -> cache-dtype array exactly as the append kernels must write it."""
    dtype = vf.KvDtype(dtype)
    if dtype == vf.KvDtype.F32:
        return np.ascontiguousarray(x, dtype=np.float32)
    if dtype == vf.KvDtype.F16:
        return oracle.f32_to_f16_bits(x)
    return oracle.f32_to_e4m3(x)


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def to_np(t):
    return t.detach().cpu().numpy()


def read_device(ptr, nbytes):
    """Bytes of a raw device allocation (e.g. the buffers a KvCache owns) as a numpy array."""
    t = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    hip = ctypes.CDLL("libamdhip64.so.7")  # resolves to the runtime already loaded by torch
    rc = hip.hipMemcpy(ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(ptr), ctypes.c_size_t(nbytes), 3)
    assert rc == 0, rc
    return to_np(t)


def gpu_split_reduce(q, k_enc, v_enc, dtype, H, Hkv, D, seq, scale, tile=64, kv_start=0, softcap=0.0,
                     poison=True, interleaved=False):
    """Runs vfkv_flash_attn_split + vfkv_flash_attn_reduce; returns (o, scratch_out, max, sum)."""
    n_tiles = (seq + tile - 1) // tile
    fill = float("nan") if poison else 0.0
    so = torch.full((H, n_tiles, D), fill, device=DEV, dtype=torch.float32)
    sm = torch.full((H, n_tiles), fill, device=DEV, dtype=torch.float32)
    ss = torch.full((H, n_tiles), fill, device=DEV, dtype=torch.float32)
    o = torch.full((H, D), fill, device=DEV, dtype=torch.float32)
    qd, kd, vd = to_dev(q), to_dev(k_enc), to_dev(v_enc)
    nt = vf.Forward.run_flash_attn_split(qd, kd, vd, dtype, so, sm, ss, H, Hkv, D, seq, scale, kv_start=kv_start,
                                         tile=tile, softcap=softcap, interleaved=interleaved)
    assert nt == n_tiles
    vf.Forward.run_flash_attn_reduce(so, sm, ss, o, H, D, n_tiles)
    torch.cuda.synchronize()
    return to_np(o), to_np(so), to_np(sm), to_np(ss)


def gpu_batch(q, k_enc, v_enc, dtype, H, Hkv, D, m, q_start, n_kv, scale, kv_start=0, softcap=0.0):
    o = torch.full((m, H, D), float("nan"), device=DEV, dtype=torch.float32)
    vf.Forward.run_flash_attn_batch(to_dev(q), to_dev(k_enc), to_dev(v_enc), dtype, o, H, Hkv, D, m, q_start, n_kv,
                                    scale, kv_start=kv_start, softcap=softcap)
    torch.cuda.synchronize()
    return to_np(o)
