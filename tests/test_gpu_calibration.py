"""The benchmark's calibration library: its instrumented copies of the FP8 prefill kernel and of the decode worker must compute what
the library's own kernels compute (same sources, stamps added), and their stamps must be in order."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, encode_np, fp16_normal, rng, to_dev, to_np

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def calib():
    lib = C.CDLL(os.path.join(ROOT, "vulkanforge_amd", "libvfkv_calib.so"))
    lib.vfkv_calib_prefill_stamps.argtypes = [C.c_void_p] * 4 + [C.c_uint32] * 5 + [C.c_float, C.c_int, C.c_void_p, C.c_void_p]
    lib.vfkv_calib_decode_stamps.argtypes = [C.c_void_p] * 6 + [C.c_uint32] * 7 + [C.c_float, C.c_void_p, C.c_void_p]
    return lib


# (shapes the launcher runs as one workgroup per (KV head, query block): the layout of the stamp buffer)
@pytest.mark.parametrize("m,q_start,f16w", [(512, 300, 0), (500, 1300, 0), (520, 2517, 1)])
def test_instrumented_prefill_kernel_equals_the_library_kernel(m, q_start, f16w):
    heads, hkv, d = 32, 8, 128
    n_kv = q_start + m
    r = rng(m * 7 + q_start)
    q = fp16_normal(r, (m, heads, d))
    k, v = encode_np(fp16_normal(r, (n_kv, hkv, d)), vf.KvDtype.F8), encode_np(fp16_normal(r, (n_kv, hkv, d)), vf.KvDtype.F8)
    scale = float(1.0 / np.sqrt(d))
    qd, kd, vd = to_dev(q), to_dev(k.reshape(n_kv, -1)), to_dev(v.reshape(n_kv, -1))
    o_lib = torch.full((m, heads, d), float("nan"), device=DEV)
    vf.Forward.run_flash_attn_batch(qd, kd, vd, vf.KvDtype.F8, o_lib, heads, hkv, d, m, q_start, n_kv, scale, f16_weights=bool(f16w))
    o_cal = torch.full((m, heads, d), float("nan"), device=DEV)
    nb = (m + 15) // 16
    stamps = torch.zeros((nb, hkv, 8, 8), dtype=torch.int64, device=DEV)
    print(f"case m={m} q_start={q_start} f16w={f16w}", flush=True)
    rc = calib().vfkv_calib_prefill_stamps(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o_cal.data_ptr(), heads, hkv, m, n_kv,
                                           q_start, scale, f16w, stamps.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(o_lib, o_cal)                       # bit for bit: the same instructions but for the stamps
    ref = oracle.attn_batch_ref(q, k, v, int(vf.KvDtype.F8), m, n_kv, heads, hkv, d, q_start, scale)
    assert np.abs(to_np(o_cal) - ref).max() < (6e-3 if f16w else 1e-3)
    s = stamps.cpu().numpy()
    assert (s[..., 0] > 0).all() and (s[..., 2] >= s[..., 1]).all() and (s[..., 1] >= s[..., 0]).all()
    live = s[..., 6] > 0                                  # wavefronts whose lanes all lie past the last query leave before the merge
    assert live.any() and (s[..., 6][live] >= s[..., 2][live]).all()


def test_calibration_entry_points_reject_bad_arguments():
    lib = calib()
    assert lib.vfkv_calib_prefill_stamps(None, None, None, None, 32, 8, 16, 32, 16, 0.1, 0, None, None) == -1
    x = torch.zeros(16, device=DEV)
    # 16 heads over 8 KV heads: not the two-head-pairs form the instrumented copy is for
    assert lib.vfkv_calib_prefill_stamps(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 16, 8, 16, 32, 16, 0.1, 0,
                                         x.data_ptr(), None) == -1
    # 64 queries x 8 KV heads: the launcher would use a third grid dimension that the stamp buffer has no room for
    assert lib.vfkv_calib_prefill_stamps(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 32, 8, 64, 364, 300, 0.1, 0,
                                         x.data_ptr(), None) == -1


@pytest.mark.parametrize("dtype,heads,hkv,d,seq,tile", [(vf.KvDtype.F8, 32, 8, 128, 3000, 128), (vf.KvDtype.F16, 16, 8, 256, 1500, 64),
                                                         (vf.KvDtype.F8, 64, 8, 64, 777, 64)])
def test_instrumented_decode_worker_equals_the_library_worker(dtype, heads, hkv, d, seq, tile):
    r = rng(seq + d)
    q = fp16_normal(r, (heads, d))
    k, v = encode_np(fp16_normal(r, (seq, hkv, d)), dtype), encode_np(fp16_normal(r, (seq, hkv, d)), dtype)
    scale = float(1.0 / np.sqrt(d))
    qd, kd, vd = to_dev(q), to_dev(k.reshape(seq, -1)), to_dev(v.reshape(seq, -1))
    nt = (seq + tile - 1) // tile
    bufs = [[torch.full((heads, nt, d), float("nan"), device=DEV), torch.full((heads, nt), float("nan"), device=DEV),
             torch.full((heads, nt), float("nan"), device=DEV)] for _ in range(2)]
    assert vf.Forward.run_flash_attn_split(qd, kd, vd, dtype, *bufs[0], heads, hkv, d, seq, scale, tile=tile, interleaved=True) == nt
    stamps = torch.zeros((hkv, nt, 1, 4, 4), dtype=torch.int64, device=DEV)
    print(f"case {dtype.label()} H={heads} Hkv={hkv} D={d} seq={seq} tile={tile}", flush=True)
    rc = calib().vfkv_calib_decode_stamps(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), *(b.data_ptr() for b in bufs[1]), int(dtype), heads,
                                          hkv, d, seq, tile, nt, scale, stamps.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    for a, b in zip(*bufs):
        assert torch.equal(a, b)                           # bit for bit
    o = torch.empty((heads, d), device=DEV)
    vf.Forward.run_flash_attn_reduce(*bufs[1], o, heads, d, nt)
    ref = oracle.attn_decode_ref(q, k, v, int(dtype), heads, hkv, d, seq, scale)
    assert np.abs(to_np(o) - ref).max() < 5e-3
    s = stamps.cpu().numpy()
    assert (s[..., 0] > 0).all() and (s[..., 1] >= s[..., 0]).all() and (s[..., 2] >= s[..., 1]).all() and (s[..., 3] >= s[..., 2]).all()
