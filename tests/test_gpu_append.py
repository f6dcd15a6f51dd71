"""GPU parity of the append / expansion kernels, through the C ABI, bit-exact against the oracle."""
import os

import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, outlier_normal, read_device, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def _store_fp8(x, n=None, offset=0, dst_bytes=None):
    n = x.size if n is None else n
    total = dst_bytes or (offset + ((n + 3) // 4) * 4 + 64)
    dst = torch.full((total,), 0xAA, dtype=torch.uint8, device=DEV)
    vf.Forward.run_kv_store_fp8(to_dev(x), dst, n, offset)
    torch.cuda.synchronize()
    return to_np(dst)


def test_store_fp8_golden_vectors(golden_dir):
    z = np.load(os.path.join(golden_dir, "e4m3_encode_vectors.npz"))
    x = z["bits"].view(np.float32)
    got = _store_fp8(x)[: x.size]
    bad = np.nonzero(got != z["expected"])[0]
    assert bad.size == 0, [(hex(z["bits"][i]), hex(got[i]), hex(z["expected"][i])) for i in bad[:8]]


def test_store_fp8_every_upper_half_pattern_and_random_bits():
    r = rng(1)
    bits = np.concatenate([(np.arange(1 << 16, dtype=np.uint32) << 16),
                           r.integers(0, 1 << 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    got = _store_fp8(x)[: x.size]
    exp = oracle.f32_to_e4m3(x)
    bad = np.nonzero(got != exp)[0]
    assert bad.size == 0, [(hex(bits[i]), hex(got[i]), hex(exp[i])) for i in bad[:8]]


def test_store_fp8_benchmark_distribution_with_outliers():
    x = outlier_normal(rng(2), 32 * 1024)
    assert (np.abs(x) == 40).sum() > 100
    assert (_store_fp8(x)[: x.size] == oracle.f32_to_e4m3(x)).all()


@pytest.mark.parametrize("n,offset", ((1, 0), (3, 4), (5, 8), (1023, 1024), (1024, 4096), (4097, 12)))
def test_store_fp8_offsets_and_ragged_tail(n, offset):
    x = (rng(n).standard_normal(n + 7) * 3).astype(np.float32)
    got = _store_fp8(x, n=n, offset=offset)
    ref = np.full(got.shape, 0xAA, dtype=np.uint8)
    assert oracle.kv_store_fp8(x, ref, n, offset) == 0
    assert (got == ref).all()


def test_store_fp8_rejects_unaligned_offset():
    x = to_dev(np.zeros(8, dtype=np.float32))
    dst = torch.zeros(64, dtype=torch.uint8, device=DEV)
    with pytest.raises(vf.VfkvError) as e:
        vf.Forward.run_kv_store_fp8(x, dst, 8, 2)
    assert e.value.status == -3


@pytest.mark.parametrize("n,offset", ((1, 0), (2, 4), (515, 512), (1024, 0), (8193, 20)))
def test_copy_fp16_matches_oracle(n, offset):
    r = rng(10 + n)
    x = np.concatenate([r.standard_normal(n) * 10, [65504.0, 65520.0, 1e-8, 6e-8, -0.0, 3.0e38]]).astype(np.float32)[:max(n, 1)]
    if n >= 8:
        x[:6] = [65504.0, 65520.0, 1e-8, 6.1e-5, -0.0, 3.0e38]
    total = offset + ((n + 1) // 2) * 4 + 64
    dst = torch.full((total,), 0xAA, dtype=torch.uint8, device=DEV)
    vf.Forward.run_kv_copy_fp16(to_dev(x), dst, n, offset)
    torch.cuda.synchronize()
    ref = np.full(total, 0xAA, dtype=np.uint8)
    assert oracle.kv_copy_fp16(x, ref, n, offset) == 0
    assert (to_np(dst) == ref).all()


def test_copy_fp16_random_bit_patterns():
    bits = rng(12).integers(0, 1 << 32, size=1 << 18, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    x = x[: (x.size // 2) * 2]
    dst = torch.zeros(x.size * 2, dtype=torch.uint8, device=DEV)
    vf.Forward.run_kv_copy_fp16(to_dev(x), dst, x.size, 0)
    torch.cuda.synchronize()
    assert (to_np(dst).view(np.uint16) == oracle.f32_to_f16_bits(x)).all()


@pytest.mark.parametrize("n,src_off,dst_off", ((256, 0, 0), (1 << 20, 0, 0), (1000, 0, 0), (1000, 1, 0),
                                               (4099, 0, 1), (17, 3, 5)))
def test_fp8_to_f16_matches_oracle(n, src_off, dst_off):
    r = rng(n)
    codes = r.integers(0, 256, size=n, dtype=np.uint16).astype(np.uint8)
    codes[: min(n, 256)] = np.arange(min(n, 256), dtype=np.uint8)
    src = torch.zeros(n + 64, dtype=torch.uint8, device=DEV)
    src[src_off:src_off + n] = to_dev(codes)
    dst = torch.full((n + 64,), 0x5555, dtype=torch.int16, device=DEV)
    vf.Forward.run_kv_fp8_to_f16(src.data_ptr() + src_off, dst.data_ptr() + 2 * dst_off, n)
    torch.cuda.synchronize()
    got = to_np(dst).view(np.uint16)
    exp = oracle.kv_fp8_to_f16(codes)
    nan = (codes & 0x7F) == 0x7F
    g = got[dst_off:dst_off + n]
    assert (g[~nan] == exp[~nan]).all()
    assert np.isnan(g[nan].view(np.float16)).all()
    assert (got[:dst_off] == 0x5555).all() and (got[dst_off + n:] == 0x5555).all()


@pytest.mark.parametrize("dtype", list(vf.KvDtype))
def test_kv_write_lands_at_the_reference_offsets(dtype):
    L, Hkv, D, S = 3, 8, 128, 40
    cache = vf.KvCache(vf.KvCacheConfig(L, Hkv, D, S, dtype=dtype))
    cache.zero_fill()
    fwd = vf.Forward(cache, 32)
    es = dtype.element_size()
    ref_k = np.zeros(cache.bytes_per_buffer(), dtype=np.uint8)
    ref_v = np.zeros_like(ref_k)
    r = rng(77)

    def ref_write(buf, x, n, off):
        if dtype == vf.KvDtype.F8:
            oracle.kv_store_fp8(x, buf, n, off)
        elif dtype == vf.KvDtype.F16:
            oracle.kv_copy_fp16(x, buf, n, off)
        else:
            buf[off:off + 4 * n] = x[:n].view(np.uint8)

    for layer, pos, n_tok in ((0, 0, 1), (1, 7, 1), (2, 39, 1), (1, 10, 13), (0, 1, 39)):
        k = outlier_normal(r, (n_tok, Hkv * D))
        v = outlier_normal(r, (n_tok, Hkv * D))
        if n_tok == 1:
            fwd.step_kv_write(layer, pos, to_dev(k), to_dev(v))
        else:
            fwd.b_step_kv_write(layer, pos, n_tok, to_dev(k), to_dev(v))
        off = cache.pos_offset_bytes(layer, pos)
        assert off == (layer * S + pos) * Hkv * D * es
        ref_write(ref_k, k.ravel(), k.size, off)
        ref_write(ref_v, v.ravel(), v.size, off)
    torch.cuda.synchronize()
    nb = cache.bytes_per_buffer()
    assert (read_device(cache.k_ptr, nb) == ref_k).all() and (read_device(cache.v_ptr, nb) == ref_v).all()
    with pytest.raises(vf.VfkvError):
        zeros = to_dev(np.zeros((11, Hkv * D), np.float32))
        fwd.b_step_kv_write(0, 30, 11, zeros, zeros)
    # zero_layer clears exactly one slab (kv_cache.rs:389-407)
    cache.zero_layer(1)
    torch.cuda.synchronize()
    lo, sz = cache.layer_offset_bytes(1), cache.layer_size_bytes(1)
    ref_k[lo:lo + sz] = 0
    ref_v[lo:lo + sz] = 0
    assert (read_device(cache.k_ptr, nb) == ref_k).all() and (read_device(cache.v_ptr, nb) == ref_v).all()
    cache.destroy()
