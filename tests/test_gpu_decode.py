"""GPU parity of split-K decode attention (worker + log-sum-exp merge) through the C ABI.

Bars (max-abs against the CPU oracle on the same decoded inputs): F16 KV 2e-3, FP8 KV 5e-3, F32 KV
1e-3 (the reference's own bar, tests/correctness.rs:2875-2894).  TIGHT is what f32 arithmetic is
expected to reach and guards against regressions hiding inside the wide bars."""
import os

import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import (DEV, TIGHT, TOL, encode_np, fp16_normal, gpu_split_reduce, outlier_normal, rng, to_dev,
                      to_np)
from refgen import D, H, HKV, decode_inputs

pytestmark = pytest.mark.gpu
SCALE = float(np.float32(1.0) / np.sqrt(np.float32(D)))


def test_single_hip_runtime_in_process():
    torch.cuda.synchronize()
    vf.lib()
    libs = {line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line}
    assert len(libs) == 1, libs


@pytest.mark.parametrize("seq", (64, 200, 2048))
def test_reference_split_fixture_f32_tile64(golden_dir, seq):
    # tests/correctness.rs:2791-2894: FlashAttnSplit + FlashAttnReduce, F32 KV, TILE 64, tol 1e-3
    golden = np.load(os.path.join(golden_dir, "attn_cases.npz"))[f"decode_seq{seq}_out"]
    q, k, v = decode_inputs(seq)
    o, so, sm, ss = gpu_split_reduce(q, k, v, vf.KvDtype.F32, H, HKV, D, seq, SCALE, tile=64)
    assert np.isfinite(o).all()
    assert np.abs(o - golden).max() < 1e-3
    assert np.abs(o - golden).max() < 2e-5
    # the per-tile partials have the reference's meaning and layout (flash_attn_split.comp:147-161)
    eo, em, es = oracle.attn_split(q, k, v, oracle.F32, H, HKV, D, seq, SCALE, tile=64)
    assert np.abs(sm - em).max() < 1e-5
    assert np.abs(ss - es).max() < 1e-4 * max(1.0, np.abs(es).max())
    assert np.abs(so - eo).max() < 1e-4 * max(1.0, np.abs(eo).max())


def test_seq1_returns_v0_exactly():
    q, k, v = decode_inputs(1)
    o, *_ = gpu_split_reduce(q, k, v, vf.KvDtype.F32, H, HKV, D, 1, SCALE, tile=64)
    assert (o == np.repeat(v[0], H // HKV, axis=0)).all()


CASES = [
    # dtype, H, Hkv, D, seq, tile, kv_start, softcap
    (vf.KvDtype.F8, 32, 8, 128, 2049, 512, 0, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 777, 64, 0, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 1000, 256, 300, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 1000, 128, 999, 0.0),
    (vf.KvDtype.F8, 8, 8, 128, 500, 64, 0, 0.0),      # G = 1
    (vf.KvDtype.F8, 16, 8, 128, 500, 192, 17, 30.0),  # G = 2
    (vf.KvDtype.F8, 24, 8, 64, 500, 64, 0, 0.0),      # G = 3
    (vf.KvDtype.F8, 64, 8, 128, 300, 64, 0, 0.0),     # G = 8 (two head groups)
    (vf.KvDtype.F8, 16, 2, 256, 600, 128, 0, 0.0),
    (vf.KvDtype.F8, 8, 2, 512, 300, 64, 100, 0.0),
    (vf.KvDtype.F8, 16, 2, 512, 2100, 256, 0, 30.0),  # head_dim 512 on the matrix-core worker: G = 8, soft-cap, several runs per stream
    (vf.KvDtype.F8, 4, 4, 512, 777, 96, 333, 0.0),    # head_dim 512, G = 1, tile not a multiple of the run, window inside a tile
    (vf.KvDtype.F8, 16, 4, 64, 900, 320, 0, 0.0),
    (vf.KvDtype.F8, 32, 2, 128, 700, 1024, 0, 0.0),   # G = 16: two slices of 8 heads, one ragged tile
    (vf.KvDtype.F8, 24, 2, 128, 1300, 448, 5, 0.0),   # G = 12: slices of 8 and 4 heads
    (vf.KvDtype.F8, 32, 8, 128, 3000, 1024, 1900, 0.0),  # window starting inside a tile, several runs per wavefront
    (vf.KvDtype.F8, 32, 8, 128, 333, 16, 40, 0.0),       # tiles shorter than a run of the matrix-core worker
    (vf.KvDtype.F16, 16, 8, 64, 1000, 48, 0, 0.0),       # tile not a multiple of the run length
    (vf.KvDtype.F16, 20, 4, 128, 1111, 320, 0, 20.0), # G = 5 with soft-cap
    (vf.KvDtype.F16, 32, 8, 128, 2049, 512, 0, 0.0),
    (vf.KvDtype.F16, 16, 8, 256, 1500, 256, 0, 50.0),
    (vf.KvDtype.F16, 16, 8, 256, 1500, 64, 1100, 50.0),
    (vf.KvDtype.F16, 8, 4, 512, 200, 64, 0, 0.0),
    (vf.KvDtype.F16, 8, 2, 512, 1900, 192, 700, 40.0),   # head_dim 512 over a 2-byte cache: window, soft-cap
    (vf.KvDtype.F16, 12, 4, 64, 1000, 512, 0, 0.0),
    # tiles with fewer full runs than the workgroup has run streams (the reference's 64-key tiles): runs of half the rows
    (vf.KvDtype.F8, 16, 8, 256, 700, 64, 100, 0.0),
    (vf.KvDtype.F16, 32, 8, 128, 900, 64, 0, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 900, 96, 50, 30.0),      # 96-key tiles: three full runs, or six of half the rows
    (vf.KvDtype.F8, 16, 8, 64, 900, 128, 0, 0.0),        # head_dim 64: two full runs of 64 rows per tile
    (vf.KvDtype.F32, 32, 8, 128, 700, 128, 0, 0.0),
    (vf.KvDtype.F32, 8, 2, 256, 300, 64, 50, 0.0),
    (vf.KvDtype.F32, 4, 2, 64, 300, 64, 0, 10.0),
    # head widths between the tiled ones (FP8 / F16): the next wider matrix-core worker with its tail masked off
    (vf.KvDtype.F16, 6, 2, 80, 333, 64, 10, 0.0),
    (vf.KvDtype.F8, 4, 4, 96, 333, 128, 0, 0.0),
    (vf.KvDtype.F8, 32, 32, 96, 1500, 256, 0, 0.0),      # Phi-3-mini geometry (G = 1)
    (vf.KvDtype.F16, 32, 32, 96, 777, 64, 100, 0.0),     # 64-key tiles (runs of 16 rows), window inside a tile
    (vf.KvDtype.F16, 32, 32, 80, 1200, 320, 0, 30.0),    # Phi-2 geometry, soft-cap
    (vf.KvDtype.F8, 16, 4, 112, 900, 128, 50, 0.0),
    (vf.KvDtype.F8, 24, 2, 96, 800, 512, 0, 0.0),        # G = 12: slices of 8 and 4 heads
    (vf.KvDtype.F8, 8, 2, 160, 700, 64, 0, 0.0),         # on the worker for 256
    (vf.KvDtype.F16, 16, 8, 192, 1300, 256, 300, 50.0),
    (vf.KvDtype.F16, 8, 4, 224, 500, 128, 0, 0.0),
    (vf.KvDtype.F32, 4, 2, 96, 300, 64, 0, 0.0),         # F32 caches: the padded form of the f32 matrix-core worker
    (vf.KvDtype.F32, 32, 32, 80, 1100, 256, 100, 20.0),
    (vf.KvDtype.F32, 20, 1, 112, 700, 128, 0, 0.0),      # G = 20: slices of 16 and 4 heads
    (vf.KvDtype.F32, 8, 4, 192, 900, 512, 333, 0.0),
    (vf.KvDtype.F32, 6, 2, 160, 400, 64, 0, 50.0),
    (vf.KvDtype.F32, 4, 4, 224, 200, 64, 0, 0.0),
    # FP8 heads of 64 elements over long spans (131 072 / n_kv_heads visible rows and more): interleaved launches take two
    # neighbouring KV heads as one row of 128 bytes (groups of up to four heads)
    (vf.KvDtype.F8, 32, 8, 64, 17000, 1024, 0, 0.0),     # G = 4: the eight heads of a pair fill the worker's columns
    (vf.KvDtype.F8, 24, 8, 64, 20000, 512, 3000, 30.0),  # G = 3, window, soft-cap
    (vf.KvDtype.F8, 6, 6, 64, 16500, 2048, 0, 0.0),      # G = 1
    (vf.KvDtype.F8, 20, 4, 64, 16400, 4096, 0, 0.0),     # G = 5: too many heads for a pair, separate heads
    (vf.KvDtype.F8, 12, 3, 64, 16400, 4096, 0, 0.0),     # odd number of KV heads: separate heads
    (vf.KvDtype.F8, 32, 32, 64, 4500, 512, 300, 0.0),    # 32 KV heads: pairs from 4 096 visible rows on
    (vf.KvDtype.F8, 64, 16, 64, 8300, 1024, 0, 20.0),    # 16 KV heads: from 8 192 on
    # shapes only the generic worker covers
    (vf.KvDtype.F32, 4, 2, 512, 200, 64, 0, 0.0),
    (vf.KvDtype.F32, 3, 1, 50, 100, 64, 0, 0.0),
    (vf.KvDtype.F16, 4, 2, 72, 300, 64, 0, 0.0),
    (vf.KvDtype.F16, 4, 2, 40, 200, 64, 0, 0.0),
]


@pytest.mark.parametrize("dtype,heads,hkv,d,seq,tile,kv_start,cap", CASES)
def test_split_reduce_matches_oracle(dtype, heads, hkv, d, seq, tile, kv_start, cap):
    r = rng(hash((int(dtype), heads, hkv, d, seq, tile)) % (1 << 31))
    q = fp16_normal(r, (heads, d))
    kf = outlier_normal(r, (seq, hkv, d)) if dtype == vf.KvDtype.F8 else fp16_normal(r, (seq, hkv, d))
    vfl = outlier_normal(r, (seq, hkv, d)) if dtype == vf.KvDtype.F8 else fp16_normal(r, (seq, hkv, d))
    k, v = encode_np(kf, dtype), encode_np(vfl, dtype)
    scale = float(1.0 / np.sqrt(d))
    print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} seq={seq} tile={tile} kv_start={kv_start} cap={cap}",
          flush=True)
    o, so, sm, ss = gpu_split_reduce(q, k, v, dtype, heads, hkv, d, seq, scale, tile=tile, kv_start=kv_start,
                                     softcap=cap)
    ref = oracle.attn_decode_ref(q, k, v, int(dtype), heads, hkv, d, seq, scale, kv_start=kv_start, softcap=cap)
    assert np.isfinite(o).all() and np.isfinite(so).all()       # NaN-poisoned scratch fully overwritten
    err = np.abs(o - ref).max()
    assert err < TOL[dtype], err
    assert err < TIGHT * max(1.0, np.abs(ref).max()), err
    # tiles wholly below the window are empty partials (flash_attn_split.comp:64-69)
    dead = kv_start // tile
    if dead:
        assert (sm[:, :dead] == np.float32(-1e30)).all() and (ss[:, :dead] == 0).all() and (so[:, :dead] == 0).all()


# The interleaved worker exists with runs of 32 rows (64 at head_dim 64) and with runs of half that; which one a launch
# takes follows from the full runs per run stream (four streams per workgroup = per tile of the call).  Per shape: many
# tiles (at most one and a half full runs per stream: half runs) and two tiles (full runs), each with a window that starts
# inside a run and a ragged end.
RUN_LENGTH_CASES = [
    (vf.KvDtype.F8, 32, 8, 128, 1501, 64, 0, 0.0),     # 24 tiles, 47 full runs over 96 streams: runs of 16 rows
    (vf.KvDtype.F8, 32, 8, 128, 1501, 768, 333, 0.0),  # 2 tiles, 8 streams: runs of 32 rows
    (vf.KvDtype.F8, 16, 4, 64, 1501, 64, 0, 20.0),     # head_dim 64: runs of 32 rows
    (vf.KvDtype.F8, 16, 4, 64, 1501, 768, 333, 0.0),   # runs of 64 rows
    (vf.KvDtype.F16, 32, 8, 128, 1501, 64, 0, 0.0),    # runs of 16 rows
    (vf.KvDtype.F16, 32, 8, 128, 650, 384, 77, 0.0),   # 2 tiles, 21 full runs over 8 streams (more than 1.5 per stream): 32 rows
    (vf.KvDtype.F16, 32, 8, 128, 1501, 768, 0, 30.0),  # 47 full runs over 8 streams, with the soft-cap: 32 rows
    (vf.KvDtype.F16, 8, 4, 64, 1501, 768, 333, 0.0),   # F16 rows of 64: 32 rows at every length
    (vf.KvDtype.F8, 16, 8, 256, 1501, 768, 333, 0.0),  # FP8 rows of 256: 16 rows at every length
    (vf.KvDtype.F16, 16, 8, 256, 1501, 768, 333, 50.0),
]


@pytest.mark.parametrize("dtype,heads,hkv,d,seq,tile,kv_start,cap", RUN_LENGTH_CASES)
def test_interleaved_worker_both_run_lengths(dtype, heads, hkv, d, seq, tile, kv_start, cap):
    test_interleaved_split_reduce_matches_oracle(dtype, heads, hkv, d, seq, tile, kv_start, cap)


@pytest.mark.parametrize("dtype,heads,hkv,d,seq,tile,kv_start,cap", CASES)
def test_interleaved_split_reduce_matches_oracle(dtype, heads, hkv, d, seq, tile, kv_start, cap):
    # vfkv_flash_attn_split_interleaved: the partials are combs of rows rather than tiles, so only the merged
    # output is compared; the same launch with contiguous tiles must agree to rounding
    r = rng(hash((int(dtype), heads, hkv, d, seq, tile, 7)) % (1 << 31))
    q = fp16_normal(r, (heads, d))
    kf = outlier_normal(r, (seq, hkv, d)) if dtype == vf.KvDtype.F8 else fp16_normal(r, (seq, hkv, d))
    vfl = outlier_normal(r, (seq, hkv, d)) if dtype == vf.KvDtype.F8 else fp16_normal(r, (seq, hkv, d))
    k, v = encode_np(kf, dtype), encode_np(vfl, dtype)
    scale = float(1.0 / np.sqrt(d))
    print(f"case interleaved dtype={dtype.label()} H={heads} Hkv={hkv} D={d} seq={seq} tile={tile} "
          f"kv_start={kv_start} cap={cap}", flush=True)
    o, so, sm, ss = gpu_split_reduce(q, k, v, dtype, heads, hkv, d, seq, scale, tile=tile, kv_start=kv_start,
                                     softcap=cap, interleaved=True)
    o_tiles, *_ = gpu_split_reduce(q, k, v, dtype, heads, hkv, d, seq, scale, tile=tile, kv_start=kv_start,
                                   softcap=cap)
    ref = oracle.attn_decode_ref(q, k, v, int(dtype), heads, hkv, d, seq, scale, kv_start=kv_start, softcap=cap)
    assert np.isfinite(o).all() and np.isfinite(so).all() and np.isfinite(sm).all() and np.isfinite(ss).all()
    err = np.abs(o - ref).max()
    assert err < TOL[dtype], err
    assert err < TIGHT * max(1.0, np.abs(ref).max()), err
    assert np.abs(o - o_tiles).max() < TIGHT * max(1.0, np.abs(ref).max())


def test_tile_invariance_and_linearity_full_size_fp8():
    # size-independent properties at the benchmark's largest single-layer shape (32768 keys, FP8)
    seq, heads, hkv, d = 32768, 32, 8, 128
    g = torch.Generator(device=DEV).manual_seed(5)
    kf = torch.randn((seq, hkv * d), device=DEV, generator=g)
    v1 = torch.randn((seq, hkv * d), device=DEV, generator=g)
    v2 = torch.randn((seq, hkv * d), device=DEV, generator=g)
    q = torch.randn((heads, d), device=DEV, generator=g).half().float()
    scale = float(1.0 / np.sqrt(d))

    def enc(x):
        out = torch.empty(x.numel(), dtype=torch.uint8, device=DEV)
        vf.Forward.run_kv_store_fp8(x, out, x.numel(), 0)
        return out

    def dec(b):
        out = torch.empty(b.numel(), dtype=torch.float16, device=DEV)
        vf.Forward.run_kv_fp8_to_f16(b, out, b.numel())
        return out.float()

    k8, va, vb = enc(kf), enc(v1), enc(v2)
    vsum = dec(va) + dec(vb)            # exact in f32; encode it as an F32-KV value tensor
    ones = enc(torch.ones_like(v1))

    def attn(k, v, dt, tile):
        n_tiles = (seq + tile - 1) // tile
        so = torch.empty((heads, n_tiles, d), device=DEV)
        sm = torch.empty((heads, n_tiles), device=DEV)
        ss = torch.empty((heads, n_tiles), device=DEV)
        o = torch.empty((heads, d), device=DEV)
        vf.Forward.run_flash_attn_split(q, k, v, dt, so, sm, ss, heads, hkv, d, seq, scale, tile=tile)
        vf.Forward.run_flash_attn_reduce(so, sm, ss, o, heads, d, n_tiles)
        return o

    o512 = attn(k8, va, vf.KvDtype.F8, 512)
    for tile in (64, 1024, 4096):
        assert (attn(k8, va, vf.KvDtype.F8, tile) - o512).abs().max().item() < 2e-5
    assert (attn(k8, ones, vf.KvDtype.F8, 512) - 1.0).abs().max().item() < 1e-5      # weights sum to one
    ob = attn(k8, vb, vf.KvDtype.F8, 512)
    # linearity in V needs one K for all three runs: decode K to f32 and use the F32-KV kernels
    kf32 = dec(k8)
    oa32 = attn(kf32, dec(va), vf.KvDtype.F32, 512)
    ob32 = attn(kf32, dec(vb), vf.KvDtype.F32, 512)
    os32 = attn(kf32, vsum, vf.KvDtype.F32, 512)
    assert (oa32 + ob32 - os32).abs().max().item() < 2e-5
    # the FP8-KV and F32-KV kernels see the same decoded values
    assert (oa32 - o512).abs().max().item() < 2e-5 and (ob32 - ob).abs().max().item() < 2e-5
    # and one full-size comparison with the oracle
    ref = oracle.attn_decode_ref(to_np(q), to_np(k8).reshape(seq, hkv, d), to_np(va).reshape(seq, hkv, d),
                                 oracle.F8, heads, hkv, d, seq, scale)
    assert np.abs(to_np(o512) - ref).max() < 5e-3
    assert np.abs(to_np(o512) - ref).max() < TIGHT


@pytest.mark.parametrize("n_tiles", (1, 2, 33, 64, 65, 127, 128, 129, 200, 256, 257, 700))
@pytest.mark.parametrize("heads,d", ((6, 64), (8, 256), (3, 512), (5, 80)))
def test_reduce_alone_matches_oracle_for_every_tile_count(n_tiles, heads, d):
    # flash_attn_reduce.comp on synthetic partials: every merge kernel (one wavefront up to 64 tiles, four up to 256,
    # the looping ones beyond and for head sizes that are no multiple of 64), with empty tiles mixed in
    r = rng(n_tiles * 1000 + d)
    so = r.standard_normal((heads, n_tiles, d)).astype(np.float32)
    sm = (r.standard_normal((heads, n_tiles)) * 6).astype(np.float32)
    ss = (r.random((heads, n_tiles)) * 50 + 0.5).astype(np.float32)
    empty = r.random((heads, n_tiles)) < 0.2
    empty[:, r.integers(0, n_tiles)] = False                 # every head keeps a live tile
    if n_tiles > 130:
        empty[0, 64:128] = True                              # a whole wavefront's share of tiles without keys
    so[empty] = 0.0
    sm[empty] = -1e30
    ss[empty] = 0.0
    o = torch.full((heads, d), float("nan"), device=DEV)
    vf.Forward.run_flash_attn_reduce(to_dev(so), to_dev(sm), to_dev(ss), o, heads, d, n_tiles)
    torch.cuda.synchronize()
    ref = oracle.attn_reduce(so, sm, ss)
    assert np.abs(to_np(o) - ref).max() < 2e-6 * max(1.0, np.abs(ref).max())


def _cache_with_history(dtype, n_layers, hkv, d, max_seq, fill, seed, hd=None, kvh=None):
    cfg = vf.KvCacheConfig(n_layers, hkv, d, max_seq, hd, kvh, dtype)
    cache = vf.KvCache(cfg)
    cache.zero_fill()
    r = rng(seed)
    hist = []
    fwd = vf.Forward(cache, 1)
    for layer in range(n_layers):
        row = cache.kv_heads_for(layer) * cache.head_dim_for(layer)
        k, v = fill(r, (max_seq, row)), fill(r, (max_seq, row))
        fwd.b_step_kv_write(layer, 0, max_seq, to_dev(k), to_dev(v))
        hist.append((k, v))
    torch.cuda.synchronize()
    return cache, hist


def test_config1_append_then_decode_f16():
    # benchmark configuration 1: one layer, F16 KV, 32/8/128, context 2048, append one token, attend
    heads, hkv, d, ctx = 32, 8, 128, 2048
    cache, hist = _cache_with_history(vf.KvDtype.F16, 1, hkv, d, ctx + 1, fp16_normal, 11)
    fwd = vf.Forward(cache, heads)
    r = rng(12)
    k_new, v_new, q = fp16_normal(r, (1, hkv * d)), fp16_normal(r, (1, hkv * d)), fp16_normal(r, (heads, d))
    fwd.step_kv_write(0, ctx, to_dev(k_new), to_dev(v_new))
    o = torch.full((heads, d), float("nan"), device=DEV)
    fwd.run_scalar_attn(0, ctx, to_dev(q), o)
    torch.cuda.synchronize()
    k_all, v_all = hist[0][0].copy(), hist[0][1].copy()
    k_all[ctx], v_all[ctx] = k_new[0], v_new[0]
    ke, ve = encode_np(k_all, vf.KvDtype.F16), encode_np(v_all, vf.KvDtype.F16)
    ref = oracle.attn_decode_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), oracle.F16, heads, hkv, d,
                                 ctx + 1, fwd.attn_scale)
    err = np.abs(to_np(o) - ref).max()
    assert err < 2e-3 and err < TIGHT, err


def test_config2_fp8_outliers_append_then_decode_two_layers():
    # benchmark configuration 2 geometry (FP8 KV, context 8192, +-40 outlier tail), two layers of the 32
    heads, hkv, d, ctx = 32, 8, 128, 8192
    cache, hist = _cache_with_history(vf.KvDtype.F8, 2, hkv, d, ctx + 1, outlier_normal, 21)
    fwd = vf.Forward(cache, heads)
    r = rng(22)
    for layer in range(2):
        k_new, v_new = outlier_normal(r, (1, hkv * d)), outlier_normal(r, (1, hkv * d))
        q = fp16_normal(r, (heads, d))
        fwd.step_kv_write(layer, ctx, to_dev(k_new), to_dev(v_new))
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.step_attention(layer, ctx, to_dev(q), o)
        torch.cuda.synchronize()
        k_all, v_all = hist[layer][0].copy(), hist[layer][1].copy()
        k_all[ctx], v_all[ctx] = k_new[0], v_new[0]
        ke, ve = encode_np(k_all, vf.KvDtype.F8), encode_np(v_all, vf.KvDtype.F8)
        # the appended FP8 bytes are bit-exact
        from gpu_util import read_device
        off = cache.pos_offset_bytes(layer, ctx)
        assert (read_device(cache.k_ptr + off, hkv * d) == ke[ctx]).all()
        assert (read_device(cache.v_ptr + off, hkv * d) == ve[ctx]).all()
        ref = oracle.attn_decode_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), oracle.F8, heads, hkv, d,
                                     ctx + 1, fwd.attn_scale)
        err = np.abs(to_np(o) - ref).max()
        assert err < 5e-3 and err < TIGHT * 40, err


@pytest.mark.parametrize("dtype,heads,hkv,d,ctx,window", [
    (vf.KvDtype.F8, 32, 8, 128, 8192, 0),       # configuration 2 geometry: the worker writes the row itself
    (vf.KvDtype.F8, 32, 8, 128, 1000, 300),     # new position in a ragged last tile, sliding window
    (vf.KvDtype.F16, 16, 8, 256, 777, 0),       # 2-byte cache, head_dim 256
    (vf.KvDtype.F16, 8, 8, 64, 64, 0),          # the new row opens a tile of its own
    (vf.KvDtype.F8, 24, 2, 128, 500, 0),        # GQA group of 12: two head slices, separate append launch
    (vf.KvDtype.F32, 8, 2, 128, 300, 0),        # 4-byte cache: separate append launch
    (vf.KvDtype.F16, 8, 1, 256, 16000, 0),      # one KV head: 250 tiles, merged by four wavefronts per 64 outputs
    (vf.KvDtype.F8, 16, 2, 512, 9000, 0),       # Gemma-4 full-attention geometry: 2 KV heads, 128 tiles
    # FP8 rows of head_dim 64 are half a 128-byte line: two workgroups (neighbouring KV heads) store into and read from the
    # same line of the new row
    (vf.KvDtype.F8, 16, 8, 64, 1000, 0),
    (vf.KvDtype.F8, 16, 8, 64, 8192, 0),        # interleaved walk: the owner of the new row is not the last workgroup
    (vf.KvDtype.F8, 16, 8, 64, 5000, 700),      # the same under a sliding window
    # the appending wavefront in the worker with full runs where the cases above take half runs (two to four full runs per stream)
    (vf.KvDtype.F16, 32, 8, 128, 8192, 0),
    (vf.KvDtype.F8, 16, 8, 64, 16384, 0),
    # head widths served by the next wider worker with its tail masked off: the row is written with its real stride
    (vf.KvDtype.F8, 32, 32, 96, 3000, 0),
    (vf.KvDtype.F16, 8, 4, 192, 2000, 500),
    (vf.KvDtype.F16, 32, 32, 80, 100, 0),       # one tile: the worker also writes the output
    # FP8 heads of 64 elements taken in pairs (8 KV heads: at least 16 384 visible rows): the pair's workgroup writes both heads' slices
    (vf.KvDtype.F8, 32, 8, 64, 33000, 0),
    (vf.KvDtype.F8, 24, 8, 64, 40000, 20000),
    (vf.KvDtype.F8, 32, 8, 64, 20000, 3000),    # a window shorter than that: separate heads
])
def test_kv_write_attention_in_one_call_matches_the_two_calls(dtype, heads, hkv, d, ctx, window):
    # step_kv_write + step_attention (executor/attention.rs:546-625) through the single entry point: cache bytes and
    # output must equal what the two separate calls produce, bit for bit, and match the oracle
    from gpu_util import read_device
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    esz = dtype.element_size()
    r = rng(77 + ctx)
    k_new, v_new, q = fill(r, (1, hkv * d)), fill(r, (1, hkv * d)), fp16_normal(r, (heads, d))
    kv_start = max(0, ctx + 1 - window) if window else 0
    outs, rows = [], []
    for fused in (False, True):
        cache, hist = _cache_with_history(dtype, 1, hkv, d, ctx + 1, fill, 70 + ctx)
        fwd = vf.Forward(cache, heads)
        o = torch.full((heads, d), float("nan"), device=DEV)
        print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} ctx={ctx} window={window} fused={fused}", flush=True)
        if fused:
            fwd.step_kv_write_attention(0, ctx, to_dev(q), to_dev(k_new), to_dev(v_new), o, kv_start=kv_start)
        else:
            fwd.step_kv_write(0, ctx, to_dev(k_new), to_dev(v_new))
            fwd.run_scalar_attn(0, ctx, to_dev(q), o, kv_start=kv_start)
        torch.cuda.synchronize()
        off = cache.pos_offset_bytes(0, ctx)
        rows.append((read_device(cache.k_ptr + off, hkv * d * esz).copy(), read_device(cache.v_ptr + off, hkv * d * esz).copy()))
        outs.append(to_np(o).copy())
        cache.destroy()
    assert (rows[0][0] == rows[1][0]).all() and (rows[0][1] == rows[1][1]).all()
    assert np.array_equal(outs[0], outs[1])
    k_all, v_all = hist[0][0].copy(), hist[0][1].copy()
    k_all[ctx], v_all[ctx] = k_new[0], v_new[0]
    ke, ve = encode_np(k_all, dtype), encode_np(v_all, dtype)
    assert (rows[1][0].view(ke.dtype) == ke[ctx].reshape(-1)).all()
    ref = oracle.attn_decode_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), int(dtype), heads, hkv, d, ctx + 1,
                                 1.0 / np.sqrt(d), kv_start=kv_start)
    assert np.abs(outs[1] - ref).max() < TOL[dtype]


@pytest.mark.parametrize("dtype,heads,hkv,d,seq", [(vf.KvDtype.F8, 32, 8, 128, 200), (vf.KvDtype.F8, 16, 2, 256, 256),
                                                  (vf.KvDtype.F16, 12, 4, 64, 129), (vf.KvDtype.F8, 40, 2, 128, 255)])
def test_spans_of_one_tile_skip_the_merge_launch(dtype, heads, hkv, d, seq):
    # up to 256 visible keys the convenience path uses one tile per KV head and the worker writes the output itself
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    cache, hist = _cache_with_history(dtype, 1, hkv, d, seq, fill, 90 + seq)
    fwd = vf.Forward(cache, heads)
    q = fp16_normal(rng(91), (heads, d))
    o = torch.full((heads, d), float("nan"), device=DEV)
    print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} seq={seq}", flush=True)
    fwd.run_scalar_attn(0, seq - 1, to_dev(q), o)
    torch.cuda.synchronize()
    ke, ve = (encode_np(x, dtype).reshape(seq, hkv, d) for x in hist[0])
    ref = oracle.attn_decode_ref(q, ke, ve, int(dtype), heads, hkv, d, seq, 1.0 / np.sqrt(d))
    assert np.abs(to_np(o) - ref).max() < TOL[dtype]


def test_config4_hd256_sliding_window_softcap_f16():
    # benchmark configuration 4 geometry: 16/8/256, F16 KV, window 4096 at context 16384, soft-cap 50;
    # layer 0 sliding, layer 1 global
    heads, hkv, d, ctx, window, cap = 16, 8, 256, 16384, 4096, 50.0
    cache, hist = _cache_with_history(vf.KvDtype.F16, 2, hkv, d, ctx, fp16_normal, 31)
    fwd = vf.Forward(cache, heads)
    q = fp16_normal(rng(32), (heads, d))
    scale = float(1.0 / np.sqrt(d))
    for layer, win in ((0, window), (1, 0)):
        kv_start = oracle.kv_start_decode(ctx - 1, win) if win else 0
        assert kv_start == (12288 if win else 0)
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.run_scalar_attn(layer, ctx - 1, to_dev(q), o, kv_start=kv_start, scale=scale, softcap=cap)
        torch.cuda.synchronize()
        ke, ve = encode_np(hist[layer][0], vf.KvDtype.F16), encode_np(hist[layer][1], vf.KvDtype.F16)
        ref = oracle.attn_decode_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), oracle.F16, heads, hkv, d,
                                     ctx, scale, kv_start=kv_start, softcap=cap)
        err = np.abs(to_np(o) - ref).max()
        assert err < 2e-3 and err < TIGHT, (layer, err)


def test_heterogeneous_cache_and_kv_share():
    # per-layer head_dim / kv heads (kv_cache.rs:256-283) and reading another layer's slab
    # (gemma4_kv_read_layer, gemma4.rs:27-49)
    hd, kvh, heads, seq = [256, 512, 256], [4, 2, 4], 8, 300
    cache, hist = _cache_with_history(vf.KvDtype.F8, 3, 999, 512, seq, fp16_normal, 41, hd=hd, kvh=kvh)
    fwd = vf.Forward(cache, heads)
    r = rng(42)
    for layer, kv_layer in ((0, 0), (1, 1), (2, 0)):
        d, g = hd[layer], kvh[layer]
        q = fp16_normal(r, (heads, d))
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.run_scalar_attn(layer, seq - 1, to_dev(q), o, kv_layer=kv_layer, scale=1.0 / np.sqrt(d))
        torch.cuda.synchronize()
        ke, ve = (encode_np(x, vf.KvDtype.F8).reshape(seq, g, d) for x in hist[kv_layer])
        ref = oracle.attn_decode_ref(q, ke, ve, oracle.F8, heads, g, d, seq, 1.0 / np.sqrt(d))
        assert np.abs(to_np(o) - ref).max() < TIGHT


def test_long_context_128k_fp8_and_window_edges():
    # four times the benchmark's context in one layer (128 MiB slabs), plus windows that start on, just before and
    # just after a run boundary and a window of a single key
    heads, hkv, d, ctx = 32, 8, 128, 131072
    cache, hist = _cache_with_history(vf.KvDtype.F8, 1, hkv, d, ctx, fp16_normal, 61)
    fwd = vf.Forward(cache, heads)
    q = fp16_normal(rng(62), (heads, d))
    ke, ve = (encode_np(x, vf.KvDtype.F8).reshape(ctx, hkv, d) for x in hist[0])
    scale = float(1.0 / np.sqrt(d))
    for pos, kv_start in ((ctx - 1, 0), (ctx - 1, ctx - 4096), (100000, 99999 - 4097), (70001, 70001 - 31), (5000, 5000)):
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.run_scalar_attn(0, pos, to_dev(q), o, kv_start=kv_start)
        torch.cuda.synchronize()
        ref = oracle.attn_decode_ref(q, ke, ve, oracle.F8, heads, hkv, d, pos + 1, scale, kv_start=kv_start)
        err = np.abs(to_np(o) - ref).max()
        assert err < TOL[vf.KvDtype.F8] and err < TIGHT, (pos, kv_start, err)
    cache.destroy()


def test_short_context_goes_through_the_same_path():
    # seq <= 64: the reference uses its single-workgroup shader (runs.rs:776-821); same attention
    heads, hkv, d = 32, 8, 128
    cache, hist = _cache_with_history(vf.KvDtype.F16, 1, hkv, d, 64, fp16_normal, 51)
    fwd = vf.Forward(cache, heads)
    q = fp16_normal(rng(52), (heads, d))
    ke, ve = (encode_np(x, vf.KvDtype.F16).reshape(64, hkv, d) for x in hist[0])
    for pos in (0, 1, 17, 63):   # one tile: the worker writes the normalised output itself, no merge launch
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.run_scalar_attn(0, pos, to_dev(q), o)
        torch.cuda.synchronize()
        ref = oracle.attn_decode_ref(q, ke, ve, oracle.F16, heads, hkv, d, pos + 1, fwd.attn_scale)
        assert np.abs(to_np(o) - ref).max() < TIGHT
    with pytest.raises(vf.VfkvError):
        fwd.run_scalar_attn(0, 64, to_dev(q), torch.empty((heads, d), device=DEV))      # beyond max_seq
    with pytest.raises(vf.VfkvError):
        fwd.run_scalar_attn(0, 10, to_dev(q), torch.empty((heads, d), device=DEV), kv_start=11)


@pytest.mark.parametrize("dtype,heads,hkv,d,ctx", [(vf.KvDtype.F8, 32, 8, 128, 4097), (vf.KvDtype.F16, 16, 8, 256, 1500)])
def test_caller_owned_buffers_give_the_same_output_at_any_relative_alignment(dtype, heads, hkv, d, ctx):
    # KvCache over buffers the caller allocated (kv_cache.rs:224-339 with the host's own allocator): equal alignment of K
    # and V modulo 512 bytes only costs speed (vfkv_cache_kv_alignment_note says so), the bytes and the output of decode
    # and prefill attention are the same as with V offset by 256 bytes
    from gpu_util import read_device
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    es = dtype.element_size()
    nbytes = ctx * hkv * d * es
    r = rng(404)
    k, v = fill(r, (ctx, hkv * d)), fill(r, (ctx, hkv * d))
    q, qb = fp16_normal(r, (heads, d)), fp16_normal(r, (16, heads, d))
    outs = []
    for skew in (0, 256, 128):
        kbuf = torch.zeros(nbytes + 512, dtype=torch.uint8, device=DEV)
        vbuf = torch.zeros(nbytes + 1024, dtype=torch.uint8, device=DEV)
        kp = (kbuf.data_ptr() + 511) // 512 * 512
        vp = (vbuf.data_ptr() + 511) // 512 * 512 + skew
        cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, ctx, dtype=dtype), k_buffer=kp, v_buffer=vp)
        note = vf._ffi.lib().vfkv_cache_kv_alignment_note(cache.handle)
        assert (b"256 bytes" in note) == (skew == 0)
        fwd = vf.Forward(cache, heads)
        fwd.b_step_kv_write(0, 0, ctx, to_dev(k), to_dev(v))
        o = torch.full((heads, d), float("nan"), device=DEV)
        fwd.run_scalar_attn(0, ctx - 1, to_dev(q), o)
        ob = torch.full((16, heads, d), float("nan"), device=DEV)
        fwd.b_step_attention(0, ctx - 16, 16, to_dev(qb), ob)
        torch.cuda.synchronize()
        outs.append((to_np(o).copy(), to_np(ob).copy(), read_device(vp, nbytes).copy()))
        cache.destroy()
    for o, ob, vbytes in outs[1:]:
        assert np.array_equal(o, outs[0][0]) and np.array_equal(ob, outs[0][1]) and np.array_equal(vbytes, outs[0][2])
    ke, ve = encode_np(k, dtype).reshape(-1, hkv, d), encode_np(v, dtype).reshape(-1, hkv, d)
    ref = oracle.attn_decode_ref(q, ke, ve, int(dtype), heads, hkv, d, ctx, 1.0 / np.sqrt(d))
    assert np.abs(outs[0][0] - ref).max() < TOL[dtype]


def test_shapes_on_the_generic_fallback_leave_a_note():
    # head_dim 72 has no tiled kernel (80 runs on the worker for 128 with its tail masked off): the result is still right,
    # and vfkv_last_note says that the call was a slow one; a shape on the tiled kernels clears it
    L = vf._ffi.lib()
    r = rng(80)
    valu = os.environ.get("VFKV_DECODE_WORKER", "")[:1] == "v"     # (that switch keeps the padded widths off the matrix-core worker)
    for d, slow in ((72, True), (80, valu), (128, False)):
        heads, hkv, seq = 8, 2, 300
        q = fp16_normal(r, (heads, d))
        k, v = encode_np(fp16_normal(r, (seq, hkv, d)), vf.KvDtype.F16), encode_np(fp16_normal(r, (seq, hkv, d)), vf.KvDtype.F16)
        scale = float(1.0 / np.sqrt(d))
        o, *_ = gpu_split_reduce(q, k, v, vf.KvDtype.F16, heads, hkv, d, seq, scale, tile=64)
        ref = oracle.attn_decode_ref(q, k, v, int(vf.KvDtype.F16), heads, hkv, d, seq, scale)
        assert np.abs(o - ref).max() < TOL[vf.KvDtype.F16]
    # (gpu_split_reduce's last library call is the merge, which leaves the note of the split alone)
        note = L.vfkv_last_note()
        assert (b"generic fallback" in note) == slow, note
    assert L.vfkv_last_error() is not None
