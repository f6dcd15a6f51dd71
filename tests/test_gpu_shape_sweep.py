"""Seeded sweep over shapes no other test names: decode (split + merge, contiguous tiles and interleaved runs),
chunked prefill, and the cache-level calls (history, decode token appended and attended in one call, a prefill chunk behind
it) against the CPU oracle, over every head width the tiled kernels serve (and a few they do not), every cache type,
grouped and ungrouped heads, ragged lengths, windows and the soft-cap.

The cases are drawn from a fixed seed, so the sweep is the same on every run; each prints its shape before it runs."""
import numpy as np
import pytest

import oracle
import vulkanforge_amd as vf
from gpu_util import TIGHT, TOL, encode_np, fp16_normal, gpu_batch, gpu_split_reduce, outlier_normal, rng

pytestmark = pytest.mark.gpu

WIDTHS = (64, 80, 96, 112, 128, 160, 192, 224, 256, 512, 40, 72)
DTYPES = (vf.KvDtype.F8, vf.KvDtype.F16, vf.KvDtype.F32)


def _draw_common(r):
    d = int(r.choice(WIDTHS))
    dtype = DTYPES[int(r.integers(0, 3))]
    hkv = int(r.choice((1, 2, 3, 4, 8, 16)))
    g = int(r.choice((1, 1, 2, 3, 4, 5, 8, 12)))
    if d >= 256:                                   # keep the oracle's share of the run time small
        hkv, g = min(hkv, 4), min(g, 4)
    cap = float(r.choice((0.0, 0.0, 20.0, 50.0)))
    return d, dtype, hkv, g, cap


def _decode_cases(n, seed):
    r = rng(seed)
    out = []
    for _ in range(n):
        d, dtype, hkv, g, cap = _draw_common(r)
        seq = int(r.integers(1, 2600))
        tile = int(r.choice((16, 48, 64, 96, 128, 320, 512, 1024)))
        kv_start = int(r.integers(0, seq)) if r.random() < 0.4 else 0
        out.append((dtype, hkv * g, hkv, d, seq, tile, kv_start, cap))
    return out


def _prefill_cases(n, seed):
    r = rng(seed)
    out = []
    for _ in range(n):
        d, dtype, hkv, g, cap = _draw_common(r)
        m = int(r.integers(1, 100))
        q_start = int(r.integers(0, 900))
        # a window must leave the first query a visible key: kv_start <= q_start
        kv_start = int(r.integers(0, q_start + 1)) if r.random() < 0.4 else 0
        out.append((dtype, hkv * g, hkv, d, m, q_start, kv_start, cap))
    return out


def _kv(r, dtype, shape):
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    return encode_np(fill(r, shape), dtype), encode_np(fill(r, shape), dtype)


@pytest.mark.parametrize("dtype,heads,hkv,d,seq,tile,kv_start,cap", _decode_cases(160, 20261125))
def test_decode_sweep(dtype, heads, hkv, d, seq, tile, kv_start, cap):
    r = rng(hash((int(dtype), heads, hkv, d, seq, tile, kv_start)) % (1 << 31))
    q = r.standard_normal((heads, d)).astype(np.float32)           # general f32 queries
    k, v = _kv(r, dtype, (seq, hkv, d))
    scale = float(1.0 / np.sqrt(d))
    print(f"case decode dtype={dtype.label()} H={heads} Hkv={hkv} D={d} seq={seq} tile={tile} kv_start={kv_start} cap={cap}",
          flush=True)
    ref = oracle.attn_decode_ref(q, k, v, int(dtype), heads, hkv, d, seq, scale, kv_start=kv_start, softcap=cap)
    for interleaved in (False, True):
        o, so, sm, ss = gpu_split_reduce(q, k, v, dtype, heads, hkv, d, seq, scale, tile=tile, kv_start=kv_start,
                                         softcap=cap, interleaved=interleaved)
        assert np.isfinite(o).all() and np.isfinite(so).all() and np.isfinite(sm).all() and np.isfinite(ss).all()
        err = np.abs(o - ref).max()
        assert err < TOL[dtype], (interleaved, err)
        assert err < TIGHT * max(1.0, np.abs(ref).max()), (interleaved, err)


@pytest.mark.parametrize("dtype,heads,hkv,d,m,q_start,kv_start,cap", _prefill_cases(160, 20261126))
def test_prefill_sweep(dtype, heads, hkv, d, m, q_start, kv_start, cap):
    r = rng(hash((int(dtype), heads, hkv, d, m, q_start, kv_start)) % (1 << 31))
    n_kv = q_start + m
    q = r.standard_normal((m, heads, d)).astype(np.float32)        # general f32 queries
    k, v = _kv(r, dtype, (n_kv, hkv, d))
    scale = float(1.0 / np.sqrt(d))
    print(f"case prefill dtype={dtype.label()} H={heads} Hkv={hkv} D={d} m={m} q_start={q_start} kv_start={kv_start} cap={cap}",
          flush=True)
    o = gpu_batch(q, k, v, dtype, heads, hkv, d, m, q_start, n_kv, scale, kv_start=kv_start, softcap=cap)
    ref = oracle.attn_batch_ref(q, k, v, int(dtype), m, n_kv, heads, hkv, d, q_start, scale, kv_start=kv_start, softcap=cap)
    assert np.isfinite(o).all()
    err = np.abs(o - ref).max()
    assert err < TOL[dtype], err
    assert err < TIGHT * max(1.0, np.abs(ref).max()), err


def _cache_cases(n, seed):
    r = rng(seed)
    out = []
    for _ in range(n):
        d, dtype, hkv, g, cap = _draw_common(r)
        ctx = int(r.integers(1, 3000))                      # rows in the cache before the decode token
        window = int(r.integers(1, ctx + 1)) if r.random() < 0.3 else 0
        m = int(r.integers(1, 70))                          # rows of the prefill chunk that follows
        if window:
            window = max(window, m)                         # (a chunk longer than the window leaves its first query no key: rejected)
        out.append((dtype, hkv * g, hkv, d, ctx, window, m, cap))
    return out


@pytest.mark.parametrize("dtype,heads,hkv,d,ctx,window,m,cap", _cache_cases(120, 20261127))
def test_cache_level_sweep(dtype, heads, hkv, d, ctx, window, m, cap):
    """One layer of a KvCache: history written through the append call, then the decode token appended and attended in one
    call (workgroup count and run length are the library's own choice), then a chunk of m rows appended and attended as a
    prefill -- cache bytes of every appended row and both outputs against the oracle."""
    import torch
    from gpu_util import DEV, read_device, to_dev, to_np
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    r = rng(hash((int(dtype), heads, hkv, d, ctx, window, m)) % (1 << 31))
    n = ctx + 1 + m
    row = hkv * d
    k_all, v_all = fill(r, (n, row)), fill(r, (n, row))
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, n, dtype=dtype))
    cache.zero_fill()
    fwd = vf.Forward(cache, heads)
    print(f"case cache dtype={dtype.label()} H={heads} Hkv={hkv} D={d} ctx={ctx} window={window} m={m} cap={cap}", flush=True)
    fwd.b_step_kv_write(0, 0, ctx, to_dev(k_all[:ctx]), to_dev(v_all[:ctx]))
    # ---- decode token at position ctx ----
    q = r.standard_normal((heads, d)).astype(np.float32)
    kv_start = max(0, ctx + 1 - window) if window else 0
    o = torch.full((heads, d), float("nan"), device=DEV)
    fwd.step_kv_write_attention(0, ctx, to_dev(q), to_dev(k_all[ctx:ctx + 1]), to_dev(v_all[ctx:ctx + 1]), o,
                                kv_start=kv_start, softcap=cap)
    torch.cuda.synchronize()
    ke, ve = encode_np(k_all, dtype), encode_np(v_all, dtype)
    esz = dtype.element_size()
    off = cache.pos_offset_bytes(0, ctx)
    assert (read_device(cache.k_ptr + off, row * esz).view(ke.dtype) == ke[ctx]).all()
    assert (read_device(cache.v_ptr + off, row * esz).view(ve.dtype) == ve[ctx]).all()
    ref = oracle.attn_decode_ref(q, ke[:ctx + 1].reshape(-1, hkv, d), ve[:ctx + 1].reshape(-1, hkv, d), int(dtype), heads, hkv,
                                 d, ctx + 1, fwd.attn_scale, kv_start=kv_start, softcap=cap)
    err = np.abs(to_np(o) - ref).max()
    assert err < TOL[dtype] and err < TIGHT * max(1.0, np.abs(ref).max()), err
    # ---- a chunk of m rows behind it ----
    base = ctx + 1
    fwd.b_step_kv_write(0, base, m, to_dev(k_all[base:]), to_dev(v_all[base:]))
    qb = r.standard_normal((m, heads, d)).astype(np.float32)
    ob = torch.full((m, heads, d), float("nan"), device=DEV)
    fwd.b_step_attention(0, base, m, to_dev(qb), ob, kv_start_window=window, softcap=cap)
    torch.cuda.synchronize()
    assert (read_device(cache.k_ptr + cache.pos_offset_bytes(0, base), m * row * esz).view(ke.dtype) == ke[base:].reshape(-1)).all()
    refb = oracle.attn_batch_ref(qb, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), int(dtype), m, n, heads, hkv, d, base,
                                 fwd.attn_scale, kv_start=oracle.kv_start_batch(base, m, window), softcap=cap)
    errb = np.abs(to_np(ob) - refb).max()
    assert errb < TOL[dtype] and errb < TIGHT * max(1.0, np.abs(refb).max()), errb
    cache.destroy()
