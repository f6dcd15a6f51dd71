"""GPU parity of vfkv_k_rope_kv_write (K RMS-norm * weight + RoPE + append of K and V in one launch) against the
oracle, through the C ABI.

Bars.  V bytes: bit-exact.  K with an F32 cache (and `k_out`): |gpu - oracle| <= max|k| * (5e-6 + pos * 2^-21) --
the only slack is one ulp of the f32 angle theta <= pos * 2^-23 between two powf implementations, the same slack
the reference grants its own GPU (tests/correctness.rs:799-815: 1e-5 / 1e-4 / 5e-4 at positions 0 / 100 / 4096
for |x| <= 3.5).  K with an F16 / FP8 cache: the stored code must lie between the codes of (oracle - tol) and
(oracle + tol), i.e. be a correct rounding of a value inside that band."""
import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from vulkanforge_amd import _ffi
from gpu_util import DEV, fp16_normal, read_device, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def k_tolerance(k_ref, pos):
    return np.abs(k_ref).max() * (5e-6 + np.asarray(pos, np.float64) * 2.0 ** -21)


def run_case(dtype, hkv, d, n_tok, pos0, rotary, mode, norm, use_pos_array, use_ff, freq_base=10000.0, k_out=True,
             seed=0, max_seq=None):
    r = rng(seed + d + n_tok + pos0)
    max_seq = max_seq or pos0 + n_tok + 3
    cache = vf.KvCache(vf.KvCacheConfig(2, hkv, d, max_seq, dtype=dtype))
    cache.zero_fill()
    fwd = vf.Forward(cache, hkv)
    k = (r.standard_normal((n_tok, hkv, d)) * 1.5).astype(np.float32)
    v = fp16_normal(r, (n_tok, hkv, d))
    w = (1 + 0.2 * r.standard_normal(d)).astype(np.float32) if norm else None
    ff = (1 + 2 * r.random(rotary // 2)).astype(np.float32) if use_ff else None
    if use_pos_array:
        positions = (pos0 + np.arange(n_tok) * 3 + (np.arange(n_tok) % 2) * 11).astype(np.int32)   # not pos0 + t on purpose
    else:
        positions = (pos0 + np.arange(n_tok)).astype(np.int32)
    ts = float(oracle.rope_theta_scale(freq_base, rotary)) if rotary else 1.0
    kd, vd = to_dev(k), to_dev(v)
    kout = torch.full_like(kd, float("nan")) if k_out else None
    layer = 1
    fwd.step_k_rope_kv_write(layer, pos0, n_tok, kd, vd, rotary, ts, k_norm_weight=to_dev(w) if norm else None,
                             positions=to_dev(positions) if use_pos_array else None,
                             freq_factors=to_dev(ff) if use_ff else None, rope_mode=mode, eps=1e-6, k_out=kout)
    torch.cuda.synchronize()
    k_ref = oracle.rms_norm_rope(k, positions, d, rotary, ts, mode=mode, weight=w, ff=ff, eps=1e-6)
    tol = k_tolerance(k_ref, positions)[:, None, None]
    es = dtype.element_size()
    off = cache.pos_offset_bytes(layer, pos0)
    nbytes = n_tok * hkv * d * es
    k_bytes = read_device(cache.k_ptr + off, nbytes)
    v_bytes = read_device(cache.v_ptr + off, nbytes)
    # ---- V: what vfkv_kv_write stores, bit for bit
    v_exp = np.zeros(nbytes, np.uint8)
    if dtype == vf.KvDtype.F8:
        oracle.kv_store_fp8(v.reshape(-1), v_exp, v.size, 0)
    elif dtype == vf.KvDtype.F16:
        oracle.kv_copy_fp16(v.reshape(-1), v_exp, v.size, 0)
    else:
        v_exp = v.reshape(-1).view(np.uint8)
    assert (v_bytes == v_exp).all()
    # ---- K
    if k_out:
        ko = to_np(kout)
        assert np.isfinite(ko).all()
        assert (np.abs(ko - k_ref) <= tol).all(), float(np.abs(ko - k_ref).max())
    if dtype == vf.KvDtype.F32:
        got = k_bytes.view(np.float32).reshape(k_ref.shape)
        assert (np.abs(got - k_ref) <= tol).all()
        if k_out:
            assert (got == ko).all()
    else:
        if dtype == vf.KvDtype.F8:
            dec = lambda b: oracle.e4m3_to_f32(b)                                           # noqa: E731
            enc = lambda x: oracle.f32_to_e4m3(x)                                           # noqa: E731
            got = dec(k_bytes).reshape(k_ref.shape)
        else:
            dec = lambda b: oracle.f16_bits_to_f32(b)                                       # noqa: E731
            enc = lambda x: oracle.f32_to_f16_bits(x)                                       # noqa: E731
            got = dec(k_bytes.view(np.uint16)).reshape(k_ref.shape)
        lo = dec(enc((k_ref - tol).astype(np.float32).reshape(-1))).reshape(k_ref.shape)
        hi = dec(enc((k_ref + tol).astype(np.float32).reshape(-1))).reshape(k_ref.shape)
        assert ((got >= lo) & (got <= hi)).all()
        if k_out:                                   # the cache holds the conversion of exactly what k_out holds
            assert (k_bytes.view(np.uint8 if dtype == vf.KvDtype.F8 else np.uint16) == enc(ko.reshape(-1))).all()
    # rows outside [pos0, pos0 + n_tok) and the other layer stay zero
    assert not read_device(cache.k_ptr, cache.pos_offset_bytes(layer, pos0)).any()
    tail = cache.pos_offset_bytes(layer, pos0 + n_tok)
    assert not read_device(cache.k_ptr + tail, cache.bytes_per_buffer() - tail).any()
    cache.destroy()
    return k_ref


CASES = [
    # dtype, hkv, d, n_tok, pos0, rotary, mode, norm, pos_array, ff
    (vf.KvDtype.F8, 8, 128, 1, 8192, 128, _ffi.ROPE_NEOX, True, False, False),     # decode step, Qwen3-style K-norm
    (vf.KvDtype.F8, 8, 128, 1, 100, 128, _ffi.ROPE_NEOX, False, False, False),     # plain KRope
    (vf.KvDtype.F8, 8, 128, 512, 4096, 128, _ffi.ROPE_NEOX, True, False, False),   # prefill chunk
    (vf.KvDtype.F16, 8, 256, 33, 1000, 256, _ffi.ROPE_NEOX, True, True, False),
    (vf.KvDtype.F16, 2, 128, 7, 0, 64, _ffi.ROPE_NEOX, True, False, True),         # partial rotary, frequency factors
    (vf.KvDtype.F32, 4, 128, 9, 50, 128, _ffi.ROPE_NORM, False, True, False),
    (vf.KvDtype.F32, 4, 64, 9, 4000, 64, _ffi.ROPE_NORM, True, False, True),
    (vf.KvDtype.F32, 1, 512, 3, 10, 128, _ffi.ROPE_NEOX, True, False, False),
    (vf.KvDtype.F8, 3, 96, 5, 77, 32, _ffi.ROPE_NORM, True, True, False),
    (vf.KvDtype.F8, 8, 128, 4, 32000, 128, _ffi.ROPE_NEOX, True, False, False),    # long context
]


@pytest.mark.parametrize("dtype,hkv,d,n_tok,pos0,rotary,mode,norm,pos_array,ff", CASES)
def test_k_rope_kv_write_matches_oracle(dtype, hkv, d, n_tok, pos0, rotary, mode, norm, pos_array, ff):
    print(f"case dtype={dtype.label()} hkv={hkv} D={d} tokens={n_tok} pos0={pos0} rotary={rotary} mode={mode} norm={norm} "
          f"pos_array={pos_array} ff={ff}", flush=True)
    run_case(dtype, hkv, d, n_tok, pos0, rotary, mode, norm, pos_array, ff)
    run_case(dtype, hkv, d, n_tok, pos0, rotary, mode, norm, pos_array, ff, k_out=False, seed=1)


@pytest.mark.parametrize("pos,threshold", ((0, 1e-5), (100, 1e-4), (4096, 5e-4)))
def test_reference_rope_neox_fixture(pos, threshold):
    # tests/correctness.rs:799-884: one head of 128, ramp input, NEOX, freq_base 1e6, the reference's thresholds
    x = (np.float32(0.1) + np.float32(3.4) * np.arange(128, dtype=np.float32) / np.float32(127)).astype(np.float32)
    half = 64
    ts = np.float32(1.0) / np.float32(1e6) ** np.float32(2.0 / 128)
    cpu = np.zeros(128, np.float32)
    for i in range(half):
        freq = np.float32(1.0)
        for _ in range(i):
            freq = np.float32(freq * ts)
        theta = np.float32(pos) * freq
        c, s = np.cos(theta, dtype=np.float32), np.sin(theta, dtype=np.float32)
        cpu[i] = x[i] * c - x[i + half] * s
        cpu[i + half] = x[i] * s + x[i + half] * c
    cache = vf.KvCache(vf.KvCacheConfig(1, 1, 128, pos + 1, dtype=vf.KvDtype.F32))
    fwd = vf.Forward(cache, 1)
    kd = to_dev(x.reshape(1, 1, 128))
    out = torch.empty_like(kd)
    fwd.step_k_rope_kv_write(0, pos, 1, kd, kd, 128, float(ts), k_out=out)
    torch.cuda.synchronize()
    got = to_np(out).reshape(-1)
    assert np.abs(got - cpu).max() < threshold
    row = read_device(cache.k_ptr + cache.pos_offset_bytes(0, pos), 512).view(np.float32)
    assert (row == got).all()
    if pos == 0:
        assert (got == x).all()
    cache.destroy()


def test_position_zero_is_the_plain_append_and_in_place_output():
    # rotation by 0 is exact, so without a norm the K bytes are what vfkv_kv_write stores; k_out may alias k_src
    r = rng(9)
    hkv, d = 8, 128
    k = fp16_normal(r, (1, hkv, d))
    v = fp16_normal(r, (1, hkv, d))
    for dtype in (vf.KvDtype.F8, vf.KvDtype.F16):
        a = vf.KvCache(vf.KvCacheConfig(1, hkv, d, 4, dtype=dtype))
        b = vf.KvCache(vf.KvCacheConfig(1, hkv, d, 4, dtype=dtype))
        a.zero_fill(); b.zero_fill()
        kd, vd = to_dev(k), to_dev(v)
        vf.Forward(a, hkv).step_k_rope_kv_write(0, 0, 1, kd, vd, d, 0.9, k_out=kd)
        vf.Forward(b, hkv).step_kv_write(0, 0, to_dev(k), vd)
        torch.cuda.synchronize()
        n = a.bytes_per_buffer()
        assert (read_device(a.k_ptr, n) == read_device(b.k_ptr, n)).all()
        assert (read_device(a.v_ptr, n) == read_device(b.v_ptr, n)).all()
        assert (to_np(kd) == k).all()
        a.destroy(); b.destroy()


def test_rotated_keys_feed_decode_attention():
    # the fused append followed by decode attention == oracle attention over oracle-rotated keys
    r = rng(21)
    h, hkv, d, seq = 32, 8, 128, 300
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, seq, dtype=vf.KvDtype.F16))
    fwd = vf.Forward(cache, h)
    k = fp16_normal(r, (seq, hkv, d))
    v = fp16_normal(r, (seq, hkv, d))
    q = fp16_normal(r, (h, d))
    w = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    ts = float(oracle.rope_theta_scale(10000.0, d))
    fwd.step_k_rope_kv_write(0, 0, seq, to_dev(k), to_dev(v), d, ts, k_norm_weight=to_dev(w))
    o = torch.empty((h, d), device=DEV)
    fwd.run_scalar_attn(0, seq - 1, to_dev(q), o)
    torch.cuda.synchronize()
    k_rot = oracle.rms_norm_rope(k, np.arange(seq, dtype=np.int32), d, d, ts, weight=w)
    k16 = oracle.f32_to_f16_bits(k_rot.reshape(-1)).reshape(seq, hkv, d)
    v16 = oracle.f32_to_f16_bits(v.reshape(-1)).reshape(seq, hkv, d)
    ref = oracle.attn_decode_ref(q, k16, v16, oracle.F16, h, hkv, d, seq, float(1 / np.sqrt(d)))
    assert np.abs(to_np(o) - ref).max() < 2e-3
    cache.destroy()


@pytest.mark.parametrize("heads,d,m,rotary,mode,norm,in_place", (
    (32, 128, 1, 128, _ffi.ROPE_NEOX, True, True),        # decode step_q_norm_rope
    (32, 128, 512, 128, _ffi.ROPE_NEOX, True, False),     # prefill chunk
    (16, 256, 7, 64, _ffi.ROPE_NEOX, False, True),        # plain RoPE, partial rotary (run_rope_neox_with_pos_offset)
    (5, 96, 9, 96, _ffi.ROPE_NORM, True, False),
))
def test_rms_norm_mul_rope_matches_oracle(heads, d, m, rotary, mode, norm, in_place):
    # the Q side of the fusion: forward/runs.rs:2492-2600 and :647-720
    r = rng(heads * 1000 + d + m)
    x = (r.standard_normal((m, heads, d)) * 1.5).astype(np.float32)
    w = (1 + 0.2 * r.standard_normal(d)).astype(np.float32) if norm else None
    pos = (4000 + np.arange(m) * 2).astype(np.int32)
    ts = float(oracle.rope_theta_scale(1e6, rotary))
    xd = to_dev(x)
    out = xd if in_place else torch.full_like(xd, float("nan"))
    vf.Forward.run_rms_norm_mul_rope(xd, to_dev(w) if norm else None, out, d, rotary, ts, heads, m, eps=1e-6,
                                     positions=to_dev(pos), rope_mode=mode)
    torch.cuda.synchronize()
    ref = oracle.rms_norm_rope(x, pos, d, rotary, ts, mode=mode, weight=w, eps=1e-6)
    got = to_np(out)
    assert (np.abs(got - ref) <= k_tolerance(ref, pos)[:, None, None]).all(), float(np.abs(got - ref).max())
    # implicit positions pos0 + t
    out2 = torch.empty_like(out)
    vf.Forward.run_rms_norm_mul_rope(to_dev(x), to_dev(w) if norm else None, out2, d, rotary, ts, heads, m, eps=1e-6,
                                     pos0=77, rope_mode=mode)
    torch.cuda.synchronize()
    ref2 = oracle.rms_norm_rope(x, (77 + np.arange(m)).astype(np.int32), d, rotary, ts, mode=mode, weight=w, eps=1e-6)
    assert (np.abs(to_np(out2) - ref2) <= k_tolerance(ref2, 77 + np.arange(m))[:, None, None]).all()


@pytest.mark.parametrize("dtype,h,hkv,d,m,pos0", ((vf.KvDtype.F8, 32, 8, 128, 1, 8192), (vf.KvDtype.F16, 16, 8, 256, 40, 100),
                                                  (vf.KvDtype.F8, 6, 3, 64, 9, 0)))
def test_qk_rope_kv_write_is_the_two_calls_in_one(dtype, h, hkv, d, m, pos0):
    # Q rows ride in the same launch: bit-identical to vfkv_rms_norm_mul_rope + vfkv_k_rope_kv_write
    r = rng(h * 31 + d + m)
    q = (r.standard_normal((m, h, d)) * 1.2).astype(np.float32)
    k = (r.standard_normal((m, hkv, d)) * 1.2).astype(np.float32)
    v = fp16_normal(r, (m, hkv, d))
    wq = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    wk = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    ts = float(oracle.rope_theta_scale(1e6, d))
    a = vf.KvCache(vf.KvCacheConfig(1, hkv, d, pos0 + m, dtype=dtype))
    b = vf.KvCache(vf.KvCacheConfig(1, hkv, d, pos0 + m, dtype=dtype))
    a.zero_fill(); b.zero_fill()
    qa, qb = to_dev(q), to_dev(q)
    ka = torch.empty((m, hkv, d), device=DEV)
    kb = torch.empty((m, hkv, d), device=DEV)
    vf.Forward(a, h).step_qk_rope_kv_write(0, pos0, m, qa, to_dev(k), to_dev(v), d, ts, q_norm_weight=to_dev(wq),
                                           k_norm_weight=to_dev(wk), k_out=ka)
    fb = vf.Forward(b, h)
    fb.run_rms_norm_mul_rope(qb, to_dev(wq), qb, d, d, ts, h, m, pos0=pos0)
    fb.step_k_rope_kv_write(0, pos0, m, to_dev(k), to_dev(v), d, ts, k_norm_weight=to_dev(wk), k_out=kb)
    torch.cuda.synchronize()
    n = a.bytes_per_buffer()
    assert (read_device(a.k_ptr, n) == read_device(b.k_ptr, n)).all()
    assert (read_device(a.v_ptr, n) == read_device(b.v_ptr, n)).all()
    assert (to_np(qa) == to_np(qb)).all() and (to_np(ka) == to_np(kb)).all()
    pos = (pos0 + np.arange(m)).astype(np.int32)
    q_ref = oracle.rms_norm_rope(q, pos, d, d, ts, weight=wq, eps=1e-6)
    assert (np.abs(to_np(qa) - q_ref) <= k_tolerance(q_ref, pos)[:, None, None]).all()
    a.destroy(); b.destroy()


FOLD_CASES = [
    # dtype, heads, hkv, d, ctx, rotary, mode, norm, ff, window, cap
    (vf.KvDtype.F8, 32, 8, 128, 8193, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),     # the decode step of a Qwen3-style layer
    (vf.KvDtype.F8, 32, 8, 128, 4097, 128, _ffi.ROPE_NORM, False, False, 0, 0.0),    # plain QRope / KRope, adjacent pairs
    (vf.KvDtype.F8, 32, 8, 128, 3000, 64, _ffi.ROPE_NEOX, True, True, 1000, 0.0),    # partial rotary, frequency factors, window
    (vf.KvDtype.F16, 16, 8, 256, 5000, 256, _ffi.ROPE_NEOX, True, False, 0, 30.0),   # head_dim 256, soft-cap
    (vf.KvDtype.F16, 16, 4, 64, 2500, 64, _ffi.ROPE_NORM, True, False, 0, 0.0),      # head_dim 64 (runs of 64 rows)
    (vf.KvDtype.F8, 8, 8, 64, 1300, 32, _ffi.ROPE_NEOX, False, False, 0, 0.0),       # FP8 rows of 64 bytes: two KV heads share a line
    (vf.KvDtype.F8, 32, 8, 128, 200, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),      # one workgroup per KV head writes the output itself
    (vf.KvDtype.F8, 32, 8, 128, 8209, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),     # 17 rows in the last run: a unit of its own
    (vf.KvDtype.F8, 96, 8, 128, 2049, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),     # 12 heads per KV head: two head slices
    (vf.KvDtype.F8, 4, 1, 512, 700, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),       # head_dim 512: the separate RoPE launch
    (vf.KvDtype.F32, 8, 2, 128, 600, 128, _ffi.ROPE_NEOX, True, False, 0, 0.0),      # F32 cache: the separate RoPE launch
    (vf.KvDtype.F8, 64, 32, 64, 5000, 64, _ffi.ROPE_NEOX, True, False, 0, 0.0),      # FP8 heads of 64, 32 KV heads, 5 000 rows: folded, separate heads
    (vf.KvDtype.F8, 64, 32, 64, 12500, 64, _ffi.ROPE_NEOX, True, False, 0, 0.0),     # 12 500 rows: the separate RoPE launch in front of paired KV heads
    (vf.KvDtype.F16, 32, 32, 96, 1500, 96, _ffi.ROPE_NEOX, False, False, 0, 0.0),    # head_dim 96 (padded worker): the separate RoPE launch
]


@pytest.mark.parametrize("dtype,heads,hkv,d,ctx,rotary,mode,norm,ff,window,cap", FOLD_CASES)
def test_qk_rope_kv_write_decode_attention_equals_the_separate_calls(dtype, heads, hkv, d, ctx, rotary, mode, norm, ff, window, cap):
    """vfkv_qk_rope_kv_write_decode_attention (norm + RoPE of the token inside the decode worker where it can) against
    vfkv_qk_rope_kv_write followed by vfkv_decode_attention: cache bytes, rotated queries and rotated K row bit-identical, the
    output within f32 rounding of the two-call output and within this path's tolerance of the oracle
    (vfo_rms_norm_rope -> cache encoding -> vfo_attn_decode_ref)."""
    from gpu_util import TOL, encode_np, outlier_normal
    r = rng(ctx * 3 + d)
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    k_hist, v_hist = fill(r, (ctx - 1, hkv * d)), fill(r, (ctx - 1, hkv * d))
    q = (r.standard_normal((heads, d)) * 1.2).astype(np.float32)
    k_new = (r.standard_normal((hkv, d)) * 1.5).astype(np.float32)
    v_new = fp16_normal(r, (hkv, d))
    qw = (1 + 0.2 * r.standard_normal(d)).astype(np.float32) if norm else None
    kw = (1 + 0.2 * r.standard_normal(d)).astype(np.float32) if norm else None
    ffv = (1 + 2 * r.random(rotary // 2)).astype(np.float32) if ff else None
    ts = float(oracle.rope_theta_scale(10000.0, rotary))
    pos = ctx - 1
    kv_start = max(0, pos + 1 - window) if window else 0
    scale = float(1.0 / np.sqrt(d))
    es = dtype.element_size()
    got = []
    for fused in (True, False):
        cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, ctx + 4, dtype=dtype))
        cache.zero_fill()
        fwd = vf.Forward(cache, heads)
        fwd.b_step_kv_write(0, 0, ctx - 1, to_dev(k_hist), to_dev(v_hist))
        qd, kd, vd = to_dev(q), to_dev(k_new), to_dev(v_new)
        q_out = torch.full((heads, d), float("nan"), device=DEV)
        k_out = torch.full((hkv, d), float("nan"), device=DEV)
        o = torch.full((heads, d), float("nan"), device=DEV)
        kwargs = dict(q_norm_weight=to_dev(qw) if norm else None, k_norm_weight=to_dev(kw) if norm else None,
                      freq_factors=to_dev(ffv) if ff else None, rope_mode=mode, eps=1e-6, k_out=k_out)
        print(f"case {dtype.label()} H={heads} Hkv={hkv} D={d} ctx={ctx} rotary={rotary} mode={mode} norm={norm} fused={fused}", flush=True)
        if fused:
            fwd.step_qk_rope_kv_write_attention(0, pos, qd, kd, vd, o, rotary, ts, q_out=q_out, kv_start=kv_start, scale=scale,
                                                softcap=cap, **kwargs)
        else:
            fwd.step_qk_rope_kv_write(0, pos, 1, qd, kd, vd, rotary, ts, q_out=q_out, **kwargs)
            fwd.run_scalar_attn(0, pos, q_out, o, kv_start=kv_start, scale=scale, softcap=cap)
        torch.cuda.synchronize()
        row = read_device(cache.k_ptr + cache.pos_offset_bytes(0, pos), hkv * d * es).copy()
        vrow = read_device(cache.v_ptr + cache.pos_offset_bytes(0, pos), hkv * d * es).copy()
        got.append((row, vrow, to_np(q_out).copy(), to_np(k_out).copy(), to_np(o).copy()))
        assert (to_np(qd) == q).all()                       # the caller's rows are left alone
        cache.destroy()
    (rk, rv, rq, rko, ro), (sk, sv, sq, sko, so_) = got
    assert (rk == sk).all() and (rv == sv).all()            # cache bytes
    assert (rq == sq).all() and (rko == sko).all()          # rotated queries and K row
    # (the two paths may run on different workers -- the fold stays with separate KV heads where the separate calls pair FP8
    # heads of 64 elements -- so their outputs agree to f32 rounding at the outputs' magnitude, not bit for bit)
    assert np.abs(ro - so_).max() < 2e-6 * max(1.0, float(np.abs(so_).max()))
    # against the oracle.  The rotation: within one ulp of the f32 angle of the oracle's (the slack the reference grants its own GPU
    # at tests/correctness.rs:799-815), the stored K code a correct rounding of a value inside that band
    q_ref = oracle.rms_norm_rope(q[None], np.array([pos], np.int32), d, rotary, ts, mode=mode, weight=qw, ff=ffv, eps=1e-6)[0]
    k_ref = oracle.rms_norm_rope(k_new[None], np.array([pos], np.int32), d, rotary, ts, mode=mode, weight=kw, ff=ffv, eps=1e-6)[0]
    assert (np.abs(rq - q_ref) <= k_tolerance(q_ref, pos)).all()
    tol = k_tolerance(k_ref, pos)
    assert (np.abs(rko - k_ref) <= tol).all()
    if dtype == vf.KvDtype.F8:
        k_code, enc = rk, oracle.f32_to_e4m3
    elif dtype == vf.KvDtype.F16:
        k_code, enc = rk.view(np.uint16), oracle.f32_to_f16_bits
    else:
        k_code, enc = rk.view(np.float32), lambda x: x                                      # noqa: E731
    assert (k_code == enc(rko.reshape(-1))).all()           # the cache holds the conversion of exactly what k_out holds
    # The attention: the oracle over the rotated queries and the row as the GPU produced them (the angle's ulp, times K entries of
    # +-40, would otherwise move a score by more than this path's output tolerance)
    ke = np.concatenate([encode_np(k_hist.reshape(ctx - 1, hkv, d), dtype), k_code.reshape(1, hkv, d)])
    ve = encode_np(np.concatenate([v_hist.reshape(ctx - 1, hkv, d), v_new[None]]), dtype)
    assert (ve[ctx - 1].reshape(-1).view(np.uint8) == rv).all()      # V bytes: what vfkv_kv_write stores
    ref = oracle.attn_decode_ref(rq, ke, ve, int(dtype), heads, hkv, d, ctx, scale, kv_start=kv_start, softcap=cap)
    assert np.abs(ro - ref).max() < TOL[dtype]


def test_qk_rope_kv_write_decode_attention_rejects_bad_arguments():
    cache = vf.KvCache(vf.KvCacheConfig(1, 2, 64, 64, dtype=vf.KvDtype.F16))
    fwd = vf.Forward(cache, 4)
    q, o, kv = torch.zeros((4, 64), device=DEV), torch.zeros((4, 64), device=DEV), torch.zeros((2, 64), device=DEV)
    with pytest.raises(vf.VfkvError):
        fwd.step_qk_rope_kv_write_attention(0, 3, q, kv, kv, o, 64, 0.9, q_out=q)            # q_out overlaps q
    with pytest.raises(vf.VfkvError):
        fwd.step_qk_rope_kv_write_attention(0, 3, q, kv, kv, o, 63, 0.9)                     # odd rotary_dim
    with pytest.raises(vf.VfkvError):
        fwd.step_qk_rope_kv_write_attention(0, 3, q, kv, kv, o, 64, 0.9, rope_mode=1)        # unsupported mode
    with pytest.raises(vf.VfkvError):
        fwd.step_qk_rope_kv_write_attention(0, 3, q, None, kv, o, 64, 0.9)                   # no K row
    cache.destroy()
