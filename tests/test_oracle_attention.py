"""Pins the oracle's attention routines (CPU only): golden outputs of the reference's closed-form
fixtures computed independently in float64 with scipy, textbook special cases, tile invariance of
split + log-sum-exp merge, and the reference's own naive-vs-tiled cases."""
import os

import numpy as np
import pytest
import scipy.special

import oracle
from refgen import (BATCH_CASES, D, DECODE_SEQS, H, HKV, batch_inputs, decode_inputs, golden_rows,
                    xorshift_floats)

SCALE = float(np.float32(1.0) / np.sqrt(np.float32(D)))


@pytest.fixture(scope="module")
def golden(golden_dir):
    return np.load(os.path.join(golden_dir, "attn_cases.npz"))


def _library_attention(q, k, v, g, scale, lo, hi, cap=0.0):
    """float64 numpy + scipy softmax; q [H,D], k/v [T,Hkv,D] (already decoded to float)."""
    out = np.zeros(q.shape)
    for h in range(q.shape[0]):
        s = (k[lo:hi, h // g].astype(np.float64) @ q[h].astype(np.float64)) * scale
        if cap:
            s = cap * np.tanh(s / cap)
        out[h] = scipy.special.softmax(s) @ v[lo:hi, h // g].astype(np.float64)
    return out


@pytest.mark.parametrize("seq", DECODE_SEQS)
def test_decode_ref_matches_golden(golden, seq):
    q, k, v = decode_inputs(seq)
    got = oracle.attn_decode_ref(q, k, v, oracle.F32, H, HKV, D, seq, SCALE)
    assert np.abs(got - golden[f"decode_seq{seq}_out"]).max() < 2e-6


@pytest.mark.parametrize("seq", (64, 200, 2048))
def test_split_reduce_matches_golden_at_reference_tolerance(golden, seq):
    # tests/correctness.rs:2875-2894: split + reduce vs CPU < 1e-3 with TILE = 64
    q, k, v = decode_inputs(seq)
    so, sm, ss = oracle.attn_split(q, k, v, oracle.F32, H, HKV, D, seq, SCALE, tile=64)
    got = oracle.attn_reduce(so, sm, ss)
    assert np.abs(got - golden[f"decode_seq{seq}_out"]).max() < 1e-3
    assert np.abs(got - golden[f"decode_seq{seq}_out"]).max() < 2e-5  # what f32 actually achieves


def test_seq1_returns_v0_exactly():
    # tests/correctness.rs:2765-2770
    q, k, v = decode_inputs(1)
    got = oracle.attn_decode_ref(q, k, v, oracle.F32, H, HKV, D, 1, SCALE)
    exp = np.repeat(v[0], H // HKV, axis=0)
    assert (got == exp).all()
    so, sm, ss = oracle.attn_split(q, k, v, oracle.F32, H, HKV, D, 1, SCALE, tile=64)
    assert (oracle.attn_reduce(so, sm, ss) == exp).all()


def test_constant_keys_give_mean_of_values():
    rng = np.random.default_rng(1)
    seq = 300
    q = rng.standard_normal((H, D)).astype(np.float32)
    k = np.broadcast_to(rng.standard_normal((1, HKV, D)).astype(np.float32), (seq, HKV, D)).copy()
    v = rng.standard_normal((seq, HKV, D)).astype(np.float32)
    got = oracle.attn_decode_ref(q, k, v, oracle.F32, H, HKV, D, seq, SCALE)
    exp = np.repeat(v.astype(np.float64).mean(axis=0), H // HKV, axis=0)
    assert np.abs(got - exp).max() < 1e-5


def test_one_dominant_key_selects_its_value():
    rng = np.random.default_rng(2)
    seq = 100
    q = rng.standard_normal((H, D)).astype(np.float32)
    k = np.zeros((seq, HKV, D), dtype=np.float32)
    v = rng.standard_normal((seq, HKV, D)).astype(np.float32)
    for h in range(HKV):
        k[17 + h, h] = 50.0 * q[h * (H // HKV)] / np.linalg.norm(q[h * (H // HKV)])
    got = oracle.attn_decode_ref(q, k, v, oracle.F32, H, HKV, D, seq, 1.0)
    for h in range(HKV):
        assert np.abs(got[h * (H // HKV)] - v[17 + h, h]).max() < 1e-6


@pytest.mark.parametrize("dtype", (oracle.F32, oracle.F16, oracle.F8))
@pytest.mark.parametrize("hkv,d", ((8, 128), (8, 256), (2, 64), (1, 512)))
def test_decode_ref_vs_library_random(dtype, hkv, d):
    rng = np.random.default_rng(100 + d + hkv)
    heads, seq = hkv * 2, 333
    q = rng.standard_normal((heads, d)).astype(np.float32)
    kf = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    vf = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    if dtype == oracle.F32:
        k, v, kd, vd = kf, vf, kf, vf
    elif dtype == oracle.F16:
        k, v = kf.astype(np.float16).view(np.uint16), vf.astype(np.float16).view(np.uint16)
        kd, vd = k.view(np.float16).astype(np.float32), v.view(np.float16).astype(np.float32)
    else:
        k, v = oracle.f32_to_e4m3(kf), oracle.f32_to_e4m3(vf)
        kd, vd = oracle.e4m3_to_f32(k), oracle.e4m3_to_f32(v)
    scale = 1.0 / np.sqrt(d)
    for kv_start, cap in ((0, 0.0), (100, 0.0), (0, 5.0), (37, 50.0)):
        got = oracle.attn_decode_ref(q, k, v, dtype, heads, hkv, d, seq, scale, kv_start=kv_start,
                                     softcap=cap)
        exp = _library_attention(q, kd, vd, 2, scale, kv_start, seq, cap)
        assert np.abs(got - exp).max() < 3e-6, (kv_start, cap)


@pytest.mark.parametrize("tile", (1, 7, 64, 100, 512, 4096))
def test_split_reduce_tile_invariance(tile):
    # tests/flash_attn_tiled_ref.rs:279-295 -- same answer for every tile shape
    rng = np.random.default_rng(9)
    seq, hkv, heads, d = 1000, 4, 16, 64
    q = rng.standard_normal((heads, d)).astype(np.float32)
    k = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    v = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    for kv_start, cap in ((0, 0.0), (130, 0.0), (999, 0.0), (64, 30.0)):
        ref = oracle.attn_decode_ref(q, k, v, oracle.F32, heads, hkv, d, seq, 0.125, kv_start=kv_start,
                                     softcap=cap)
        so, sm, ss = oracle.attn_split(q, k, v, oracle.F32, heads, hkv, d, seq, 0.125, tile=tile,
                                       kv_start=kv_start, softcap=cap)
        assert np.abs(oracle.attn_reduce(so, sm, ss) - ref).max() < 1e-5


def test_split_partials_below_window_are_empty():
    # flash_attn_split.comp:64-69: tiles entirely below kv_start contribute zero partials
    q, k, v = decode_inputs(400)
    so, sm, ss = oracle.attn_split(q, k, v, oracle.F32, H, HKV, D, 400, SCALE, tile=64, kv_start=200)
    assert (sm[:, :3] == np.float32(-1e30)).all() and (ss[:, :3] == 0).all() and (so[:, :3] == 0).all()
    assert (ss[:, 3:] > 0).all()
    # weights of each head sum to one after the merge: merge of (l_j) alone gives L, and O = acc / L
    ones = np.ones_like(v)
    so1, sm1, ss1 = oracle.attn_split(q, k, ones, oracle.F32, H, HKV, D, 400, SCALE, tile=64, kv_start=200)
    assert np.abs(oracle.attn_reduce(so1, sm1, ss1) - 1.0).max() < 1e-6


def test_kv_start_equals_shifted_slab():
    rng = np.random.default_rng(21)
    seq, s0 = 500, 123
    q = rng.standard_normal((H, D)).astype(np.float32)
    k = rng.standard_normal((seq, HKV, D)).astype(np.float32)
    v = rng.standard_normal((seq, HKV, D)).astype(np.float32)
    a = oracle.attn_decode_ref(q, k, v, oracle.F32, H, HKV, D, seq, SCALE, kv_start=s0)
    b = oracle.attn_decode_ref(q, k[s0:].copy(), v[s0:].copy(), oracle.F32, H, HKV, D, seq - s0, SCALE)
    assert (a == b).all()


@pytest.mark.parametrize("m,q_start", BATCH_CASES)
def test_batch_ref_matches_golden(golden, m, q_start):
    q, k, v = batch_inputs(m, q_start)
    got = oracle.attn_batch_ref(q, k, v, oracle.F32, m, q_start + m, H, HKV, D, q_start, SCALE)
    assert np.abs(got[golden_rows(m)] - golden[f"batch_m{m}_qs{q_start}_out"]).max() < 1e-6


@pytest.mark.parametrize("m,q_start,tol", ((1, 0, 1e-4), (4, 0, 1e-3), (16, 0, 1e-3), (64, 0, 1e-3),
                                           (200, 0, 5e-3), (4, 60, 1e-3)))
def test_batch_shader_within_reference_tolerances(golden, m, q_start, tol):
    # tests/correctness.rs:3158-3201
    q, k, v = batch_inputs(m, q_start)
    got = oracle.attn_batch_shader(q, k, v, oracle.F32, m, q_start + m, H, HKV, D, q_start, SCALE)
    err = np.abs(got[golden_rows(m)] - golden[f"batch_m{m}_qs{q_start}_out"]).max()
    assert err < tol and err < 2e-5


def test_batch_m1_equals_decode_and_causal_isolation():
    # tests/correctness.rs:3203-3279 and :3281-3386
    q, k, v = batch_inputs(4, 0)
    full = oracle.attn_batch_ref(q, k, v, oracle.F32, 4, 4, H, HKV, D, 0, SCALE)
    one = oracle.attn_batch_ref(q[:1].copy(), k[:1].copy(), v[:1].copy(), oracle.F32, 1, 1, H, HKV, D, 0, SCALE)
    assert np.abs(full[0] - one[0]).max() < 1e-6
    assert (np.abs(full[3] - one[0]) > 1e-3).sum() > H * D // 8
    dec = oracle.attn_decode_ref(q[3], k, v, oracle.F32, H, HKV, D, 4, SCALE)
    assert np.abs(dec - full[3]).max() < 1e-6
    sh = oracle.attn_batch_shader(q, k, v, oracle.F32, 4, 4, H, HKV, D, 0, SCALE)
    assert np.abs(sh - full).max() < 1e-5


@pytest.mark.parametrize("dtype", (oracle.F32, oracle.F8))
def test_batch_ref_vs_library_with_window_and_cap(dtype):
    rng = np.random.default_rng(33)
    m, q_start, hkv, heads, d = 24, 200, 2, 8, 64
    n_kv = q_start + m
    q = rng.standard_normal((m, heads, d)).astype(np.float32)
    kf = rng.standard_normal((n_kv, hkv, d)).astype(np.float32)
    vf = rng.standard_normal((n_kv, hkv, d)).astype(np.float32)
    if dtype == oracle.F8:
        k, v = oracle.f32_to_e4m3(kf), oracle.f32_to_e4m3(vf)
        kd, vd = oracle.e4m3_to_f32(k), oracle.e4m3_to_f32(v)
    else:
        k, v, kd, vd = kf, vf, kf, vf
    for kv_start, cap in ((0, 0.0), (70, 0.0), (129, 20.0)):
        got = oracle.attn_batch_ref(q, k, v, dtype, m, n_kv, heads, hkv, d, q_start, 0.125,
                                    kv_start=kv_start, softcap=cap)
        sh = oracle.attn_batch_shader(q, k, v, dtype, m, n_kv, heads, hkv, d, q_start, 0.125,
                                      kv_start=kv_start, softcap=cap)
        for i in (0, 11, m - 1):
            exp = _library_attention(q[i], kd, vd, heads // hkv, 0.125, kv_start, q_start + i + 1, cap)
            assert np.abs(got[i] - exp).max() < 1e-6
            assert np.abs(sh[i] - exp).max() < 1e-5


@pytest.mark.parametrize("hd,seq,kv,q_start,seed", ((128, 32, 32, 0, 44), (128, 32, 96, 64, 45),
                                                    (128, 30, 64, 34, 46), (128, 128, 1152, 1024, 200)))
def test_reference_tiled_ref_cases(hd, seq, kv, q_start, seed):
    # tests/flash_attn_tiled_ref.rs:262-303: single head, xorshift inputs, naive == tiled < 1e-4
    q = xorshift_floats(seq * hd, seed).reshape(seq, 1, hd)
    k = xorshift_floats(kv * hd, seed + 1).reshape(kv, 1, hd)
    v = xorshift_floats(kv * hd, seed + 2).reshape(kv, 1, hd)
    scale = float(np.float32(1.0) / np.sqrt(np.float32(hd)))
    a = oracle.attn_batch_ref(q, k, v, oracle.F32, seq, kv, 1, 1, hd, q_start, scale)
    b = oracle.attn_batch_shader(q, k, v, oracle.F32, seq, kv, 1, 1, hd, q_start, scale)
    assert np.abs(a - b).max() < 1e-4
    i = seq - 1
    exp = _library_attention(q[i], k, v, 1, scale, 0, min(q_start + i + 1, kv))
    assert np.abs(a[i] - exp).max() < 1e-6
