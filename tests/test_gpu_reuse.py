"""Cross-request prefix reuse and cross-layer KV share on the GPU.

Prefix reuse restates the three scenarios of the reference's byte-identity gate (tests/kv_reuse_ident.rs:1-32: clean,
divergent, overshoot) at the level of this path: a request is a token sequence, a token maps to fixed per-layer q / k / v
rows, the chunk goes through norm + RoPE + append and causal attention.  Keeping rows [0, k) of the previous request and
prefilling from base_pos k (server/state.rs:199-224) must leave the cache and the outputs as a fresh prefill leaves them.
"""
import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, fp16_normal, read_device, rng, to_dev, to_np

pytestmark = pytest.mark.gpu

H, HKV, D, LAYERS, VOCAB, MAX_SEQ = 8, 2, 128, 2, 40, 96


class Stack:
    """Two attention layers over one cache; a token id selects its rows in seeded tables."""

    def __init__(self, dtype):
        r = rng(1234)
        self.q = fp16_normal(r, (LAYERS, VOCAB, H, D))
        self.k = fp16_normal(r, (LAYERS, VOCAB, HKV, D))
        self.v = fp16_normal(r, (LAYERS, VOCAB, HKV, D))
        self.wq = (1 + 0.1 * r.standard_normal(D)).astype(np.float32)
        self.wk = (1 + 0.1 * r.standard_normal(D)).astype(np.float32)
        self.ts = float(oracle.rope_theta_scale(1e6, D))
        self.cache = vf.KvCache(vf.KvCacheConfig(LAYERS, HKV, D, MAX_SEQ, dtype=dtype))
        self.cache.zero_fill()
        self.fwd = vf.Forward(self.cache, H)
        self.cached_tokens = []

    def prefill(self, tokens, base_pos, use_workspace=False):
        """Rows [base_pos, len(tokens)) of every layer; returns the attention outputs of those rows."""
        ids = np.asarray(tokens[base_pos:], dtype=np.int64)
        m = len(ids)
        outs = []
        for layer in range(LAYERS):
            q = to_dev(self.q[layer][ids])
            o = torch.empty((m, H, D), device=DEV)
            self.fwd.step_qk_rope_kv_write(layer, base_pos, m, q, to_dev(self.k[layer][ids]), to_dev(self.v[layer][ids]),
                                           D, self.ts, q_norm_weight=to_dev(self.wq), k_norm_weight=to_dev(self.wk))
            self.fwd.b_step_attention(layer, base_pos, m, q, o, use_workspace=use_workspace)
            outs.append(o)
        torch.cuda.synchronize()
        self.cache.current_seq_len = len(tokens)
        return np.stack([to_np(o) for o in outs])

    def request(self, tokens, overshoot=0):
        """ServerSession::generate_reuse (server/state.rs:199-224) without the generation."""
        k = vf.prefix_reuse_start(self.cached_tokens, tokens)
        k = min(k + overshoot, len(self.cached_tokens), len(tokens) - 1)      # the VF_KV_REUSE_OVERSHOOT hook, :206-212
        if k == 0:
            self.cache.reset()
        else:
            self.cache.current_seq_len = k
        out = self.prefill(tokens, k)
        self.cached_tokens = list(tokens)
        return k, out

    def rows(self, n):
        """The first n rows of every layer, K then V, as bytes."""
        got = []
        for ptr in (self.cache.k_ptr, self.cache.v_ptr):
            buf = read_device(ptr, self.cache.bytes_per_buffer())
            for layer in range(LAYERS):
                off = self.cache.layer_offset_bytes(layer)
                got.append(buf[off:off + n * self.cache.row_bytes(layer)].copy())
        return np.concatenate(got)


@pytest.mark.parametrize("dtype", (vf.KvDtype.F8, vf.KvDtype.F16))
def test_clean_and_divergent_reuse_match_a_fresh_prefill(dtype):
    r = rng(5)
    first = list(r.integers(0, VOCAB, 50))
    clean = first + list(r.integers(0, VOCAB, 21))                 # the previous request plus a suffix
    divergent = clean[:33] + [(clean[33] + 1) % VOCAB] + list(r.integers(0, VOCAB, 30))   # overwrites stale rows 33..
    served = Stack(dtype)
    served.request(first)
    for tokens, want_k in ((clean, 50), (divergent, 33)):
        print(f"case dtype={dtype.label()} n={len(tokens)} k={want_k}", flush=True)
        k, out = served.request(tokens)
        assert k == want_k and served.cache.current_seq_len == len(tokens)
        # the same two chunks on an empty cache: bit-identical rows and outputs
        fresh = Stack(dtype)
        fresh.prefill(tokens[:k], 0)
        out2 = fresh.prefill(tokens, k)
        assert (served.rows(len(tokens)) == fresh.rows(len(tokens))).all()
        assert (out == out2).all()
        # one chunk on an empty cache: the same rows; the outputs agree to f32 rounding (other tile boundaries)
        single = Stack(dtype)
        full = single.prefill(tokens, 0)
        assert (served.rows(len(tokens)) == single.rows(len(tokens))).all()
        assert np.abs(full[:, k:] - out).max() < 2e-5
        fresh.cache.destroy(); single.cache.destroy()
    served.cache.destroy()


def test_short_suffix_over_a_long_reused_prefix_with_the_workspace():
    # the serving pattern of prefix reuse: a few new tokens over thousands of resident rows.  With the decode workspace the
    # keys are cut into chunks over workgroups; the result is that of a fresh prefill of the whole sequence.
    global MAX_SEQ
    old_max, MAX_SEQ = MAX_SEQ, 3000
    try:
        r = rng(9)
        first = list(r.integers(0, VOCAB, 2900))
        second = first[:2870] + list(r.integers(0, VOCAB, 40))
        served = Stack(vf.KvDtype.F8)
        served.fwd.workspace = vf.Workspace(H, D, 32768)
        served.request(first)
        k = vf.prefix_reuse_start(served.cached_tokens, second)
        assert k >= 2870
        served.cache.current_seq_len = k
        out = served.prefill(second, k, use_workspace=True)
        single = Stack(vf.KvDtype.F8)
        full = single.prefill(second, 0)
        assert (served.rows(len(second)) == single.rows(len(second))).all()
        assert np.abs(full[:, k:] - out).max() < 2e-5
        served.cache.destroy(); single.cache.destroy()
    finally:
        MAX_SEQ = old_max


def test_reuse_past_the_common_prefix_is_detectably_wrong():
    # the fault-injection scenario: rows [k, k + 4) still hold the previous request's tokens
    r = rng(6)
    first = list(r.integers(0, VOCAB, 40))
    second = first[:20] + [(t + 7) % VOCAB for t in first[20:30]] + list(r.integers(0, VOCAB, 12))
    served = Stack(vf.KvDtype.F8)
    served.request(first)
    k, out = served.request(second, overshoot=4)
    assert k == 24
    single = Stack(vf.KvDtype.F8)
    full = single.prefill(second, 0)
    assert (served.rows(20) == single.rows(20)).all()
    assert (served.rows(len(second)) != single.rows(len(second))).any()
    assert np.abs(full[:, k:] - out).max() > 1e-2
    served.cache.destroy(); single.cache.destroy()


def test_reset_keeps_the_bytes_and_zero_layer_clears_one_slab():
    # `reset()` only zeroes the counter (server/state.rs:221-224, kv_cache.rs:492-494); zero_layer, kv_cache.rs:389-407
    s = Stack(vf.KvDtype.F16)
    s.request(list(range(30)))
    before = s.rows(30)
    s.cache.reset()
    assert s.cache.current_seq_len == 0 and (s.rows(30) == before).all()
    s.cache.zero_layer(1)
    torch.cuda.synchronize()
    after = s.rows(30)
    per = 30 * s.cache.row_bytes(0)
    assert (after[:per] == before[:per]).all() and (after[per:2 * per] == 0).all()          # K: layer 0 kept, layer 1 zero
    assert (after[2 * per:3 * per] == before[2 * per:3 * per]).all() and (after[3 * per:] == 0).all()
    s.cache.destroy()


def test_subscriber_layers_read_the_publishers_rows():
    # Gemma-4 KV share (forward/arch/gemma4.rs:27-49, runs.rs:734): a subscriber layer attends over the slab of the first
    # publisher of its kind; its own slab is never written.  Sliding layers 128-wide, the full layer 256-wide.
    K = vf.kv_cache
    srcs = vf.build_kv_sources([True, False, True, False, True], 2, 5)
    assert srcs == [K.KV_OWN_PUBLISHES_SLIDING, K.KV_OWN_PUBLISHES_FULL, K.KV_SUBSCRIBES_SLIDING, K.KV_SUBSCRIBES_FULL,
                    K.KV_SUBSCRIBES_SLIDING]
    hd = [128, 256, 128, 256, 128]
    n, heads, hkv = 300, 8, 2
    cache = vf.KvCache(vf.KvCacheConfig(5, hkv, 128, n, dtype=vf.KvDtype.F16, per_layer_head_dim=hd))
    cache.zero_fill()
    fwd = vf.Forward(cache, heads)
    r = rng(77)
    kv = {}
    for layer in (0, 1):
        k, v = fp16_normal(r, (n, hkv, hd[layer])), fp16_normal(r, (n, hkv, hd[layer]))
        fwd.b_step_kv_write(layer, 0, n, to_dev(k), to_dev(v))
        kv[layer] = (k, v)
    for layer in range(5):
        d = hd[layer]
        src = vf.gemma4_kv_read_layer(srcs, layer)
        assert src == (layer if layer < 2 else (1 if layer == 3 else 0))
        q = fp16_normal(r, (heads, d))
        o = torch.empty((heads, d), device=DEV)
        window = 64 if layer % 2 == 0 else 0
        kv_start = vf._ffi.lib().vfkv_kv_start_decode(n - 1, window) if window else 0
        print(f"case layer={layer} kv_layer={src} head_dim={d} kv_start={kv_start}", flush=True)
        fwd.run_scalar_attn(layer, n - 1, to_dev(q), o, kv_layer=src, kv_start=kv_start)
        torch.cuda.synchronize()
        k, v = kv[src]
        ref = oracle.attn_decode_ref(q, oracle.f32_to_f16_bits(k), oracle.f32_to_f16_bits(v), int(vf.KvDtype.F16), heads, hkv, d,
                                     n, float(1.0 / np.sqrt(d)), kv_start=kv_start)
        assert np.abs(to_np(o) - ref).max() < 2e-3
    cache.destroy()
