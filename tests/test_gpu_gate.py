"""Gated attention output on the GPU (executor/attention.rs:632-680, 2405-2444; vk_shaders/sigmoid_mul.comp).

The standalone kernel is checked against the CPU oracle (the exponential differs between libraries by an ulp, hence a
relative bound of 4 ulp of the product); the fused decode / prefill calls must be bit-identical to attention followed by
the standalone kernel, whose parity with the oracle the other files establish."""
import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, fp16_normal, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


def close_to_oracle(got, want):
    # below the smallest normal f32 the two differ by construction: exp(-g) overflows in f32 (the shader's arithmetic, so the
    # product is 0) where the oracle's f64 evaluation still yields a subnormal
    return (np.abs(got - want) <= 4 * np.spacing(np.abs(want).astype(np.float32)) + np.float32(1.2e-38)).all()


@pytest.mark.parametrize("tokens,chunk,stride,offset", (
    (1, 4096, 4096, 4096),     # decode, 32 heads x 128 (gate behind Q in q_buf)
    (512, 128, 256, 128),      # a prefill chunk, per (token, head) slices [Q | G]: 32 heads -> 32 chunks per token
    (7, 96, 200, 52),          # 16-byte path with odd sizes
    (5, 30, 71, 3),            # scalar path
    (3, 1, 2, 1),
))
def test_sigmoid_mul_matches_oracle(tokens, chunk, stride, offset):
    r = rng(tokens * 1000 + chunk)
    n_chunks = tokens * (32 if (chunk, stride) == (128, 256) else 1)
    ne = n_chunks * chunk
    gate = (r.standard_normal(n_chunks * stride + offset + chunk) * 4).astype(np.float32)
    gate[:8] = [0.0, -100.0, 100.0, -1000.0, 88.0, -88.0, 1e-8, -20.0]
    data = r.standard_normal(ne).astype(np.float32)
    print(f"case ne={ne} chunk={chunk} stride={stride} offset={offset}", flush=True)
    d = to_dev(data)
    vf.Forward.run_sigmoid_mul(to_dev(gate), d, ne, chunk, stride, offset)
    torch.cuda.synchronize()
    got, want = to_np(d), oracle.sigmoid_mul(gate, data, chunk, stride, offset)
    assert np.isfinite(got).all() and close_to_oracle(got, want)


def test_sigmoid_mul_special_values_and_unaligned_views():
    g = np.array([0.0, 100.0, -1000.0, 0.0], dtype=np.float32)
    x = np.array([3.0, 3.0, 3.0, -8.0], dtype=np.float32)
    d = to_dev(x)
    vf.Forward.run_sigmoid_mul(to_dev(g), d, 4, 4, 4, 0)
    torch.cuda.synchronize()
    assert (to_np(d) == np.array([1.5, 3.0, 0.0, -4.0], dtype=np.float32)).all()
    # 4-byte aligned views of both buffers: the scalar kernel serves them, neighbours stay untouched
    r = rng(3)
    gate, data = r.standard_normal(64).astype(np.float32), r.standard_normal(64).astype(np.float32)
    gd, dd = to_dev(gate), to_dev(data)
    vf.Forward.run_sigmoid_mul(gd[1:], dd[3:], 40, 8, 8, 0)
    torch.cuda.synchronize()
    got = to_np(dd)
    want = data.copy()
    want[3:43] = oracle.sigmoid_mul(gate[1:], data[3:43], 8, 8, 0)
    assert (got[:3] == data[:3]).all() and (got[43:] == data[43:]).all() and close_to_oracle(got, want)
    # ne = 0 is a no-op
    vf.Forward.run_sigmoid_mul(gd, dd, 0, 8, 8, 0)


DECODE_CASES = (
    # dtype, H, Hkv, D, n (context), window, append
    (vf.KvDtype.F8, 32, 8, 128, 5000, 0, True),        # merge applies the gate, worker appends
    (vf.KvDtype.F8, 32, 8, 128, 5000, 0, False),
    (vf.KvDtype.F16, 16, 8, 256, 3000, 1024, True),
    (vf.KvDtype.F8, 16, 4, 128, 100, 0, True),         # one tile: the worker writes o, the gate runs as its own launch
    (vf.KvDtype.F32, 8, 2, 64, 700, 0, True),          # vector-ALU worker, separate append
    (vf.KvDtype.F8, 6, 2, 80, 300, 0, False),          # head_dim 80: the ragged form of the merge applies the gate
    (vf.KvDtype.F16, 32, 32, 96, 2500, 0, True),       # Phi-3 geometry with a gate
    (vf.KvDtype.F32, 6, 2, 72, 300, 0, False),         # generic worker; the ragged merge still takes the gate
    (vf.KvDtype.F32, 2, 1, 72, 9000, 0, False),        # generic kernels with more than 64 partials: the merge cannot take the gate
    (vf.KvDtype.F16, 8, 1, 256, 12000, 0, True),       # one KV head, 188 tiles: the four-wavefront merge applies the gate
)


@pytest.mark.parametrize("dtype,heads,hkv,d,n,window,append", DECODE_CASES)
def test_decode_attention_gated_is_attention_then_gate(dtype, heads, hkv, d, n, window, append):
    r = rng(n + d)
    caches = [vf.KvCache(vf.KvCacheConfig(1, hkv, d, n, dtype=dtype)) for _ in range(2)]
    k, v = fp16_normal(r, (n, hkv, d)), fp16_normal(r, (n, hkv, d))
    q_dim = heads * d
    qbuf = np.concatenate([fp16_normal(r, q_dim), (r.standard_normal(q_dim) * 3).astype(np.float32)])   # [Q | G] as q_buf holds them
    outs = []
    pos = n - 1
    kv_start = vf._ffi.lib().vfkv_kv_start_decode(pos, window) if window else 0
    print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} n={n} kv_start={kv_start} append={append}", flush=True)
    for i, cache in enumerate(caches):
        fwd = vf.Forward(cache, heads)
        hist = n - 1 if append else n
        fwd.b_step_kv_write(0, 0, hist, to_dev(k[:hist]), to_dev(v[:hist]))
        qd = to_dev(qbuf)
        o = torch.empty(q_dim, device=DEV)
        kn, vn = (to_dev(k[pos]), to_dev(v[pos])) if append else (None, None)
        if i == 0:
            fwd.step_attention_gated(0, pos, qd, o, qd, q_dim, q_dim, q_dim, k_src=kn, v_src=vn, kv_start=kv_start)
        else:
            if append:
                fwd.step_kv_write_attention(0, pos, qd, kn, vn, o, kv_start=kv_start)
            else:
                fwd.run_scalar_attn(0, pos, qd, o, kv_start=kv_start)
            fwd.step_attn_gated_output(o, qd, q_dim)
        torch.cuda.synchronize()
        outs.append(to_np(o))
    assert (outs[0] == outs[1]).all()
    # and against the oracle end to end
    from gpu_util import TOL, encode_np
    ref = oracle.attn_decode_ref(qbuf[:q_dim].reshape(heads, d), encode_np(k, dtype), encode_np(v, dtype), int(dtype), heads, hkv, d,
                                 n, float(1.0 / np.sqrt(d)), kv_start=kv_start)
    ref = oracle.sigmoid_mul(qbuf, ref.reshape(-1), q_dim, q_dim, q_dim)
    assert np.abs(outs[0] - ref).max() < TOL[dtype]
    for c in caches:
        c.destroy()


@pytest.mark.parametrize("dtype,heads,hkv,d,m,base", (
    (vf.KvDtype.F8, 16, 4, 128, 70, 300), (vf.KvDtype.F16, 8, 2, 256, 33, 0),
    (vf.KvDtype.F8, 12, 4, 128, 17, 40),        # odd group: a padded head slot stores nothing
    (vf.KvDtype.F8, 8, 2, 512, 21, 100),        # two wavefronts share a head, each gates its own output columns
    (vf.KvDtype.F16, 4, 4, 64, 1, 0),
    (vf.KvDtype.F32, 4, 2, 128, 20, 10),        # kernels without a gated store: the gate follows as its own launch
    (vf.KvDtype.F8, 6, 2, 96, 20, 10),          # heads of 96 elements on the kernel for 128: the gate keeps its real stride
    (vf.KvDtype.F16, 32, 32, 80, 40, 100),      # one head per wavefront
    (vf.KvDtype.F16, 8, 4, 192, 18, 30),
    (vf.KvDtype.F8, 8, 8, 128, 45, 100),        # groups of one head: each of a wavefront's two query blocks gates its own rows
    (vf.KvDtype.F8, 128, 32, 128, 125, 200),    # 256 workgroups: two head pairs x four key splits, every wavefront gates the tiles it stores
))
def test_prefill_attention_gated_is_attention_then_gate(dtype, heads, hkv, d, m, base):
    r = rng(m + d)
    n = base + m
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, n, dtype=dtype))
    fwd = vf.Forward(cache, heads)
    k, v = fp16_normal(r, (n, hkv, d)), fp16_normal(r, (n, hkv, d))
    fwd.b_step_kv_write(0, 0, n, to_dev(k), to_dev(v))
    qg = r.standard_normal((m, heads, 2, d)).astype(np.float32)      # per (token, head): [Q | G]
    q = to_dev(np.ascontiguousarray(qg[:, :, 0]))
    gate = to_dev(qg)
    a, b = torch.empty((m, heads, d), device=DEV), torch.empty((m, heads, d), device=DEV)
    fwd.b_step_attention_gated(0, base, m, q, a, gate, d, 2 * d, d)
    fwd.b_step_attention(0, base, m, q, b)
    fwd.b_step_attn_gated_output(b, gate, m, d)
    torch.cuda.synchronize()
    assert (to_np(a) == to_np(b)).all()
    from gpu_util import TOL, encode_np
    ref = oracle.attn_batch_ref(np.ascontiguousarray(qg[:, :, 0]), encode_np(k, dtype), encode_np(v, dtype), int(dtype), m, n, heads,
                                hkv, d, base, float(1.0 / np.sqrt(d)))
    ref = oracle.sigmoid_mul(qg.reshape(-1), ref.reshape(-1), d, 2 * d, d).reshape(m, heads, d)
    assert np.abs(to_np(a) - ref).max() < TOL[dtype]
    cache.destroy()


@pytest.mark.parametrize("layout", ("token_chunks", "token_chunks_interleaved", "half_head_chunks", "unaligned_gate"))
def test_prefill_attention_gated_gate_layouts(layout):
    # gate geometries that do and do not qualify for the attention kernel's own gated store give the same bits
    dtype, heads, hkv, d, m, base = vf.KvDtype.F8, 8, 2, 128, 40, 200
    r = rng(len(layout))
    n = base + m
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, n, dtype=dtype))
    fwd = vf.Forward(cache, heads)
    fwd.b_step_kv_write(0, 0, n, to_dev(fp16_normal(r, (n, hkv, d))), to_dev(fp16_normal(r, (n, hkv, d))))
    q = to_dev(r.standard_normal((m, heads, d)).astype(np.float32))
    row = heads * d
    chunk, stride, off = {"token_chunks": (row, row, 0), "token_chunks_interleaved": (row, 2 * row, row),
                          "half_head_chunks": (d // 2, d, d // 2), "unaligned_gate": (row, row, 0)}[layout]
    n_gate = (m * row // chunk) * stride + off + chunk
    gbuf = to_dev(r.standard_normal(n_gate + 1).astype(np.float32) * 3)
    gate = gbuf[1:] if layout == "unaligned_gate" else gbuf[:-1]
    a, b = torch.empty((m, heads, d), device=DEV), torch.empty((m, heads, d), device=DEV)
    fwd.b_step_attention_gated(0, base, m, q, a, gate, chunk, stride, off)
    fwd.b_step_attention(0, base, m, q, b)
    torch.cuda.synchronize()
    plain = to_np(b).reshape(-1)
    fwd.run_sigmoid_mul(gate, b, m * row, chunk, stride, off)
    torch.cuda.synchronize()
    assert (to_np(a) == to_np(b)).all()
    assert close_to_oracle(to_np(a).reshape(-1), oracle.sigmoid_mul(to_np(gate), plain, chunk, stride, off))
    cache.destroy()


def test_gated_calls_reject_bad_arguments():
    cache = vf.KvCache(vf.KvCacheConfig(2, 2, 64, 64, dtype=vf.KvDtype.F16))
    fwd = vf.Forward(cache, 4)
    q, o = torch.zeros(256, device=DEV), torch.zeros(256, device=DEV)
    with pytest.raises(vf.VfkvError):
        fwd.step_attention_gated(0, 3, q, o, None, 256, 256, 0)                     # no gate
    with pytest.raises(vf.VfkvError):
        fwd.step_attention_gated(0, 3, q, o, q, 0, 256, 0)                          # chunk 0
    with pytest.raises(vf.VfkvError):
        fwd.step_attention_gated(0, 3, q, o, q, 256, 256, 0, k_src=q[:128])         # K without V
    with pytest.raises(vf.VfkvError):
        fwd.step_attention_gated(1, 3, q, o, q, 256, 256, 0, k_src=q[:128], v_src=q[:128], kv_layer=0)   # appends into a foreign slab
    with pytest.raises(vf.VfkvError):
        vf.Forward.run_sigmoid_mul(q, None, 16, 16, 16, 0)
    cache.destroy()
