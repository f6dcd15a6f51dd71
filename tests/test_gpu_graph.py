"""The decode entry points only enqueue kernels (no allocation, no memset, no synchronisation), so a caller may
capture them into a HIP graph.  A captured decode step is replayed several times with new inputs, with eager work
and synchronisations between the replays, and every replay must reproduce the eager result bit for bit."""
import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, fp16_normal, read_device, rng, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,ctx", ((vf.KvDtype.F8, 3000), (vf.KvDtype.F16, 200)))
def test_captured_decode_step_replays_like_eager(dtype, ctx):
    r = rng(int(dtype) * 100 + ctx)
    layers, h, hkv, d = 3, 32, 8, 128
    ts = float(oracle.rope_theta_scale(1e6, d))
    caches = [vf.KvCache(vf.KvCacheConfig(layers, hkv, d, ctx + 8, dtype=dtype)) for _ in range(2)]
    fwds = [vf.Forward(c, h) for c in caches]
    k0 = to_dev(fp16_normal(r, (ctx, hkv * d)))
    v0 = to_dev(fp16_normal(r, (ctx, hkv * d)))
    for c, f in zip(caches, fwds):
        c.zero_fill()
        for layer in range(layers):
            f.b_step_kv_write(layer, 0, ctx, k0, v0)
    w = to_dev((1 + 0.1 * r.standard_normal(d)).astype(np.float32))
    # static buffers of the graph
    q = torch.zeros((layers, h, d), device=DEV)
    kn = torch.zeros((layers, hkv * d), device=DEV)
    vn = torch.zeros((layers, hkv * d), device=DEV)
    o = torch.zeros((layers, h, d), device=DEV)
    pos = ctx

    def step(fwd, out):
        for layer in range(layers):
            # K-norm + RoPE + append of the new token, then append-free attention over [0, pos]
            fwd.step_k_rope_kv_write(layer, pos, 1, kn[layer], vn[layer], d, ts, k_norm_weight=w)
            fwd.run_scalar_attn(layer, pos, q[layer], out[layer])

    def step_fused(fwd, out):
        for layer in range(layers):
            fwd.step_kv_write_attention(layer, pos, q[layer], kn[layer], vn[layer], out[layer])

    for body in (step, step_fused):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body(fwds[0], o)                     # first use outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            body(fwds[0], o)
        for rep in range(4):
            q.copy_(to_dev(fp16_normal(r, (layers, h, d))))
            kn.copy_(to_dev(fp16_normal(r, (layers, hkv * d))))
            vn.copy_(to_dev(fp16_normal(r, (layers, hkv * d))))
            graph.replay()
            torch.cuda.synchronize()
            got = to_np(o).copy()
            # the same step issued eagerly on the second cache
            o_eager = torch.full_like(o, float("nan"))
            body(fwds[1], o_eager)
            torch.cuda.synchronize()
            assert np.isfinite(got).all()
            assert (got == to_np(o_eager)).all(), (body.__name__, rep)
            n = caches[0].bytes_per_buffer()
            assert (read_device(caches[0].k_ptr, n) == read_device(caches[1].k_ptr, n)).all()
            assert (read_device(caches[0].v_ptr, n) == read_device(caches[1].v_ptr, n)).all()
            (q * 2).sum().item()                 # unrelated eager work between replays
    for c in caches:
        c.destroy()


def test_captured_zero_layer_clears_on_every_replay():
    # zero_layer (kv_cache.rs:389-407: the MTP scratch layer is cleared per step) inside a graph: the rows written between
    # the replays are gone after each one, the neighbouring layers keep theirs.  Odd sizes exercise the byte-wise ends.
    hkv, d, n = 3, 20, 37                                  # F8 rows of 60 bytes: the layer slab is not a multiple of 16
    cache = vf.KvCache(vf.KvCacheConfig(3, hkv, d, n, dtype=vf.KvDtype.F8))
    fwd = vf.Forward(cache, 3)
    cache.zero_fill()
    r = rng(8)
    rows = to_dev(fp16_normal(r, (n, hkv * d)) + 1.0)
    for layer in range(3):
        fwd.b_step_kv_write(layer, 0, n, rows, rows)
    torch.cuda.synchronize()
    full = read_device(cache.k_ptr, cache.bytes_per_buffer()).copy()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        cache.zero_layer(1, stream=side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cache.zero_layer(1, stream=torch.cuda.current_stream().cuda_stream)
    lo, hi = cache.layer_offset_bytes(1), cache.layer_offset_bytes(2)
    for rep in range(3):
        fwd.b_step_kv_write(1, 0, n, rows, rows)           # eager work between the replays
        torch.cuda.synchronize()
        assert (read_device(cache.k_ptr, cache.bytes_per_buffer()) == full).all()
        graph.replay()
        torch.cuda.synchronize()
        for ptr in (cache.k_ptr, cache.v_ptr):
            got = read_device(ptr, cache.bytes_per_buffer())
            assert (got[lo:hi] == 0).all() and (got[:lo] == full[:lo]).all() and (got[hi:] == full[hi:]).all()
    cache.destroy()
