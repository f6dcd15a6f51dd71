"""The allocation-free decode entry point (vfkv_decode_attention_static) against vfkv_decode_attention: same inputs,
called through the C ABI, outputs must be bit-identical (same kernels, same tile choice; only where the partials live
differs) and within the path's tolerance of the CPU oracle.  Two calls in a row share the library's static array; the
second is smaller, so anything the first one left behind would be visible."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, TOL, encode_np, fp16_normal, outlier_normal, rng, to_dev, to_np
from vulkanforge_amd import _ffi

pytestmark = pytest.mark.gpu


def _filled_cache(dtype, hkv, d, max_seq, seed):
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, max_seq, dtype=dtype))
    cache.zero_fill()
    r = rng(seed)
    k, v = fill(r, (max_seq, hkv * d)), fill(r, (max_seq, hkv * d))
    vf.Forward(cache, 1).b_step_kv_write(0, 0, max_seq, to_dev(k), to_dev(v))
    torch.cuda.synchronize()
    return cache, k, v


def _both(cache, heads, d, q, position, kv_start, softcap=0.0):
    """(output of the static entry point, output of vfkv_decode_attention) for one query."""
    L = _ffi.lib()
    scale = 1.0 / np.sqrt(d)
    stream = torch.cuda.current_stream().cuda_stream
    qd = to_dev(q)
    o_static = torch.full((heads, d), float("nan"), device=DEV)
    o_ws = torch.full((heads, d), float("nan"), device=DEV)
    _ffi.check(L.vfkv_decode_attention_static(cache.handle, 0, 0, heads, qd.data_ptr(), o_static.data_ptr(), position,
                                              kv_start, scale, softcap, stream))
    ws = C.c_void_p()
    _ffi.check(L.vfkv_workspace_create(heads, d, position + 1, C.byref(ws)))
    _ffi.check(L.vfkv_decode_attention(cache.handle, 0, 0, heads, qd.data_ptr(), o_ws.data_ptr(), position, kv_start,
                                       scale, softcap, ws, stream))
    torch.cuda.synchronize()
    L.vfkv_workspace_destroy(ws)
    return to_np(o_static), to_np(o_ws)


@pytest.mark.parametrize("dtype,heads,hkv,d,first,second", [
    (vf.KvDtype.F8, 32, 8, 128, (8191, 0), (1499, 0)),          # 32 partials per head, then 8
    (vf.KvDtype.F16, 16, 8, 256, (6000, 1904), (700, 0)),       # sliding window, then a short context
    (vf.KvDtype.F8, 16, 2, 512, (9000, 0), (100, 0)),           # 128 partials per head (four-wavefront merge), then 2
    (vf.KvDtype.F32, 8, 2, 128, (2500, 0), (63, 0)),            # vector-ALU worker, then a single tile
])
def test_static_scratch_matches_workspace_call_twice_in_a_row(dtype, heads, hkv, d, first, second):
    max_seq = first[0] + 1
    cache, k, v = _filled_cache(dtype, hkv, d, max_seq, 300 + d + heads)
    ke, ve = encode_np(k, dtype).reshape(-1, hkv, d), encode_np(v, dtype).reshape(-1, hkv, d)
    for n, (position, kv_start) in enumerate((first, second)):
        print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} position={position} kv_start={kv_start} call={n}", flush=True)
        q = fp16_normal(rng(310 + n), (heads, d))
        o_static, o_ws = _both(cache, heads, d, q, position, kv_start)
        assert np.array_equal(o_static, o_ws)
        ref = oracle.attn_decode_ref(q, ke, ve, int(dtype), heads, hkv, d, position + 1, 1.0 / np.sqrt(d), kv_start=kv_start)
        assert np.abs(o_static - ref).max() < TOL[dtype]
    cache.destroy()


def test_static_scratch_call_captured_into_a_graph_replays_like_eager():
    # the callers this entry point is for: a decode step under HIP graph capture.  The array's address is looked up on the
    # first (eager) call; the captured calls then only enqueue kernels.  Every replay, with new queries and eager work in
    # between, must reproduce the eager call bit for bit.
    dtype, heads, hkv, d, ctx, layers = vf.KvDtype.F8, 32, 8, 128, 5000, 2
    L = _ffi.lib()
    cache = vf.KvCache(vf.KvCacheConfig(layers, hkv, d, ctx, dtype=dtype))
    cache.zero_fill()
    r = rng(910)
    fwd = vf.Forward(cache, heads)
    for layer in range(layers):
        fwd.b_step_kv_write(layer, 0, ctx, to_dev(outlier_normal(r, (ctx, hkv * d))), to_dev(outlier_normal(r, (ctx, hkv * d))))
    q = torch.zeros((layers, heads, d), device=DEV)
    o = torch.zeros((layers, heads, d), device=DEV)
    scale = 1.0 / np.sqrt(d)

    def step(out):
        stream = torch.cuda.current_stream().cuda_stream
        for layer in range(layers):
            _ffi.check(L.vfkv_decode_attention_static(cache.handle, layer, layer, heads, q[layer].data_ptr(), out[layer].data_ptr(),
                                                      ctx - 1, 0, scale, 0.0, stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(o)                                  # first use outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(o)
    for rep in range(3):
        print(f"case graph replay {rep}", flush=True)
        q.copy_(to_dev(fp16_normal(r, (layers, heads, d))))
        graph.replay()
        torch.cuda.synchronize()
        got = to_np(o).copy()
        o_eager = torch.full_like(o, float("nan"))
        step(o_eager)
        torch.cuda.synchronize()
        assert np.isfinite(got).all() and np.array_equal(got, to_np(o_eager)), rep
        (q * 2).sum().item()                     # unrelated eager work between replays
    cache.destroy()
