"""GPU parity of chunked-prefill causal attention (flash_attn_batch) through the C ABI."""
import os

import numpy as np
import pytest
import torch

import oracle
import vulkanforge_amd as vf
from gpu_util import DEV, TIGHT, TOL, encode_np, fp16_normal, gpu_batch, outlier_normal, rng, to_dev, to_np
from refgen import BATCH_CASES, D, H, HKV, batch_inputs, golden_rows

pytestmark = pytest.mark.gpu
SCALE = float(np.float32(1.0) / np.sqrt(np.float32(D)))
REF_TOL = {(1, 0): 1e-4, (4, 0): 1e-3, (16, 0): 1e-3, (64, 0): 1e-3, (200, 0): 5e-3, (4, 60): 1e-3}


@pytest.mark.parametrize("m,q_start", BATCH_CASES)
def test_reference_batch_fixtures_f32(golden_dir, m, q_start):
    # tests/correctness.rs:3073-3201
    golden = np.load(os.path.join(golden_dir, "attn_cases.npz"))[f"batch_m{m}_qs{q_start}_out"]
    q, k, v = batch_inputs(m, q_start)
    o = gpu_batch(q, k, v, vf.KvDtype.F32, H, HKV, D, m, q_start, q_start + m, SCALE)
    assert np.isfinite(o).all()
    err = np.abs(o[golden_rows(m)] - golden).max()
    assert err < REF_TOL[(m, q_start)] and err < 2e-5, err
    ref = oracle.attn_batch_ref(q, k, v, oracle.F32, m, q_start + m, H, HKV, D, q_start, SCALE)
    assert np.abs(o - ref).max() < 2e-5


def test_m1_equals_decode_and_causal_isolation():
    # tests/correctness.rs:3203-3279 (M=1 == single-query attention) and :3281-3386
    q, k, v = batch_inputs(4, 0)
    full = gpu_batch(q, k, v, vf.KvDtype.F32, H, HKV, D, 4, 0, 4, SCALE)
    one = gpu_batch(q[:1].copy(), k[:1].copy(), v[:1].copy(), vf.KvDtype.F32, H, HKV, D, 1, 0, 1, SCALE)
    assert np.abs(full[0] - one[0]).max() < 1e-5
    assert (np.abs(full[3] - one[0]) > 1e-3).sum() > H * D // 8
    from gpu_util import gpu_split_reduce
    dec, *_ = gpu_split_reduce(q[3], k, v, vf.KvDtype.F32, H, HKV, D, 4, SCALE, tile=64)
    assert np.abs(dec - full[3]).max() < 1e-5


CASES = [
    # dtype, H, Hkv, D, m, q_start, kv_start, softcap
    (vf.KvDtype.F8, 32, 8, 128, 64, 200, 0, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 37, 0, 0, 0.0),
    (vf.KvDtype.F8, 32, 8, 128, 50, 300, 111, 0.0),
    (vf.KvDtype.F8, 16, 8, 128, 33, 100, 0, 25.0),
    (vf.KvDtype.F8, 8, 2, 256, 20, 150, 64, 0.0),
    (vf.KvDtype.F16, 32, 8, 128, 64, 200, 0, 0.0),
    (vf.KvDtype.F16, 16, 8, 256, 48, 500, 300, 50.0),
    (vf.KvDtype.F16, 4, 1, 512, 10, 70, 0, 0.0),
    (vf.KvDtype.F32, 12, 4, 64, 30, 90, 5, 0.0),
    (vf.KvDtype.F8, 6, 2, 80, 19, 45, 0, 0.0),
    (vf.KvDtype.F8, 64, 8, 128, 21, 77, 0, 0.0),      # G = 8
    (vf.KvDtype.F8, 4, 4, 64, 100, 30, 0, 0.0),       # G = 1, head_dim 64
    (vf.KvDtype.F16, 8, 8, 64, 17, 200, 190, 0.0),
    (vf.KvDtype.F16, 48, 4, 128, 5, 40, 0, 0.0),      # G = 12
    (vf.KvDtype.F8, 24, 8, 128, 40, 1000, 0, 0.0),    # G = 3: one head per wavefront, four key splits
    (vf.KvDtype.F8, 12, 2, 128, 23, 2100, 1500, 0.0), # G = 6: three head pairs, two key splits, window
    (vf.KvDtype.F8, 16, 8, 64, 70, 600, 0, 30.0),     # G = 2: one head pair, eight key splits, soft-cap
    (vf.KvDtype.F16, 16, 2, 128, 33, 900, 0, 0.0),    # G = 8 on a 2-byte cache
    (vf.KvDtype.F32, 32, 8, 128, 37, 500, 0, 0.0),    # F32 cache on the f32 matrix-core kernel: G = 4
    (vf.KvDtype.F32, 16, 2, 128, 20, 333, 120, 30.0), # G = 8 (two workgroups per KV head), window, soft-cap
    (vf.KvDtype.F32, 3, 3, 256, 18, 70, 0, 0.0),      # G = 1, head_dim 256
    (vf.KvDtype.F32, 10, 2, 64, 49, 0, 0, 0.0),       # G = 5: a workgroup with one live wavefront, from position 0
    (vf.KvDtype.F8, 28, 4, 128, 45, 800, 0, 0.0),     # G = 7: four head pairs per KV head, the last one half empty
    (vf.KvDtype.F16, 14, 2, 128, 19, 300, 100, 25.0), # G = 7 on a 2-byte cache, window, soft-cap
    (vf.KvDtype.F8, 10, 2, 64, 50, 400, 0, 0.0),      # G = 5, head_dim 64
    (vf.KvDtype.F16, 9, 3, 64, 31, 0, 0, 0.0),        # G = 3 from position 0
    (vf.KvDtype.F8, 8, 2, 512, 40, 300, 0, 30.0),     # head_dim 512 (two wavefronts per head, each half of the output columns), soft-cap
    (vf.KvDtype.F32, 4, 2, 512, 23, 150, 0, 0.0),     # head_dim 512 over an F32 cache: the same split on the f32 matrix-core kernel
    (vf.KvDtype.F8, 3, 1, 512, 70, 1000, 0, 0.0),     # head_dim 512, G = 3, several query blocks
    (vf.KvDtype.F16, 16, 2, 512, 20, 100, 64, 0.0),   # head_dim 512, G = 8, window
    (vf.KvDtype.F8, 12, 4, 96, 33, 200, 0, 0.0),      # head_dim 96: 4-byte loads of the 24-byte row quarters
    (vf.KvDtype.F16, 6, 6, 96, 17, 50, 10, 0.0),
    (vf.KvDtype.F32, 8, 4, 96, 21, 80, 0, 0.0),
    # the other head widths between the tiled ones, on the same f32 matrix-core kernel
    (vf.KvDtype.F16, 32, 32, 80, 40, 300, 0, 0.0),    # Phi-2 geometry (G = 1)
    (vf.KvDtype.F8, 8, 2, 80, 19, 100, 30, 20.0),
    (vf.KvDtype.F32, 6, 2, 112, 33, 150, 0, 0.0),
    (vf.KvDtype.F8, 16, 4, 112, 25, 90, 0, 0.0),
    (vf.KvDtype.F16, 8, 2, 160, 21, 200, 50, 0.0),
    (vf.KvDtype.F8, 12, 4, 192, 35, 120, 0, 30.0),
    (vf.KvDtype.F16, 4, 4, 224, 18, 70, 0, 0.0),
    (vf.KvDtype.F32, 4, 2, 192, 17, 60, 0, 0.0),
    # groups of one head: two blocks of 16 queries of the same head per wavefront, 32 queries per workgroup
    (vf.KvDtype.F16, 8, 8, 128, 47, 300, 0, 0.0),     # ragged: the last workgroup has 15 queries, all in its first block
    (vf.KvDtype.F16, 8, 8, 128, 49, 0, 0, 0.0),       # from position 0; the last workgroup's second block holds one query
    (vf.KvDtype.F8, 4, 4, 64, 100, 250, 200, 30.0),   # window that starts inside a tile, soft-cap
    (vf.KvDtype.F8, 16, 16, 256, 33, 500, 0, 0.0),
    (vf.KvDtype.F16, 4, 4, 256, 64, 300, 100, 0.0),   # window that starts past a tile boundary
    (vf.KvDtype.F8, 2, 2, 128, 17, 1000, 0, 0.0),     # one query in the second block
    (vf.KvDtype.F16, 3, 3, 64, 16, 40, 0, 0.0),       # 16 queries: one block, the one-head-per-wavefront form stays
    # more than eight KV heads over FP8 rows: the workgroups are renumbered so that an XCD takes one KV head at a time
    (vf.KvDtype.F8, 16, 16, 128, 50, 300, 0, 0.0),    # G = 1, ragged last query block
    (vf.KvDtype.F8, 32, 16, 64, 70, 200, 100, 0.0),   # G = 2 at head_dim 64, window
    (vf.KvDtype.F8, 32, 32, 96, 40, 300, 0, 0.0),     # Phi-3 geometry over an FP8 cache
    (vf.KvDtype.F8, 48, 24, 256, 20, 100, 0, 30.0),   # 24 KV heads, head_dim 256, soft-cap
    (vf.KvDtype.F8, 16, 8, 256, 48, 700, 0, 50.0),    # head_dim 256, G = 2: three key splits, soft-cap
    (vf.KvDtype.F16, 8, 2, 256, 35, 260, 100, 0.0),   # head_dim 256, G = 4 on a 2-byte cache, window
    (vf.KvDtype.F8, 32, 4, 256, 18, 130, 0, 0.0),     # head_dim 256, G = 8: the group is spread over workgroups so that the Q planes fit
    (vf.KvDtype.F16, 16, 16, 256, 20, 90, 0, 20.0),   # head_dim 256, G = 1: seven key splits
    (vf.KvDtype.F8, 32, 8, 128, 100, 2517, 0, 0.0),   # FP8 rows of 128 elements (V loaded straight into LDS): many two-tile passes, ragged end
    (vf.KvDtype.F8, 16, 4, 128, 33, 6005, 4100, 30.0),  # the same kernel: window that starts inside a tile, soft-cap
    (vf.KvDtype.F8, 40, 8, 128, 7, 1037, 0, 0.0),     # G = 5: a padded head slot beside the rotation of V buffers
    (vf.KvDtype.F8, 32, 8, 128, 45, 1300, 0, 0.0),    # the same kernel, three query blocks, the last one ragged (24 workgroups: launched as one head pair x eight key splits)
    (vf.KvDtype.F8, 16, 2, 128, 96, 700, 650, 0.0),   # G = 8, six query blocks (12 workgroups: one head pair x eight key splits per workgroup), window that starts after some blocks' first tile
    (vf.KvDtype.F8, 8, 4, 128, 130, 37, 0, 20.0),     # G = 2: one head pair (no mirroring), eight key splits dealt 3:2, nine query blocks, soft-cap
    (vf.KvDtype.F8, 32, 8, 128, 256, 0, 0, 0.0),      # from position 0: the first query blocks see fewer tiles than a workgroup has key splits
    # launches of at least 256 workgroups take the form the 512 x 4 608 benchmark runs: two head pairs x four key splits per
    # workgroup, mirrored query blocks, wavefronts 4-7 turned by one head pair, tiles dealt 3:2
    (vf.KvDtype.F8, 128, 32, 128, 125, 300, 0, 0.0),  # G = 4: 8 query blocks x 32 KV heads, ragged last block
    (vf.KvDtype.F8, 128, 32, 128, 125, 700, 519, 30.0),  # the same with a window that starts inside a tile, and the soft-cap
    (vf.KvDtype.F8, 128, 16, 128, 250, 100, 0, 0.0),  # G = 8: two such workgroups per (KV head, query block)
    (vf.KvDtype.F8, 128, 32, 128, 128, 0, 0, 0.0),    # from position 0: query blocks with fewer tiles than key splits
]


@pytest.mark.parametrize("dtype,heads,hkv,d,m,q_start,kv_start,cap", CASES)
def test_batch_matches_oracle(dtype, heads, hkv, d, m, q_start, kv_start, cap):
    r = rng(hash((int(dtype), heads, hkv, d, m, q_start)) % (1 << 31))
    n_kv = q_start + m
    q = fp16_normal(r, (m, heads, d))
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    k, v = encode_np(fill(r, (n_kv, hkv, d)), dtype), encode_np(fill(r, (n_kv, hkv, d)), dtype)
    scale = float(1.0 / np.sqrt(d))
    print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} m={m} q_start={q_start} kv_start={kv_start} cap={cap}",
          flush=True)
    o = gpu_batch(q, k, v, dtype, heads, hkv, d, m, q_start, n_kv, scale, kv_start=kv_start, softcap=cap)
    ref = oracle.attn_batch_ref(q, k, v, int(dtype), m, n_kv, heads, hkv, d, q_start, scale, kv_start=kv_start,
                                softcap=cap)
    assert np.isfinite(o).all()
    err = np.abs(o - ref).max()
    assert err < TOL[dtype], err


@pytest.mark.parametrize("f32_queries", (False, True))
@pytest.mark.parametrize("f16_weights,fp8_scores", ((False, False), (True, False), (False, True), (True, True)))
def test_fp8_head_dim_128_two_head_pairs_per_workgroup_every_option(f32_queries, f16_weights, fp8_scores):
    """The form of the V-through-LDS kernel that a full launch takes (two head pairs x four key splits per workgroup: 256
    workgroups and more), with general f32 queries (remainder pass of the first product) and with each precision option; K
    three times as wide as usual so that the reference maximum moves inside two-tile passes; 125 queries, ragged last block."""
    H, HKV, D, m, q_start = 128, 32, 128, 125, 1100
    r = rng(977 + int(f32_queries))
    n_kv = q_start + m
    q = r.standard_normal((m, H, D)).astype(np.float32) if f32_queries else fp16_normal(r, (m, H, D))
    k = encode_np(fp16_normal(r, (n_kv, HKV, D), 3.0), vf.KvDtype.F8)
    v = encode_np(fp16_normal(r, (n_kv, HKV, D)), vf.KvDtype.F8)
    scale = float(1.0 / np.sqrt(D))
    o = torch.full((m, H, D), float("nan"), device=DEV)
    print(f"case f32_queries={f32_queries} f16_weights={f16_weights} fp8_scores={fp8_scores}", flush=True)
    vf.Forward.run_flash_attn_batch(to_dev(q), to_dev(k.reshape(n_kv, -1)), to_dev(v.reshape(n_kv, -1)), vf.KvDtype.F8, o, H, HKV, D,
                                    m, q_start, n_kv, scale, f16_weights=f16_weights, fp8_scores=fp8_scores)
    torch.cuda.synchronize()
    ref = oracle.attn_batch_ref(q, k, v, int(vf.KvDtype.F8), m, n_kv, H, HKV, D, q_start, scale)
    err = np.abs(to_np(o) - ref).max()
    assert err < (2e-4 if not (f16_weights or fp8_scores) else 6e-3), err


@pytest.mark.parametrize("f32_queries", (False, True))
@pytest.mark.parametrize("f16_weights,fp8_scores", ((False, False), (True, False), (False, True), (True, True)))
def test_fp8_head_dim_128_long_context_with_moving_maximum(f32_queries, f16_weights, fp8_scores):
    """The kernel that loads V tiles straight into LDS (FP8 rows of 128 elements, GQA group >= 2), every form of it: K
    three times as wide as usual, so that the reference maximum moves in the middle of two-tile passes and the loop
    leaves and re-enters its fast path with scores already computed; 3 000 keys, ragged last tile."""
    H, HKV, D, m, q_start = 32, 8, 128, 48, 2953
    r = rng(4242 + int(f32_queries))
    n_kv = q_start + m
    q = r.standard_normal((m, H, D)).astype(np.float32) if f32_queries else fp16_normal(r, (m, H, D))
    k = encode_np(fp16_normal(r, (n_kv, HKV, D), 3.0), vf.KvDtype.F8)
    v = encode_np(fp16_normal(r, (n_kv, HKV, D)), vf.KvDtype.F8)
    scale = float(1.0 / np.sqrt(D))
    o = torch.full((m, H, D), float("nan"), device=DEV)
    vf.Forward.run_flash_attn_batch(to_dev(q), to_dev(k.reshape(n_kv, -1)), to_dev(v.reshape(n_kv, -1)), vf.KvDtype.F8, o, H, HKV, D,
                                    m, q_start, n_kv, scale, f16_weights=f16_weights, fp8_scores=fp8_scores)
    torch.cuda.synchronize()
    ref = oracle.attn_batch_ref(q, k, v, int(vf.KvDtype.F8), m, n_kv, H, HKV, D, q_start, scale)
    err = np.abs(to_np(o) - ref).max()
    # default: f32-level; the options: weights to 11 bits (2^-11 max|v|, |v| <= 5 here) and scores through the FP8 instruction
    assert err < (2e-4 if not (f16_weights or fp8_scores) else 6e-3), err


@pytest.mark.parametrize("dtype", (vf.KvDtype.F8, vf.KvDtype.F16))
def test_batch_with_f32_queries_keeps_f32_accuracy(dtype):
    # Q values that are not representable in f16: the kernel must not lose them (hi + lo split)
    heads, hkv, d, m, q_start = 16, 4, 128, 40, 500
    r = rng(91)
    n_kv = q_start + m
    q = (r.standard_normal((m, heads, d)) * 3).astype(np.float32)
    k = encode_np(fp16_normal(r, (n_kv, hkv, d)), dtype)
    v = encode_np(fp16_normal(r, (n_kv, hkv, d)), dtype)
    scale = float(1.0 / np.sqrt(d))
    o = gpu_batch(q, k, v, dtype, heads, hkv, d, m, q_start, n_kv, scale)
    ref = oracle.attn_batch_ref(q, k, v, int(dtype), m, n_kv, heads, hkv, d, q_start, scale)
    assert np.abs(o - ref).max() < 1e-3


@pytest.mark.parametrize("dtype,heads,hkv,d", [(vf.KvDtype.F8, 32, 8, 128), (vf.KvDtype.F16, 32, 8, 128), (vf.KvDtype.F8, 16, 8, 256),
                                                (vf.KvDtype.F16, 8, 2, 512), (vf.KvDtype.F8, 8, 4, 64)])
def test_f16_queries_option_is_the_call_on_queries_rounded_to_f16(dtype, heads, hkv, d):
    """VFKV_PREFILL_F16_QUERIES: general f32 queries take the path of f16-representable ones.  Bit-identical to rounding the
    queries first; against the oracle on the unrounded queries a score is off by at most 2^-12 of the sum of its |k q|
    products times scale, inside the path's tolerance on these inputs."""
    m, q_start = 40, 700
    r = rng(77)
    n_kv = q_start + m
    q = (r.standard_normal((m, heads, d)) * 2).astype(np.float32)
    k = encode_np(fp16_normal(r, (n_kv, hkv, d)), dtype)
    v = encode_np(fp16_normal(r, (n_kv, hkv, d)), dtype)
    scale = float(1.0 / np.sqrt(d))

    def run(qq, **kw):
        o = torch.full((m, heads, d), float("nan"), device=DEV)
        vf.Forward.run_flash_attn_batch(to_dev(qq), to_dev(k.reshape(n_kv, -1)), to_dev(v.reshape(n_kv, -1)), dtype, o, heads, hkv, d,
                                        m, q_start, n_kv, scale, **kw)
        torch.cuda.synchronize()
        return to_np(o)

    o_opt = run(q, f16_queries=True)
    o_cast = run(q.astype(np.float16).astype(np.float32))
    assert np.array_equal(o_opt, o_cast)
    ref = oracle.attn_batch_ref(q, k, v, int(dtype), m, n_kv, heads, hkv, d, q_start, scale)
    assert np.abs(o_opt - ref).max() < 2e-3             # 1.0e-3 measured on the first case (queries of standard deviation 2)
    assert np.abs(run(q) - ref).max() < (6e-5 if dtype == vf.KvDtype.F8 and d == 128 else 2e-5)   # the default keeps the remainder (FP8 rows of 128 elements: as E4M3 codes, 15 bits of q in all; 2.1e-5 measured)


def test_config5_chunk_append_then_prefill_fp8_one_layer():
    # benchmark configuration 5, one of its 32 layers: FP8 cache filled to 4096, append 512 tokens, then
    # 512 causal queries over 4608 keys (32/8/128).  The oracle is run on a sample of query rows.
    heads, hkv, d, base, m = 32, 8, 128, 4096, 512
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, base + m, dtype=vf.KvDtype.F8))
    fwd = vf.Forward(cache, heads)
    r = rng(61)
    hist_k, hist_v = fp16_normal(r, (base, hkv * d)), fp16_normal(r, (base, hkv * d))
    new_k, new_v = fp16_normal(r, (m, hkv * d)), fp16_normal(r, (m, hkv * d))
    q = fp16_normal(r, (m, heads, d))
    fwd.b_step_kv_write(0, 0, base, to_dev(hist_k), to_dev(hist_v))
    fwd.b_step_kv_write(0, base, m, to_dev(new_k), to_dev(new_v))
    o = torch.full((m, heads, d), float("nan"), device=DEV)
    fwd.b_step_attention(0, base, m, to_dev(q), o)
    torch.cuda.synchronize()
    o = to_np(o)
    assert np.isfinite(o).all()
    ke = encode_np(np.concatenate([hist_k, new_k]), vf.KvDtype.F8).reshape(-1, hkv, d)
    ve = encode_np(np.concatenate([hist_v, new_v]), vf.KvDtype.F8).reshape(-1, hkv, d)
    from gpu_util import read_device
    assert (read_device(cache.k_ptr, ke.size) == ke.ravel()).all()          # appended bytes bit-exact
    for i in (0, 1, 63, 64, 255, 400, 511):
        ref = oracle.attn_decode_ref(q[i], ke, ve, oracle.F8, heads, hkv, d, base + i + 1, fwd.attn_scale)
        err = np.abs(o[i] - ref).max()
        assert err < 5e-3, (i, err)
    cache.destroy()


def test_window_uses_the_last_querys_lower_bound():
    # executor/attention.rs:2215-2219: kv_start = base + m - window for every row of the batch
    heads, hkv, d, base, m, window = 8, 2, 128, 300, 40, 128
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, base + m, dtype=vf.KvDtype.F16))
    fwd = vf.Forward(cache, heads)
    r = rng(71)
    k, v = fp16_normal(r, (base + m, hkv * d)), fp16_normal(r, (base + m, hkv * d))
    q = fp16_normal(r, (m, heads, d))
    fwd.b_step_kv_write(0, 0, base + m, to_dev(k), to_dev(v))
    o = torch.full((m, heads, d), float("nan"), device=DEV)
    fwd.b_step_attention(0, base, m, to_dev(q), o, kv_start_window=window)
    torch.cuda.synchronize()
    kv_start = oracle.kv_start_batch(base, m, window)
    assert kv_start == base + m - window
    ke, ve = (encode_np(x, vf.KvDtype.F16).reshape(-1, hkv, d) for x in (k, v))
    ref = oracle.attn_batch_ref(q, ke, ve, oracle.F16, m, base + m, heads, hkv, d, base, fwd.attn_scale,
                                kv_start=kv_start)
    assert np.abs(to_np(o) - ref).max() < TIGHT
    cache.destroy()


@pytest.mark.parametrize("dtype", (vf.KvDtype.F16, vf.KvDtype.F8, vf.KvDtype.F32))
@pytest.mark.parametrize("shape", ("ascending", "descending", "steps"))
def test_scores_that_drift_past_the_running_maximum(dtype, shape):
    # the kernel keeps a reference maximum that is allowed to lag behind the true one; scores that climb slowly, fall, or
    # jump by hundreds between tiles must come out as the oracle computes them
    heads, hkv, d, m, q_start = 8, 2, 128, 40, 700
    n_kv = q_start + m
    r = rng({"ascending": 1, "descending": 2, "steps": 3}[shape] + int(dtype))
    u = r.standard_normal(d).astype(np.float32)
    u /= np.linalg.norm(u)
    t = np.arange(n_kv, dtype=np.float32)
    if shape == "ascending":
        level = 70.0 * t / n_kv                               # +3 per tile of 32 keys: below the slack tile after tile
    elif shape == "descending":
        level = 70.0 * (1.0 - t / n_kv)
    else:
        level = 40.0 * ((t // 96) % 3)                        # plateaus 0 / 40 / 80, up and down
    k = (level[:, None, None] * u[None, None, :] * np.ones((1, hkv, 1), np.float32)).astype(np.float32)
    k += 0.05 * r.standard_normal(k.shape).astype(np.float32)
    q = np.broadcast_to(u * np.float32(np.sqrt(d)), (m, heads, d)).astype(np.float32).copy()
    q += 0.05 * r.standard_normal(q.shape).astype(np.float32)
    v = fp16_normal(r, (n_kv, hkv, d))
    ke, ve = encode_np(k, dtype), encode_np(v, dtype)
    scale = float(1.0 / np.sqrt(d))
    print(f"case dtype={dtype.label()} shape={shape}", flush=True)
    o = gpu_batch(q, ke, ve, dtype, heads, hkv, d, m, q_start, n_kv, scale)
    ref = oracle.attn_batch_ref(q, ke, ve, int(dtype), m, n_kv, heads, hkv, d, q_start, scale)
    assert np.isfinite(o).all()
    assert np.abs(o - ref).max() < 1e-4


@pytest.mark.parametrize("dtype,heads,hkv,d,m,base,window,cap", (
    (vf.KvDtype.F8, 32, 8, 128, 64, 4096, 0, 0.0),       # the suffix of a request over its reused prefix
    (vf.KvDtype.F16, 32, 8, 128, 20, 9000, 0, 0.0),      # one partly filled query block, four-heads-per-wavefront form
    (vf.KvDtype.F8, 16, 8, 256, 37, 3000, 2048, 30.0),   # window and soft-cap: chunks start at the window
    (vf.KvDtype.F8, 8, 2, 512, 16, 2500, 0, 0.0),        # head_dim 512: output slices and key chunks together
    (vf.KvDtype.F16, 8, 1, 512, 21, 3624, 3000, 0.0),    # head_dim 512: the two wavefronts of a head swap score halves behind a
                                                         # barrier per tile, so every wavefront also walks (masked) padding tiles
                                                         # past the end of its key chunk
    (vf.KvDtype.F16, 8, 8, 512, 20, 2001, 0, 0.0),       # head_dim 512, one head per KV head: two key splits of unequal length
    (vf.KvDtype.F16, 28, 4, 128, 50, 1500, 0, 0.0),      # G = 7
    (vf.KvDtype.F8, 32, 8, 128, 512, 4096, 0, 0.0),      # a full chunk: plenty of workgroups, the plain path is taken
    (vf.KvDtype.F32, 8, 2, 128, 16, 2000, 0, 0.0),       # F32 cache: no key chunks, same result
    (vf.KvDtype.F16, 32, 32, 96, 24, 5000, 0, 0.0),      # heads of 96 elements on the kernel for 128: partials with their real stride
    (vf.KvDtype.F8, 8, 2, 192, 16, 3000, 1000, 20.0),    # heads of 192 on the kernel for 256, window, soft-cap
    (vf.KvDtype.F8, 8, 8, 128, 40, 6000, 0, 0.0),        # groups of one head: two query blocks per wavefront, partials per query
))
def test_prefill_with_workspace_matches_plain_call_and_oracle(dtype, heads, hkv, d, m, base, window, cap):
    # vfkv_prefill_attention_ws cuts the keys into chunks over workgroups and merges the partials
    r = rng(base + m + d)
    n = base + m
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, n, dtype=dtype))
    fwd = vf.Forward(cache, heads)
    fwd.workspace = vf.Workspace(heads, d, 32768)            # sized for a serving context, as the decode path has it
    fill = outlier_normal if dtype == vf.KvDtype.F8 else fp16_normal
    k, v = fill(r, (n, hkv, d)), fill(r, (n, hkv, d))
    fwd.b_step_kv_write(0, 0, n, to_dev(k), to_dev(v))
    q = to_dev(r.standard_normal((m, heads, d)).astype(np.float32))
    a = torch.full((m, heads, d), float("nan"), device=DEV)
    b = torch.full((m, heads, d), float("nan"), device=DEV)
    print(f"case dtype={dtype.label()} H={heads} Hkv={hkv} D={d} m={m} base={base} window={window} cap={cap}", flush=True)
    for rep in range(2):                                     # twice: the workspace is reused
        fwd.b_step_attention(0, base, m, q, a, kv_start_window=window, softcap=cap, use_workspace=True)
    fwd.b_step_attention(0, base, m, q, b, kv_start_window=window, softcap=cap)
    torch.cuda.synchronize()
    assert np.isfinite(to_np(a)).all()
    assert np.abs(to_np(a) - to_np(b)).max() < 2e-6 * max(1.0, float(np.abs(to_np(b)).max())) + 2e-5   # f32 rounding of another summation order
    kv_start = oracle.kv_start_batch(base, m, window)
    ref = oracle.attn_batch_ref(to_np(q), encode_np(k, dtype), encode_np(v, dtype), int(dtype), m, n, heads, hkv, d, base,
                                float(1.0 / np.sqrt(d)), kv_start=kv_start, softcap=cap)
    assert np.abs(to_np(a) - ref).max() < TOL[dtype]
    cache.destroy()


def test_prefill_with_a_small_workspace_falls_back():
    heads, hkv, d, m, base = 32, 8, 128, 64, 4096
    r = rng(5)
    cache = vf.KvCache(vf.KvCacheConfig(1, hkv, d, base + m, dtype=vf.KvDtype.F8))
    fwd = vf.Forward(cache, heads)
    fwd.workspace = vf.Workspace(heads, d, 64)               # one tile per head: no room for partials of 64 x 32 rows
    k = fp16_normal(r, (base + m, hkv, d))
    fwd.b_step_kv_write(0, 0, base + m, to_dev(k), to_dev(k))
    q = to_dev(fp16_normal(r, (m, heads, d)))
    a, b = torch.empty((m, heads, d), device=DEV), torch.empty((m, heads, d), device=DEV)
    fwd.b_step_attention(0, base, m, q, a, use_workspace=True)
    fwd.b_step_attention(0, base, m, q, b)
    torch.cuda.synchronize()
    assert (to_np(a) == to_np(b)).all()
    cache.destroy()


@pytest.mark.parametrize("dtype,heads,hkv,vscale", [(vf.KvDtype.F8, 32, 8, 1.0), (vf.KvDtype.F16, 32, 8, 1.0),
                                                    (vf.KvDtype.F8, 32, 8, 8.0), (vf.KvDtype.F16, 24, 8, 8.0)])
def test_f16_weights_option_stays_inside_its_stated_bound(dtype, heads, hkv, vscale):
    # VFKV_PREFILL_F16_WEIGHTS: one product with the f16 rounding of the softmax weights.  Every weight is off by at most
    # 2^-11 relative, so every output element by at most 2^-11 * max|v| (plus the f32 rounding of the default path); on
    # N(0,1) inputs that is far inside this path's tolerance.  Without the option the call is the default path, bit for bit.
    d, base, m = 128, 1536, 96
    n_kv = base + m
    r = rng(640 + int(vscale))
    k = fp16_normal(r, (n_kv, hkv * d))
    v = fp16_normal(r, (n_kv, hkv * d), vscale)
    q = fp16_normal(r, (m, heads, d))
    ke, ve = encode_np(k, dtype), encode_np(v, dtype)
    scale = 1.0 / np.sqrt(d)
    o_def = gpu_batch(q, ke, ve, dtype, heads, hkv, d, m, base, n_kv, scale)
    o_opt = torch.full((m, heads, d), float("nan"), device=DEV, dtype=torch.float32)
    vf.Forward.run_flash_attn_batch(to_dev(q), to_dev(ke), to_dev(ve), dtype, o_opt, heads, hkv, d, m, base, n_kv, scale,
                                    f16_weights=True)
    torch.cuda.synchronize()
    o_opt = to_np(o_opt)
    ref = oracle.attn_batch_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), int(dtype), m, n_kv, heads, hkv, d, base, scale)
    vmax = float(np.abs(v).max())                            # |decoded v| <= |v| * (1 + 2^-4) for E4M3, equal for F16
    vmax *= 1.0625 if dtype == vf.KvDtype.F8 else 1.0
    assert np.abs(o_def - ref).max() < TIGHT
    err = np.abs(o_opt - ref).max()
    assert err <= 2.0 ** -11 * vmax + 1e-5, (err, vmax)
    if vscale == 1.0:
        assert err < TIGHT                                   # 4.5e-5 measured on the benchmark's distribution
    assert not np.array_equal(o_opt, o_def)                  # the option really took the other path


@pytest.mark.parametrize("f16_weights", [False, True])
def test_fp8_scores_option_on_the_benchmark_distribution(f16_weights):
    # VFKV_PREFILL_FP8_SCORES: K.Q^T on the FP8 matrix instruction (K rows as stored, Q as three E4M3 terms).  The terms are
    # exact for f16-representable queries; what remains is the instruction's own summation (about 15 bits over the 128
    # products of a score).  On the benchmark's N(0,1) inputs the output stays two orders of magnitude inside the 5e-3 bound
    # of this path, also with queries far from 1 in magnitude (the terms carry a block exponent) and together with the
    # f16-weights option.
    heads, hkv, d, base, m = 32, 8, 128, 1536, 96
    n_kv = base + m
    scale = 1.0 / np.sqrt(d)
    for qscale in (1.0, 300.0, 1e-3):
        r = rng(700)
        k, v = fp16_normal(r, (n_kv, hkv * d)), fp16_normal(r, (n_kv, hkv * d))
        q = fp16_normal(r, (m, heads, d), qscale)
        ke, ve = encode_np(k, vf.KvDtype.F8), encode_np(v, vf.KvDtype.F8)
        o = torch.full((m, heads, d), float("nan"), device=DEV, dtype=torch.float32)
        vf.Forward.run_flash_attn_batch(to_dev(q), to_dev(ke), to_dev(ve), vf.KvDtype.F8, o, heads, hkv, d, m, base, n_kv,
                                        scale / qscale, f16_weights=f16_weights, fp8_scores=True)
        torch.cuda.synchronize()
        ref = oracle.attn_batch_ref(q, ke.reshape(-1, hkv, d), ve.reshape(-1, hkv, d), oracle.F8, m, n_kv, heads, hkv, d, base,
                                    scale / qscale)
        err = np.abs(to_np(o) - ref).max()
        assert err < (TIGHT if f16_weights else 5e-5), (qscale, err)
