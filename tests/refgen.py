"""Closed-form input generators used by the reference's own attention tests, restated so the
same inputs can be rebuilt anywhere (they are formulas, not data files).

* decode:  tests/correctness.rs:2806-2817  (q = sin(0.001 i), k = cos((t+1)*0.01 + 0.001 d),
  v = sin(0.013 t + 0.7 kvh + 0.0007 d)), H/Hkv/D = 32/8/128.
* batch:   tests/correctness.rs:3093-3111.
* xorshift PRNG in [-1, 1): tests/flash_attn_tiled_ref.rs:189-203.
All arithmetic inside sin/cos is float32, as in the reference (f32 casts of the indices).
"""
import numpy as np

H, HKV, D = 32, 8, 128
f = np.float32


def decode_inputs(seq, n_heads=H, n_kv_heads=HKV, head_dim=D):
    i = np.arange(n_heads * head_dim, dtype=f)
    q = np.sin(i * f(0.001)).reshape(n_heads, head_dim)
    t = np.arange(seq, dtype=f)[:, None, None]
    kvh = np.arange(n_kv_heads, dtype=f)[None, :, None]
    d = np.arange(head_dim, dtype=f)[None, None, :]
    k = np.cos((t + f(1.0)) * f(0.01) + d * f(0.001)) + f(0.0) * kvh
    v = np.sin(t * f(0.013) + kvh * f(0.7) + d * f(0.0007))
    return q.astype(f), np.ascontiguousarray(k.astype(f)), np.ascontiguousarray(v.astype(f))


def batch_inputs(m, q_start, n_heads=H, n_kv_heads=HKV, head_dim=D):
    n_kv = q_start + m
    qi = np.arange(m, dtype=f)[:, None, None]
    hh = np.arange(n_heads, dtype=f)[None, :, None]
    d = np.arange(head_dim, dtype=f)[None, None, :]
    q = np.sin(qi * f(0.017) + hh * f(0.011) + d * f(0.003))
    t = np.arange(n_kv, dtype=f)[:, None, None]
    kvh = np.arange(n_kv_heads, dtype=f)[None, :, None]
    k = np.cos((t + f(1.0)) * f(0.01) + d * f(0.001) + kvh * f(0.7))
    v = np.sin(t * f(0.013) + kvh * f(0.5) + d * f(0.0007))
    return (np.ascontiguousarray(q.astype(f)), np.ascontiguousarray(k.astype(f)),
            np.ascontiguousarray(v.astype(f)))


def xorshift_floats(n, seed):
    mask = (1 << 64) - 1
    state = (seed * 0x9E3779B97F4A7C15 + 1) & mask
    out = np.empty(n, dtype=f)
    for i in range(n):
        state ^= (state << 13) & mask
        state ^= state >> 7
        state ^= (state << 17) & mask
        bits = state & 0x00FFFFFF
        out[i] = f(f(bits) / f(1 << 24)) * f(2.0) - f(1.0)
    return out


# rows of the batch cases whose float64 outputs are kept as golden data
BATCH_CASES = ((1, 0), (4, 0), (16, 0), (64, 0), (200, 0), (4, 60))
DECODE_SEQS = (1, 64, 200, 2048)


def golden_rows(m):
    if m <= 16:
        return list(range(m))
    if m == 64:
        return [0, 1, 31, 62, 63]
    return [0, 63, 64, 65, 127, 128, m - 1]
