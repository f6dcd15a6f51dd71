"""Writes the golden fixtures under tests/golden/ from sources that are independent of the oracle:

* ``e4m3_decode_table.npy``   -- f32 value of every E4M3FN code, from torch.float8_e4m3fn.
* ``e4m3_encode_vectors.npz`` -- f32 bit patterns and the byte each must encode to.  Expected bytes
  for finite |x| < 448 come from torch's float8_e4m3fn cast (round-to-nearest-even, a library
  routine); saturation / Inf / NaN rows follow the reference's stated rule
  (src/backend/vulkan/fp8_ext.rs:126-142: NaN -> 0x7F, |x| >= 448 incl. Inf -> sign|0x7E) and the
  reference's own unit-test vectors (fp8_ext.rs:225-247) are included verbatim as data.
* ``attn_cases.npz``          -- outputs of the reference's closed-form attention fixtures
  (tests/correctness.rs:2806-2817 decode, :3093-3111 batch; inputs rebuilt by tests/refgen.py),
  computed here in float64 with numpy + scipy.special.softmax (no oracle code involved); for the
  larger batches only the query rows listed by refgen.golden_rows are kept.

Run:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import scipy.special
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))  # tests/refgen.py: the closed-form input generators


def decode_table():
    codes = torch.arange(256, dtype=torch.uint8)
    vals = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    np.save(os.path.join(HERE, "e4m3_decode_table.npy"), vals)
    return vals


def encode_vectors(table):
    rng = np.random.default_rng(20240607)
    finite = table[np.isfinite(table)]
    pos = np.sort(np.unique(np.abs(finite)))
    xs = [pos, -pos]
    # midpoints between adjacent representable magnitudes (exact in f32) and their f32 neighbours
    mid = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    for m in (mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))):
        xs += [m, -m]
    # every power of two across the f32 range that matters, and its neighbours
    p2 = np.ldexp(np.float32(1.0), np.arange(-30, 12)).astype(np.float32)
    xs += [p2, -p2, np.nextafter(p2, np.float32(0)), np.nextafter(p2, np.float32(np.inf))]
    # benchmark-style data: N(0,1)*0.5 with a +-40 outlier tail, and N(0,1) cast to fp16
    xs.append((rng.standard_normal(1500) * 0.5).astype(np.float32))
    xs.append(rng.standard_normal(800).astype(np.float16).astype(np.float32))
    xs.append(np.array([40.0, -40.0, 447.9, 448.0, -448.0, 463.9, 464.0, 465.0, 1000.0, -1000.0,
                        3.0e38, -3.0e38, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -10 * 1.0000001,
                        1.0e-30, -1.0e-30, 1.0e-45, 0.0, -0.0], dtype=np.float32))
    x = np.concatenate(xs).astype(np.float32)
    inb = np.abs(x) < np.float32(448.0)
    exp = np.zeros(x.shape, dtype=np.uint8)
    exp[inb] = torch.from_numpy(x[inb]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    sat = ~inb
    exp[sat] = np.where(np.signbit(x[sat]), 0xFE, 0x7E).astype(np.uint8)
    # special rows (rule-based): +-Inf saturate, NaN -> 0x7F regardless of sign
    special_bits = np.array([0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00000, 0x7F800001, 0xFFFFFFFF],
                            dtype=np.uint32)
    special_exp = np.array([0x7E, 0xFE, 0x7F, 0x7F, 0x7F, 0x7F], dtype=np.uint8)
    # reference unit-test vectors, fp8_ext.rs:225-247
    ref_x = np.array([0.0, -0.0, 1.0, 448.0, 1000.0], dtype=np.float32)
    ref_exp = np.array([0x00, 0x80, 0x38, 0x7E, 0x7E], dtype=np.uint8)
    bits = np.concatenate([x.view(np.uint32), special_bits, ref_x.view(np.uint32)])
    expected = np.concatenate([exp, special_exp, ref_exp])
    np.savez_compressed(os.path.join(HERE, "e4m3_encode_vectors.npz"), bits=bits, expected=expected)
    return bits.size


def _gqa_attention_f64(q, k, v, g, scale, lens):
    """q [m,H,D], k/v [T,Hkv,D] float64; lens[i] = number of visible keys of query i."""
    m, H, D = q.shape
    out = np.zeros((m, H, D))
    for i in range(m):
        n = lens[i]
        for h in range(H):
            kvh = h // g
            s = (k[:n, kvh, :] @ q[i, h, :]) * scale
            w = scipy.special.softmax(s)
            out[i, h, :] = w @ v[:n, kvh, :]
    return out


def attention_cases():
    from refgen import BATCH_CASES, DECODE_SEQS, H, HKV, D, batch_inputs, decode_inputs, golden_rows
    g = H // HKV
    scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
    out = {}
    for seq in DECODE_SEQS:
        q, k, v = decode_inputs(seq)
        o = _gqa_attention_f64(q[None].astype(np.float64), k.astype(np.float64), v.astype(np.float64), g,
                               scale, [seq])
        out[f"decode_seq{seq}_out"] = o[0].astype(np.float32)
    for m, q_start in BATCH_CASES:
        q, k, v = batch_inputs(m, q_start)
        rows = golden_rows(m)
        lens = [min(q_start + i + 1, q_start + m) for i in rows]
        o = _gqa_attention_f64(q[rows].astype(np.float64), k.astype(np.float64), v.astype(np.float64), g,
                               scale, lens)
        out[f"batch_m{m}_qs{q_start}_out"] = o.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "attn_cases.npz"), **out)
    return sorted(out)


if __name__ == "__main__":
    tab = decode_table()
    print("decode table:", tab.shape)
    print("encode vectors:", encode_vectors(tab))
    print("attention cases:", attention_cases())
