"""Pins the oracle's E4M3FN / f16 conversions and the append routines (CPU only)."""
import os

import numpy as np
import pytest
import torch

import oracle


@pytest.fixture(scope="module")
def table(golden_dir):
    return np.load(os.path.join(golden_dir, "e4m3_decode_table.npy"))


def test_reference_known_values():
    # src/backend/vulkan/fp8_ext.rs:217-263 -- the reference's own unit-test vectors
    L = oracle.lib()
    assert L.vfo_f32_to_e4m3(0.0) == 0x00 and L.vfo_f32_to_e4m3(-0.0) == 0x80
    assert L.vfo_f32_to_e4m3(1.0) == 0x38 and L.vfo_f32_to_e4m3(448.0) == 0x7E
    assert L.vfo_f32_to_e4m3(1000.0) == 0x7E
    for code, val in ((0x38, 1.0), (0x40, 2.0), (0x48, 4.0), (0xB8, -1.0), (0x30, 0.5), (0x3C, 1.5),
                      (0x7E, 448.0), (0x00, 0.0)):
        assert L.vfo_e4m3_to_f32(code) == val
    assert np.signbit(np.float32(L.vfo_e4m3_to_f32(0x80)))
    assert np.isnan(L.vfo_e4m3_to_f32(0x7F)) and np.isnan(L.vfo_e4m3_to_f32(0xFF))


def test_decode_all_codes_vs_library(table):
    got = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8))
    nan = np.isnan(table)
    assert nan.sum() == 2 and np.isnan(got[nan]).all()
    assert (got[~nan].view(np.uint32) == table[~nan].view(np.uint32)).all()  # incl. the sign of -0


def test_decode_closed_form():
    codes = np.arange(256, dtype=np.uint8)
    s = np.where(codes & 0x80, -1.0, 1.0)
    e = ((codes >> 3) & 0xF).astype(np.int32)
    m = (codes & 7).astype(np.float64)
    val = np.where(e == 0, s * m / 8 * 2.0 ** -6, s * (1 + m / 8) * np.exp2(e - 7.0))
    got = oracle.e4m3_to_f32(codes).astype(np.float64)
    ok = ~((e == 15) & (m == 7))
    assert (got[ok] == val[ok]).all()


def test_encode_golden_vectors(golden_dir):
    z = np.load(os.path.join(golden_dir, "e4m3_encode_vectors.npz"))
    x = z["bits"].view(np.float32)
    got = oracle.f32_to_e4m3(x)
    bad = np.nonzero(got != z["expected"])[0]
    assert bad.size == 0, [(hex(z["bits"][i]), hex(got[i]), hex(z["expected"][i])) for i in bad[:8]]


def test_encode_round_trip_all_codes(table):
    codes = np.arange(256, dtype=np.uint8)
    keep = ~np.isnan(table)
    assert (oracle.f32_to_e4m3(table[keep]) == codes[keep]).all()


def test_encode_ties_to_even(table):
    pos = np.sort(table[np.isfinite(table) & ~np.signbit(table)])
    codes = oracle.f32_to_e4m3(pos)
    mid = ((pos[:-1].astype(np.float64) + pos[1:]) / 2).astype(np.float32)
    got = oracle.f32_to_e4m3(mid)
    even = np.where(codes[:-1] % 2 == 0, codes[:-1], codes[1:])
    assert (got == even).all()
    assert (oracle.f32_to_e4m3(np.nextafter(mid, np.float32(np.inf))) == codes[1:]).all()
    assert (oracle.f32_to_e4m3(np.nextafter(mid, np.float32(-np.inf))) == codes[:-1]).all()


def _independent_encode(x, table):
    """ldexp / rint formulation: quantum 2^(max(e,-6)-3), np.rint is ties-to-even."""
    x = x.astype(np.float64)
    ax = np.abs(x)
    e = np.floor(np.log2(np.where(ax > 0, ax, 1.0)))
    e = np.maximum(e, -6.0)
    quantum = np.exp2(e - 3.0)
    r = np.rint(ax / quantum) * quantum
    r = np.minimum(r, 448.0)
    lut = {float(v): c for c, v in enumerate(table[:128]) if np.isfinite(v)}
    out = np.array([lut[float(v)] for v in r], dtype=np.uint8)
    return out | np.where(np.signbit(x), 0x80, 0).astype(np.uint8)


def test_encode_vs_independent_formulation_upper_half_patterns(table):
    # every f32 whose low 16 bits are zero (all exponents, both signs), plus random full patterns
    rng = np.random.default_rng(7)
    bits = np.concatenate([(np.arange(1 << 16, dtype=np.uint32) << 16),
                           rng.integers(0, 1 << 32, size=200_000, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    fin = np.isfinite(x)
    got = oracle.f32_to_e4m3(x)
    assert (got[np.isnan(x)] == 0x7F).all()
    inf = np.isinf(x)
    assert (got[inf] == np.where(np.signbit(x[inf]), 0xFE, 0x7E)).all()
    exp = _independent_encode(x[fin], table)
    assert (got[fin] == exp).all()


def test_encode_vs_torch_cast_in_range():
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(300_000) * 0.5, rng.standard_normal(100_000) * 60,
                        rng.uniform(-448, 448, 100_000), rng.standard_normal(100_000) * 1e-2]).astype(np.float32)
    x = x[np.abs(x) < 448]
    exp = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert (oracle.f32_to_e4m3(x) == exp).all()


def test_f16_vs_numpy_all_halves_and_random():
    h = np.arange(1 << 16, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(h)
    ref = h.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert (f[~nan].view(np.uint32) == ref[~nan].view(np.uint32)).all() and np.isnan(f[nan]).all()
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 1 << 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    x = np.concatenate([bits.view(np.float32), (rng.standard_normal(1 << 18) * 100).astype(np.float32),
                        np.array([65504.0, 65519.9, 65520.0, 65536.0, 1e-8, 5.96e-8, 2.98e-8, 2.9803e-8],
                                 dtype=np.float32)])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        exp = x.astype(np.float16).view(np.uint16)
    assert (oracle.f32_to_f16_bits(x) == exp).all()


def test_kv_store_fp8_layout_and_tail():
    rng = np.random.default_rng(5)
    src = (rng.standard_normal(1031) * 3).astype(np.float32)
    dst = np.full(4096, 0xAA, dtype=np.uint8)
    assert oracle.kv_store_fp8(src, dst, 1031, 1024) == 0
    assert (dst[:1024] == 0xAA).all()
    assert (dst[1024:1024 + 1031] == oracle.f32_to_e4m3(src)).all()
    assert (dst[1024 + 1031:1024 + 1032] == 0).all()        # tail of the last word is zero-padded
    assert (dst[1024 + 1032:] == 0xAA).all()
    assert oracle.kv_store_fp8(src, dst, 4, 1022) != 0       # runs.rs:2448-2453: offset must be 4-aligned


def test_kv_copy_fp16_layout_and_tail():
    rng = np.random.default_rng(6)
    src = rng.standard_normal(515).astype(np.float32)
    dst = np.full(4096, 0xAA, dtype=np.uint8)
    assert oracle.kv_copy_fp16(src, dst, 515, 512) == 0
    got = dst[512:512 + 2 * 516].view(np.uint16)
    assert (got[:515] == src.astype(np.float16).view(np.uint16)).all() and got[515] == 0
    assert (dst[:512] == 0xAA).all() and (dst[512 + 2 * 516:] == 0xAA).all()
    assert oracle.kv_copy_fp16(src, dst, 2, 514) != 0


def test_kv_fp8_to_f16_vs_library():
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.kv_fp8_to_f16(codes)
    exp = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float16).view(torch.uint16).numpy()
    nan = (codes & 0x7F) == 0x7F
    assert (got[~nan] == exp[~nan]).all()
    assert np.isnan(got[nan].view(np.float16)).all()
    # exactness: every finite code survives fp8 -> f16 -> f32 unchanged
    assert (oracle.f16_bits_to_f32(got[~nan]) == oracle.e4m3_to_f32(codes[~nan])).all()
