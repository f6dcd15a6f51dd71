"""Pins the oracle's RMS-norm * weight + RoPE (the step in front of the KV append) without running the reference:
the reference's own generator case and CPU formula with its thresholds (tests/correctness.rs:799-884), an
independent numpy formulation (complex rotation, f64), and what the mathematics fixes (rotations preserve pair
norms, position 0 is the identity, positions add, the norm is scale-invariant)."""
import numpy as np
import pytest

import oracle

HEAD_DIM = 128
FREQ_BASE = 1_000_000.0


def reference_case(pos):
    # rope_neox_case, tests/correctness.rs:819-845: input ramp, f32 powi / cos / sin, split-half rotation
    x = (np.float32(0.1) + np.float32(3.4) * np.arange(HEAD_DIM, dtype=np.float32) / np.float32(HEAD_DIM - 1))
    half = HEAD_DIM // 2
    theta_scale = np.float32(1.0) / np.float32(FREQ_BASE) ** np.float32(2.0 / HEAD_DIM)
    cpu = np.zeros(HEAD_DIM, np.float32)
    for i in range(half):
        freq = np.float32(1.0)
        for _ in range(i):                      # powi by repeated f32 multiplication
            freq = np.float32(freq * theta_scale)
        theta = np.float32(pos) * freq
        c, s = np.cos(theta, dtype=np.float32), np.sin(theta, dtype=np.float32)
        cpu[i] = x[i] * c - x[i + half] * s
        cpu[i + half] = x[i] * s + x[i + half] * c
    return x.astype(np.float32), theta_scale, cpu


@pytest.mark.parametrize("pos,threshold", ((0, 1e-5), (100, 1e-4), (4096, 5e-4)))
def test_reference_rope_neox_cases(pos, threshold):
    x, theta_scale, cpu = reference_case(pos)
    got = oracle.rms_norm_rope(x.reshape(1, 1, HEAD_DIM), [pos], HEAD_DIM, HEAD_DIM, theta_scale)[0, 0]
    assert np.abs(got - cpu).max() < threshold          # the reference's own bar for its GPU
    # the two f32 evaluations of theta_scale^i (powi by multiplication there, pow here) may differ by a few ulp of theta
    assert np.abs(got - cpu).max() < 4.0 * (1e-6 + pos * 2.0 ** -22)
    if pos == 0:
        assert (got == x).all()


def numpy_rope(x, pos, n_dims, theta_scale, mode, ff=None, freq_scale=1.0, attn_factor=1.0):
    """Independent formulation: each rotary pair is a complex number multiplied by exp(i theta), in f64.  theta is the f32
    number the shader forms (pos * pow(theta_scale, p) / ff * freq_scale), so that both sides rotate by the same angle."""
    m, heads, d = x.shape
    half = n_dims // 2
    p = np.arange(half, dtype=np.float32)
    out = x.astype(np.float64).copy()
    for t in range(m):
        theta_base = np.float32(pos[t]) * np.power(np.float32(theta_scale), p, dtype=np.float32)
        theta = np.float32(freq_scale) * (theta_base / (np.ones(half, np.float32) if ff is None else ff.astype(np.float32)))
        rot = np.exp(1j * theta.astype(np.float64)) * attn_factor
        ia, ib = (np.arange(half), np.arange(half) + half) if mode == oracle.ROPE_NEOX else (2 * np.arange(half), 2 * np.arange(half) + 1)
        z = (x[t, :, ia].astype(np.float64) + 1j * x[t, :, ib].astype(np.float64)) * rot[:, None]
        out[t, :, ia] = z.real
        out[t, :, ib] = z.imag
    return out


@pytest.mark.parametrize("mode", (oracle.ROPE_NEOX, oracle.ROPE_NORM))
@pytest.mark.parametrize("d,n_dims", ((128, 128), (128, 64), (64, 64), (256, 128), (96, 32)))
def test_rope_matches_complex_rotation(mode, d, n_dims):
    r = np.random.default_rng(d * 7 + n_dims + mode)
    m, heads = 5, 3
    x = r.standard_normal((m, heads, d)).astype(np.float32) * 2
    pos = np.array([0, 1, 17, 1000, 4095], np.int32)
    ts = oracle.rope_theta_scale(10000.0, n_dims)
    ff = (1.0 + r.random(n_dims // 2) * 3).astype(np.float32)
    for factors in (None, ff):
        got = oracle.rms_norm_rope(x, pos, d, n_dims, ts, mode=mode, ff=factors, freq_scale=0.75, attn_factor=1.25)
        exp = numpy_rope(x, pos, n_dims, ts, mode, ff=factors, freq_scale=0.75, attn_factor=1.25)
        # numpy's f32 power and libm's powf may differ in the last bit, i.e. by one ulp of theta <= pos * 2^-23 rad
        tol = np.abs(x).max() * (2e-6 + pos.astype(np.float64) * 2.0 ** -21)
        assert (np.abs(got - exp).max(axis=(1, 2)) < tol).all()
        assert (got[:, :, n_dims:] == x[:, :, n_dims:]).all()          # rope_funcs.glsl:56-61,90-95


def test_rope_invariants():
    r = np.random.default_rng(3)
    d = 128
    x = r.standard_normal((4, 2, d)).astype(np.float32)
    ts = oracle.rope_theta_scale(FREQ_BASE, d)
    for mode in (oracle.ROPE_NEOX, oracle.ROPE_NORM):
        a = oracle.rms_norm_rope(x, [3, 50, 700, 2000], d, d, ts, mode=mode)
        ia, ib = (slice(0, d // 2), slice(d // 2, d)) if mode == oracle.ROPE_NEOX else (slice(0, d, 2), slice(1, d, 2))
        n0 = x[..., ia].astype(np.float64) ** 2 + x[..., ib].astype(np.float64) ** 2
        n1 = a[..., ia].astype(np.float64) ** 2 + a[..., ib].astype(np.float64) ** 2
        assert np.abs(n0 - n1).max() < 1e-5                           # a rotation keeps every pair's norm
        assert (oracle.rms_norm_rope(x, [0, 0, 0, 0], d, d, ts, mode=mode) == x).all()   # position 0: identity, exactly
        b = oracle.rms_norm_rope(a, [5, 14, 300, 48], d, d, ts, mode=mode)              # positions add
        c = oracle.rms_norm_rope(x, [8, 64, 1000, 2048], d, d, ts, mode=mode)
        assert np.abs(b - c).max() < 2e-3
    # NEOX and NORM agree after permuting the elements into each other's pairing
    perm = np.empty(d, np.int64)
    perm[0::2] = np.arange(d // 2)
    perm[1::2] = np.arange(d // 2) + d // 2
    neox = oracle.rms_norm_rope(x, [3, 50, 700, 2000], d, d, ts, mode=oracle.ROPE_NEOX)
    norm = oracle.rms_norm_rope(x[..., perm], [3, 50, 700, 2000], d, d, ts, mode=oracle.ROPE_NORM)
    assert (norm == neox[..., perm]).all()


def test_rms_norm_part():
    r = np.random.default_rng(5)
    d = 128
    x = (r.standard_normal((3, 4, d)) * 3).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    eps = 1e-6
    # n_dims = 0: no rotation, the pure rms_norm * weight (CPU formula of tests/correctness.rs:680-700)
    got = oracle.rms_norm_rope(x, [7, 8, 9], d, 0, 1.0, weight=w, eps=eps)
    x64 = x.astype(np.float64)
    exp = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps) * w
    assert np.abs(got - exp).max() < 1e-6 * np.abs(exp).max() + 1e-7
    ones = np.ones(d, np.float32)
    unit = oracle.rms_norm_rope(x, [0, 0, 0], d, 0, 1.0, weight=ones, eps=0.0)
    assert np.abs((unit.astype(np.float64) ** 2).mean(-1) - 1).max() < 1e-6          # unit mean square
    assert np.abs(oracle.rms_norm_rope(x * 8, [0, 0, 0], d, 0, 1.0, weight=ones, eps=0.0) - unit).max() < 1e-6   # scale-invariant
    # norm then rotation == rotation of the normed row
    ts = oracle.rope_theta_scale(10000.0, d)
    both = oracle.rms_norm_rope(x, [7, 80, 900], d, d, ts, weight=w, eps=eps)
    two = oracle.rms_norm_rope(got, [7, 80, 900], d, d, ts)
    assert (both == two).all()
