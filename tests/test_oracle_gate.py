"""Pins the oracle's gated-output routine (vk_shaders/sigmoid_mul.comp:40-53).  The reference has no test of this
shader, so the checks are a library sigmoid, closed-form values and a literal pure-Python restatement of the index map."""
import numpy as np
import pytest
from scipy.special import expit

import oracle


def test_sigmoid_values_match_scipy_and_closed_forms():
    g = np.concatenate([np.linspace(-30, 30, 4001), [0.0, -100.0, 100.0, -1e-8, 88.0, -88.0, -1000.0]]).astype(np.float32)
    x = np.full(g.shape, 3.0, dtype=np.float32)
    out = oracle.sigmoid_mul(g, x, g.size, g.size, 0)
    want = np.float32(3.0) * expit(g.astype(np.float64)).astype(np.float32)
    assert (out == want).all()
    assert out[4001] == np.float32(1.5)                      # sigmoid(0) = 1/2
    assert 0.0 < out[4002] < 1e-42 and out[4003] == np.float32(3.0)   # sigmoid(-100) is an f32 subnormal, sigmoid(100) rounds to 1
    assert out[-1] == 0.0                                       # exp overflows to +inf: 1 / inf = 0, no NaN
    assert np.isfinite(out).all()
    # sigmoid(g) + sigmoid(-g) = 1
    a = oracle.sigmoid_mul(g, np.ones_like(g), g.size, g.size, 0)
    b = oracle.sigmoid_mul(-g, np.ones_like(g), g.size, g.size, 0)
    assert np.abs(a + b - 1).max() < 1.2e-7


@pytest.mark.parametrize("tokens,chunk,stride,offset", (
    (1, 24, 24, 24),      # decode: gate behind Q in q_buf (executor/attention.rs:655-664)
    (5, 8, 16, 8),        # batch: per (token, head) slice [Q | G] (executor/attention.rs:2433-2441)
    (3, 6, 10, 2),
    (4, 1, 3, 1),
))
def test_index_map_against_a_literal_loop(tokens, chunk, stride, offset):
    r = np.random.default_rng(chunk * 100 + stride)
    ne = tokens * chunk
    gate = r.standard_normal(tokens * stride + offset + chunk).astype(np.float32)
    data = r.standard_normal(ne).astype(np.float32)
    out = oracle.sigmoid_mul(gate, data, chunk, stride, offset)
    for i in range(ne):
        token = i // chunk
        within = i - token * chunk
        g = float(gate[token * stride + offset + within])
        want = np.float32(data[i]) * np.float32(1.0 / (1.0 + np.exp(-g)))
        assert out[i] == want, i
    # elements whose gate is never addressed do not matter
    used = np.zeros(gate.size, bool)
    for i in range(ne):
        used[(i // chunk) * stride + offset + i % chunk] = True
    gate2 = np.where(used, gate, np.float32(77.0))
    assert (oracle.sigmoid_mul(gate2, data, chunk, stride, offset) == out).all()


def test_empty_input():
    assert oracle.sigmoid_mul(np.zeros(4, np.float32), np.zeros(0, np.float32), 4, 4, 0).size == 0
