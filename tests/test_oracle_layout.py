"""Pins the oracle's cache-layout arithmetic against the figures in the reference's unit tests
(src/backend/vulkan/kv_cache.rs:518-587) and against closed forms."""
import numpy as np

import oracle


def test_reference_size_figures():
    # kv_cache.rs:553-587 -- Qwen3-8B: 36 layers x 8 kv heads x 128 x 2048
    off32 = oracle.layout_offsets(36, 8, 128, 2048, oracle.F32)
    off16 = oracle.layout_offsets(36, 8, 128, 2048, oracle.F16)
    off8 = oracle.layout_offsets(36, 8, 128, 2048, oracle.F8)
    assert 2 * int(off32[-1]) == 576 * 1024 * 1024
    assert 2 * int(off16[-1]) == 288 * 1024 * 1024
    assert 2 * int(off8[-1]) == 144 * 1024 * 1024
    assert (np.diff(off32) == 2048 * 8 * 128 * 4).all()


def test_bytes_per_token_reference_cases():
    # kv_cache.rs:518-551
    assert oracle.kv_bytes_per_token(40, 8, 128, 2) == 2 * 2 * 40 * 8 * 128
    assert oracle.kv_bytes_per_token(40, 8, 128, 1) * 2 == oracle.kv_bytes_per_token(40, 8, 128, 2)
    got = oracle.kv_bytes_per_token(4, 999, 999, 1, [256, 256, 512, 512], [2, 2, 4, 4])
    assert got == 10_240
    assert oracle.kv_bytes_per_token(40, 8, 128, 2) * 12288 == 2 * 40 * 8 * 12288 * 128 * 2


def test_heterogeneous_offsets():
    off = oracle.layout_offsets(4, 999, 999, 100, oracle.F8, [256, 256, 512, 512], [2, 2, 4, 4])
    assert list(off) == [0, 51200, 102400, 307200, 512000]
    off = oracle.layout_offsets(3, 8, 64, 10, oracle.F16, per_layer_head_dim=[64, 128, 64])
    assert list(off) == [0, 10240, 30720, 40960]


def test_overflow_is_an_error():
    assert oracle.layout_offsets(2, 0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF, oracle.F32) is None
    assert oracle.layout_offsets(1 << 10, 1 << 20, 1 << 20, 1 << 20, oracle.F32) is None


def test_kv_start_rules():
    # gemma4.rs:59-73 and executor/attention.rs:2215-2219
    assert oracle.kv_start_decode(16383, 4096) == 12288
    assert oracle.kv_start_decode(100, 4096) == 0
    assert oracle.kv_start_decode(4095, 4096) == 0 and oracle.kv_start_decode(4096, 4096) == 1
    assert oracle.kv_start_batch(4096, 512, 0) == 0
    assert oracle.kv_start_batch(4096, 512, 1024) == 3584
    assert oracle.kv_start_batch(10, 20, 1024) == 0
