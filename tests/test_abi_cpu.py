"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header declares, does
the layout arithmetic of the reference (kv_cache.rs), and rejects bad arguments before touching a
device.  No compute entry point is exercised here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle
import vulkanforge_amd as vf
from vulkanforge_amd import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "vfkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vfkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _ffi.lib()
    names = _declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(L, n), n
    assert sorted(_ffi.SIGNATURES) == names          # the ctypes table and the header agree
    assert L.vfkv_abi_version() == 1
    assert L.vfkv_status_string(0) == b"ok" and L.vfkv_status_string(-3) == b"misaligned offset"


def _c_prototypes():
    """name -> number of parameters, from include/vfkv.h."""
    text = open(os.path.join(ROOT, "include", "vfkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for name, args in re.findall(r"\b(vfkv_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = args.strip()
        protos[name] = 0 if args in ("", "void") else args.count(",") + 1
    return protos


def test_rust_binding_file_declares_every_exported_symbol_with_the_same_arity():
    # the extern "C" block a Rust host compiles (vulkanforge_amd/host/rust/ffi.rs) must not drift from the header
    text = open(os.path.join(ROOT, "vulkanforge_amd", "host", "rust", "ffi.rs")).read()
    text = re.sub(r"//[^\n]*", "", text)
    rust = {}
    for name, args in re.findall(r"pub fn (vfkv_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*(?:->[^;]*)?;", text, flags=re.S):
        args = args.strip()
        rust[name] = 0 if args == "" else args.count(",") + 1
    protos = _c_prototypes()
    assert sorted(protos) == _declared_symbols()
    assert rust == protos
    # the build script compiles every translation unit the Makefile links into the library
    build = open(os.path.join(ROOT, "vulkanforge_amd", "host", "rust", "build.rs")).read()
    mk = open(os.path.join(ROOT, "vulkanforge_amd", "csrc", "Makefile")).read()
    srcs = re.search(r"^SRCS\s*:=\s*(.*)$", mk, flags=re.M).group(1).split()
    assert sorted(re.findall(r'"([a-z_]+\.hip)"', build)) == sorted(srcs)


def test_param_structs_are_32_bytes():
    # pipeline.rs:569 and :611
    assert C.sizeof(_ffi.SplitParams) == 32 and C.sizeof(_ffi.BatchParams) == 32
    assert _ffi.SplitParams.scale.offset == 20 and _ffi.SplitParams.kv_start.offset == 28
    assert _ffi.BatchParams.scale.offset == 24 and _ffi.BatchParams.kv_start.offset == 28


@pytest.mark.parametrize("dtype", list(vf.KvDtype))
def test_uniform_layout_matches_reference_figures(dtype):
    # kv_cache.rs:553-587: 36 x 8 x 128 x 2048 -> 576 / 288 MiB (and 144 for FP8)
    c = vf.KvCache(vf.KvCacheConfig(36, 8, 128, 2048, dtype=dtype), layout_only=True)
    es = dtype.element_size()
    assert 2 * c.bytes_per_buffer() == {4: 576, 2: 288, 1: 144}[es] * 1024 * 1024
    assert c.row_bytes(0) == 8 * 128 * es
    assert c.layer_size_bytes(5) == 2048 * 8 * 128 * es
    assert c.layer_offset_bytes(5) == 5 * 2048 * 8 * 128 * es
    assert c.layer_offset_elems(5) == 5 * 2048 * 8 * 128
    assert c.pos_offset_bytes(5, 77) == c.layer_offset_bytes(5) + 77 * c.row_bytes(5)
    assert c.head_dim_for(3) == 128 and c.kv_heads_for(3) == 8
    off = oracle.layout_offsets(36, 8, 128, 2048, int(dtype))
    assert [c.layer_offset_bytes(i) for i in range(36)] == list(map(int, off[:-1]))
    assert c.current_seq_len == 0
    c.current_seq_len = 17
    assert c.current_seq_len == 17
    c.reset()
    assert c.current_seq_len == 0
    assert c.k_ptr == 0 and c.v_ptr == 0
    c.destroy()


def test_heterogeneous_layout_matches_oracle():
    hd, kvh = [256, 256, 512, 256, 512], [8, 8, 2, 8, 2]
    c = vf.KvCache(vf.KvCacheConfig(5, 999, 999, 1000, hd, kvh, vf.KvDtype.F8), layout_only=True)
    off = oracle.layout_offsets(5, 999, 999, 1000, oracle.F8, hd, kvh)
    for i in range(5):
        assert c.layer_offset_bytes(i) == int(off[i])
        assert c.layer_size_bytes(i) == int(off[i + 1] - off[i])
        assert c.row_bytes(i) == hd[i] * kvh[i]
        assert c.head_dim_for(i) == hd[i] and c.kv_heads_for(i) == kvh[i]
        assert c.pos_offset_bytes(i, 999) == int(off[i]) + 999 * hd[i] * kvh[i]
    assert c.bytes_per_buffer() == int(off[-1])
    with pytest.raises(ValueError):
        vf.KvCache(vf.KvCacheConfig(5, 8, 128, 10, per_layer_head_dim=[1, 2]), layout_only=True)


def test_kv_bytes_per_token_reference_cases():
    # kv_cache.rs:518-551
    assert vf.kv_bytes_per_token(40, 8, 128, None, None, 2) == 2 * 2 * 40 * 8 * 128
    assert vf.kv_bytes_per_token(4, 999, 999, [256, 256, 512, 512], [2, 2, 4, 4], 1) == 10_240
    assert vf.kv_bytes_per_token(3, 0xFFFFFFFF, 0xFFFFFFFF, None, None, 1 << 40) == (1 << 64) - 1  # saturates


def test_size_overflow_is_an_error_not_a_wrap():
    with pytest.raises(vf.VfkvError) as e:
        vf.KvCache(vf.KvCacheConfig(0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF, dtype=vf.KvDtype.F32),
                   layout_only=True)
    assert e.value.status == -2
    with pytest.raises(vf.VfkvError) as e:
        vf.KvCache(vf.KvCacheConfig(2, 8, 128, 0xFFFFFFFF, [0xFFFFFFFF, 1], [0xFFFFFFFF, 1], vf.KvDtype.F32),
                   layout_only=True)
    assert e.value.status == -2


def test_guard_kv_precision():
    # kv_cache.rs:596-630
    for kv in (vf.KvDtype.F32, vf.KvDtype.F16):
        with pytest.raises(vf.VfkvError) as e:
            vf.guard_kv_precision(True, kv)
        assert "FP8" in str(e.value)
        vf.guard_kv_precision(True, kv, force=True)
        vf.guard_kv_precision(False, kv)
    vf.guard_kv_precision(True, vf.KvDtype.F8)


def test_kv_start_helpers_match_oracle():
    L = _ffi.lib()
    for pos, win in ((16383, 4096), (100, 4096), (4095, 4096), (4096, 4096), (0, 1), (0xFFFFFFFE, 5)):
        assert L.vfkv_kv_start_decode(pos, win) == oracle.kv_start_decode(pos, win)
    for base, n, win in ((4096, 512, 0), (4096, 512, 1024), (10, 20, 1024), (0, 1, 1)):
        assert L.vfkv_kv_start_batch(base, n, win) == oracle.kv_start_batch(base, n, win)


def test_bad_arguments_are_rejected_before_any_device_work():
    L = _ffi.lib()
    fake = 0x1000  # never dereferenced: every call below must fail in validation
    assert L.vfkv_store_fp8(fake, fake, 8, 2, None) == -3       # runs.rs:2448-2453
    assert L.vfkv_copy_fp16(fake, fake, 8, 6, None) == -3       # runs.rs:2400-2404
    assert b"uint-aligned" in L.vfkv_last_error()
    assert L.vfkv_store_fp8(None, fake, 8, 0, None) == -1
    assert L.vfkv_store_fp8(None, None, 0, 0, None) == 0        # nothing to do
    assert L.vfkv_fp8_to_f16(None, fake, 4, None) == -1
    p = _ffi.SplitParams(30, 8, 128, 100, 0, 0.1, 2, 0)
    assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 64, 0.0, None) == -1
    assert b"multiple" in L.vfkv_last_error()
    p = _ffi.SplitParams(32, 8, 128, 0, 0, 0.1, 0, 0)
    assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 64, 0.0, None) == -1
    p = _ffi.SplitParams(32, 8, 128, 100, 0, 0.1, 3, 0)          # n_tiles must be ceil(100/64) = 2
    assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 64, 0.0, None) == -1
    p = _ffi.SplitParams(32, 8, 1024, 100, 0, 0.1, 2, 0)
    assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 64, 0.0, None) == -4
    p = _ffi.SplitParams(32, 8, 128, 100, 0, 0.1, 2, 0)
    assert L.vfkv_flash_attn_split(fake, fake, fake, 7, fake, fake, fake, C.byref(p), 64, 0.0, None) == -1
    assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 60, 0.0, None) == -1
    assert L.vfkv_flash_attn_reduce(fake, fake, fake, fake, 32, 128, 0, None) == -1
    b = _ffi.BatchParams(32, 8, 128, 4, 64, 60, 0.1, 61)        # kv_start hides every key of query 0
    assert L.vfkv_flash_attn_batch(fake, fake, fake, 0, fake, C.byref(b), 0.0, None) == -1
    b = _ffi.BatchParams(32, 5, 128, 4, 64, 60, 0.1, 0)
    assert L.vfkv_flash_attn_batch(fake, fake, fake, 0, fake, C.byref(b), 0.0, None) == -1
    h = C.c_void_p()
    assert L.vfkv_workspace_create(0, 128, 100, C.byref(h)) == -1
    # a layout-only cache has no buffers: compute entry points refuse it
    c = vf.KvCache(vf.KvCacheConfig(2, 8, 128, 64, dtype=vf.KvDtype.F8), layout_only=True)
    assert L.vfkv_kv_write(c.handle, 0, 0, 1, fake, fake, None) == -1
    assert L.vfkv_cache_zero_fill(c.handle, None) == -1
    assert L.vfkv_decode_attention(c.handle, 0, 0, 32, fake, fake, 3, 0, 0.1, 0.0, None, None) == -1


def test_product_package_does_not_reach_into_the_oracle():
    pkg = os.path.join(ROOT, "vulkanforge_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", ".hpp")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"import\s+oracle|from\s+oracle|oracle/|vfkv_oracle|vfo_", text), \
                    os.path.join(dirpath, f)


def test_no_device_means_loud_failure():
    if _ffi.lib().vfkv_device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(vf.VfkvError):
        vf.KvCache(vf.KvCacheConfig(1, 1, 64, 16, dtype=vf.KvDtype.F8))
    with pytest.raises(ValueError):
        import torch
        vf.Forward.run_kv_store_fp8(torch.zeros(8), torch.zeros(8, dtype=torch.uint8), 8, 0, stream=0)


def test_k_rope_kv_write_rejects_bad_arguments():
    # validation happens before any device work: the buffers below are never dereferenced
    cache = vf.KvCache(vf.KvCacheConfig(2, 8, 128, 64, dtype=vf.KvDtype.F8), k_buffer=0x10000, v_buffer=0x20000)
    L = _ffi.lib()
    fake = 0x1000

    def call(mode=_ffi.ROPE_NEOX, rot=128, fs=1.0, layer=0, pos=0, n=1, k=fake, v=fake, params=True):
        p = _ffi.RopeParams(mode, rot, 0.9, fs, 1.0, 1e-6)
        return L.vfkv_k_rope_kv_write(cache.handle, layer, pos, n, k, v, None, None, None,
                                      C.byref(p) if params else None, None, None)

    assert call(n=0) == 0                       # nothing to do
    assert call(mode=8) == -4                   # MROPE / VISION are not built
    assert b"rope_mode" in L.vfkv_last_error()
    assert call(rot=127) == -1 and call(rot=130) == -1
    assert call(layer=2) == -1 and call(pos=64) == -1 and call(pos=60, n=5) == -1
    assert call(k=None) == -1 and call(v=None) == -1 and call(params=False) == -1
    assert call(fs=0.0) == -1
    p = _ffi.RopeParams(_ffi.ROPE_NEOX, 128, 0.9, 1.0, 1.0, 1e-6)
    assert L.vfkv_qk_rope_kv_write(cache.handle, 0, 0, 1, 32, None, None, fake, fake, fake, None, None, None, C.byref(p),
                                   None, None) == -1          # NULL query
    assert L.vfkv_qk_rope_kv_write(cache.handle, 0, 0, 1, 0, fake, None, fake, fake, fake, None, None, None, C.byref(p),
                                   None, None) == -1          # no heads
    cache.destroy()


def test_rms_norm_mul_rope_rejects_bad_arguments():
    L = _ffi.lib()
    fake = 0x1000

    def call(mode=_ffi.ROPE_NEOX, rot=128, hd=128, heads=32, m=1, fs=1.0, x=fake, out=fake, params=True):
        p = _ffi.RopeParams(mode, rot, 0.9, fs, 1.0, 1e-6)
        return L.vfkv_rms_norm_mul_rope(x, None, out, hd, heads, m, None, 0, None, C.byref(p) if params else None, None)

    assert call(m=0) == 0 and call(heads=0) == 0
    assert call(mode=24) == -4 and call(hd=1024, rot=64) == -4 and call(hd=130, rot=64) == -4
    assert call(rot=129) == -1 and call(rot=256) == -1 and call(fs=-1.0) == -1
    assert call(x=None) == -1 and call(out=None) == -1 and call(params=False) == -1


def test_build_kv_sources_reference_patterns():
    # gguf.rs:1531-1567 (E2B: 35 layers, every fifth is a full layer, the first 15 own their rows)
    pattern = [(i % 5) != 4 for i in range(35)]
    srcs = vf.build_kv_sources(pattern, 15, 35)
    assert srcs[13] == vf.kv_cache.KV_OWN_PUBLISHES_SLIDING
    assert srcs[14] == vf.kv_cache.KV_OWN_PUBLISHES_FULL
    for i in (0, 1, 2, 3, 5, 6, 7, 8, 10, 11, 12, 4, 9):
        assert srcs[i] == vf.kv_cache.KV_OWN, i
    for i in range(15, 35):
        want = vf.kv_cache.KV_SUBSCRIBES_FULL if i % 5 == 4 else vf.kv_cache.KV_SUBSCRIBES_SLIDING
        assert srcs[i] == want, i
    # gguf.rs:1569-1590: no full layer among the owners
    p = [True] * 10
    p[7] = False
    srcs = vf.build_kv_sources(p, 5, 10)
    assert srcs[4] == vf.kv_cache.KV_OWN_PUBLISHES_SLIDING
    assert srcs[7] == vf.kv_cache.KV_SUBSCRIBES_FULL
    assert [srcs[i] for i in (5, 6, 8, 9)] == [vf.kv_cache.KV_SUBSCRIBES_SLIDING] * 4
    assert srcs[:4] == [vf.kv_cache.KV_OWN] * 4
    # a pattern shorter than the stack: the missing layers count as sliding (gguf.rs:916-918)
    assert vf.build_kv_sources([False], 2, 3) == [vf.kv_cache.KV_OWN_PUBLISHES_FULL, vf.kv_cache.KV_OWN_PUBLISHES_SLIDING,
                                                   vf.kv_cache.KV_SUBSCRIBES_SLIDING]


def test_kv_read_layer_follows_the_first_publisher():
    # forward/arch/gemma4.rs:27-49 on the E2B stack: sliding subscribers read layer 13, full subscribers layer 14
    srcs = vf.build_kv_sources([(i % 5) != 4 for i in range(35)], 15, 35)
    for layer in range(35):
        want = layer if layer < 15 else (14 if layer % 5 == 4 else 13)
        assert vf.gemma4_kv_read_layer(srcs, layer) == want, layer
    assert vf.gemma4_kv_read_layer(None, 7) == 7                    # not a Gemma-4 stack
    assert vf.gemma4_kv_read_layer(srcs, 99) == 99
    # a subscriber without publisher reads itself (`unwrap_or(layer)`)
    srcs = vf.build_kv_sources([True] * 5 + [True, True, False, True, True], 5, 10)
    assert vf.gemma4_kv_read_layer(srcs, 7) == 7
    assert vf.gemma4_kv_read_layer(srcs, 8) == 4
    # two publishers of one kind (hand-built): the first wins (`find`)
    K = vf.kv_cache
    assert vf.gemma4_kv_read_layer([K.KV_OWN_PUBLISHES_FULL, K.KV_OWN_PUBLISHES_FULL, K.KV_SUBSCRIBES_FULL], 2) == 0


def test_prefix_reuse_start_reference_cases():
    # server/state.rs:363-396
    assert vf.prefix_reuse_start([], [1, 2, 3]) == 0
    assert vf.prefix_reuse_start([9, 8, 7], [1, 2, 3]) == 0
    assert vf.prefix_reuse_start([10, 11, 12, 13, 14], [10, 11, 12, 99]) == 3
    assert vf.prefix_reuse_start([1, 2, 3, 4, 5], [1, 2, 3]) == 2        # lcp 3, capped at len - 1
    assert vf.prefix_reuse_start([1, 2, 3], [1, 2, 3]) == 2
    assert vf.prefix_reuse_start([1, 2, 3, 4], [1, 2, 3, 4]) == 3        # "k must be len-1, not the full length"
    assert vf.prefix_reuse_start([1, 2, 3], []) == 0
    assert vf.prefix_reuse_start([5], [5]) == 0


def test_gated_entry_points_reject_bad_arguments_before_any_device_work():
    L = _ffi.lib()
    g = _ffi.Gate(0, 16, 16, 0)
    assert L.vfkv_sigmoid_mul(C.byref(g), 64, 16, None) == -1                      # NULL gate buffer
    assert L.vfkv_sigmoid_mul(None, 64, 16, None) == -1
    g = _ffi.Gate(64, 0, 16, 0)
    assert L.vfkv_sigmoid_mul(C.byref(g), 64, 16, None) == -1                      # chunk 0
    assert b"chunk" in L.vfkv_last_error()
    g = _ffi.Gate(66, 16, 16, 0)
    assert L.vfkv_sigmoid_mul(C.byref(g), 64, 16, None) < 0                        # misaligned gate
    g = _ffi.Gate(64, 16, 16, 0)
    assert L.vfkv_sigmoid_mul(C.byref(g), 0, 16, None) == -1                       # NULL data
    assert L.vfkv_sigmoid_mul(C.byref(g), 0, 0, None) == 0                         # nothing to do
    assert L.vfkv_decode_attention_gated(None, 0, 0, 4, 64, None, None, 64, 0, 0, 1.0, 0.0, None, None, None) == -1
    assert L.vfkv_prefill_attention_gated(None, 0, 0, 4, 64, 64, 1, 0, 0, 1.0, 0.0, None, None) == -1
    assert L.vfkv_prefill_attention_gated(None, 0, 0, 4, 64, 64, 1, 0, 0, 1.0, 0.0, C.byref(g), None) == -1   # no cache


def test_prefill_attention_ws_rejects_bad_arguments_before_any_device_work():
    L = _ffi.lib()
    assert L.vfkv_prefill_attention_ws(None, 0, 0, 4, 64, 64, 1, 0, 0, 1.0, 0.0, None, None) == -1      # no workspace
    assert b"workspace" in L.vfkv_last_error()
    assert L.vfkv_prefill_attention_ws(None, 0, 0, 4, 64, 64, 1, 0, 0, 1.0, 0.0, 64, None) == -1        # no cache


def test_static_decode_call_rejects_partials_beyond_its_array():
    # vfkv_decode_attention_static holds its partials in a fixed device array; a launch whose partials exceed it must
    # fail with VFKV_ERR_WORKSPACE before any device work.  The library's own tile choice never needs more than the
    # array holds, so the case is forced with 64-key tiles (VFKV_DECODE_TILE is read once per process: child process).
    import subprocess
    import sys
    code = (
        "import ctypes as C\n"
        "from vulkanforge_amd import _ffi\n"
        "L = _ffi.lib()\n"
        "cfg = _ffi.CacheConfig(1, 8, 128, 65536, None, None, 2)\n"
        "h = C.c_void_p()\n"
        "assert L.vfkv_cache_create_external(C.byref(cfg), 0x1000, 0x2000, C.byref(h)) == 0\n"
        "rc = L.vfkv_decode_attention_static(h, 0, 0, 32, 0x1000, 0x1000, 65535, 0, 1.0, 0.0, None)\n"
        "msg = L.vfkv_last_error().decode()\n"
        "assert rc == -7, (rc, msg)\n"
        "assert 'static buffer holds 5242880' in msg, msg\n"
        "rc = L.vfkv_decode_attention_static(h, 0, 0, 32, None, 0x1000, 10, 0, 1.0, 0.0, None)\n"
        "assert rc == -1\n"
        "print('ok')\n")
    env = dict(os.environ, VFKV_DECODE_TILE="64", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stderr


def test_validation_of_out_pointer_kv_layer_geometry_and_scale():
    L = _ffi.lib()
    fake = 0x1000
    cfg = _ffi.CacheConfig(2, 8, 128, 64, None, None, 2)
    assert L.vfkv_cache_create(C.byref(cfg), None) == -1                       # NULL out: an error, not a crash
    # a layer may only read the slab of a layer with the same row geometry (heterogeneous cache, gemma4.rs:27-49)
    hd = (C.c_uint32 * 3)(256, 512, 256)
    kvh = (C.c_uint32 * 3)(8, 2, 8)
    cfg = _ffi.CacheConfig(3, 8, 256, 128, hd, kvh, 2)
    h = C.c_void_p()
    assert L.vfkv_cache_create_external(C.byref(cfg), fake, fake + 256, C.byref(h)) == 0
    ws = C.c_void_p(fake)                                                      # never dereferenced: validation fails first
    assert L.vfkv_decode_attention(h, 0, 1, 16, fake, fake, 10, 0, 0.1, 0.0, ws, None) == -1
    assert b"cannot read the slab" in L.vfkv_last_error()
    assert L.vfkv_prefill_attention(h, 0, 1, 16, fake, fake, 4, 0, 0, 0.1, 0.0, None) == -1
    assert L.vfkv_decode_attention_static(h, 2, 1, 16, fake, fake, 10, 0, 0.1, 0.0, None) == -1
    # the softmax scale must be positive and finite
    for bad in (0.0, -0.5, float("inf"), float("nan")):
        assert L.vfkv_decode_attention(h, 0, 2, 16, fake, fake, 10, 0, bad, 0.0, ws, None) == -1
        assert b"scale" in L.vfkv_last_error()
        p = _ffi.SplitParams(32, 8, 128, 100, 0, bad, 2, 0)
        assert L.vfkv_flash_attn_split(fake, fake, fake, 2, fake, fake, fake, C.byref(p), 64, 0.0, None) == -1
        b = _ffi.BatchParams(32, 8, 128, 4, 64, 60, bad, 0)
        assert L.vfkv_flash_attn_batch(fake, fake, fake, 0, fake, C.byref(b), 0.0, None) == -1
        assert L.vfkv_prefill_attention(h, 0, 2, 16, fake, fake, 4, 0, 0, bad, 0.0, None) == -1
    L.vfkv_cache_destroy(h)


def test_external_buffers_of_equal_alignment_leave_a_note_not_an_error():
    L = _ffi.lib()
    cfg = _ffi.CacheConfig(1, 8, 128, 64, None, None, 2)
    h = C.c_void_p()
    assert L.vfkv_flash_attn_reduce(None, None, None, None, 1, 1, 1, None) == -1     # leaves an error text behind
    err = L.vfkv_last_error()
    assert L.vfkv_cache_create_external(C.byref(cfg), 0x10000, 0x20000, C.byref(h)) == 0
    assert b"256 bytes" in L.vfkv_cache_kv_alignment_note(h)
    assert L.vfkv_last_error() == err                  # a successful call neither writes nor clears the error text
    L.vfkv_cache_destroy(h)
    assert L.vfkv_cache_create_external(C.byref(cfg), 0x10000, 0x20100, C.byref(h)) == 0
    assert L.vfkv_cache_kv_alignment_note(h) == b""
    L.vfkv_cache_destroy(h)
    assert L.vfkv_cache_kv_alignment_note(None) == b"" and L.vfkv_last_note() == b""


def test_dynamic_symbol_table_holds_the_declared_entry_points_only():
    import subprocess
    so = os.path.join(ROOT, "vulkanforge_amd", "libvfkv.so")
    out = subprocess.run(["nm", "-D", "--defined-only", so], check=True, capture_output=True, text=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == _declared_symbols()
