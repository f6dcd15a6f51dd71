"""ctypes front-end of the CPU oracle (``vfkv_oracle.c``).

Test infrastructure only: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvfkv_oracle.so")

F32, F16, F8 = 0, 1, 2
ELEM_SIZE = {F32: 4, F16: 2, F8: 1}
NP_DTYPE = {F32: np.float32, F16: np.uint16, F8: np.uint8}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _declare(_lib)
    return _lib


_u8p, _u16p, _u32p, _u64p, _f32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_uint32, C.c_uint64, C.c_float))


def _declare(L: C.CDLL) -> None:
    L.vfo_e4m3_to_f32.argtypes = [C.c_uint8]
    L.vfo_e4m3_to_f32.restype = C.c_float
    L.vfo_f32_to_e4m3.argtypes = [C.c_float]
    L.vfo_f32_to_e4m3.restype = C.c_uint8
    L.vfo_f32_to_f16.argtypes = [C.c_float]
    L.vfo_f32_to_f16.restype = C.c_uint16
    L.vfo_f16_to_f32.argtypes = [C.c_uint16]
    L.vfo_f16_to_f32.restype = C.c_float
    for name in ("vfo_f32_to_e4m3_array", "vfo_e4m3_to_f32_array", "vfo_f32_to_f16_array",
                 "vfo_f16_to_f32_array"):
        getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
        getattr(L, name).restype = None
    for name in ("vfo_kv_store_fp8", "vfo_kv_copy_fp16"):
        getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint64]
        getattr(L, name).restype = C.c_int
    L.vfo_kv_fp8_to_f16.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
    L.vfo_kv_fp8_to_f16.restype = None
    L.vfo_layout_offsets.argtypes = [C.c_uint32] * 4 + [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
    L.vfo_layout_offsets.restype = C.c_int
    L.vfo_kv_bytes_per_token.argtypes = [C.c_uint32] * 3 + [C.c_void_p, C.c_void_p, C.c_uint64]
    L.vfo_kv_bytes_per_token.restype = C.c_uint64
    L.vfo_kv_start_decode.argtypes = [C.c_uint32, C.c_uint32]
    L.vfo_kv_start_decode.restype = C.c_uint32
    L.vfo_kv_start_batch.argtypes = [C.c_uint32] * 3
    L.vfo_kv_start_batch.restype = C.c_uint32
    L.vfo_attn_decode_ref.argtypes = ([C.c_void_p] * 3 + [C.c_uint32] * 6 + [C.c_float] * 2
                                      + [C.c_void_p, C.c_int])
    L.vfo_attn_decode_ref.restype = None
    L.vfo_attn_split.argtypes = ([C.c_void_p] * 3 + [C.c_uint32] * 6 + [C.c_float] * 2
                                 + [C.c_uint32] * 2 + [C.c_void_p] * 3 + [C.c_int])
    L.vfo_attn_split.restype = None
    L.vfo_attn_reduce.argtypes = [C.c_void_p] * 3 + [C.c_uint32] * 3 + [C.c_void_p]
    L.vfo_attn_reduce.restype = None
    for name in ("vfo_attn_batch_ref", "vfo_attn_batch_shader"):
        getattr(L, name).argtypes = ([C.c_void_p] * 3 + [C.c_uint32] * 8 + [C.c_float] * 2
                                     + [C.c_void_p, C.c_int])
        getattr(L, name).restype = None
    L.vfo_rms_norm_rope.argtypes = [C.c_void_p] * 5 + [C.c_uint32] * 5 + [C.c_float] * 4
    L.vfo_rms_norm_rope.restype = None
    L.vfo_sigmoid_mul.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32]
    L.vfo_sigmoid_mul.restype = None
    L.vfo_max_threads.argtypes = []
    L.vfo_max_threads.restype = C.c_int


def _p(a: np.ndarray) -> C.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def _opt_u32(a):
    if a is None:
        return None, C.c_void_p(0)
    arr = np.ascontiguousarray(a, dtype=np.uint32)
    return arr, _p(arr)


def default_threads() -> int:
    return int(lib().vfo_max_threads())


# ---- element conversions ------------------------------------------------------------------
def f32_to_e4m3(x) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().vfo_f32_to_e4m3_array(_p(x), _p(out), x.size)
    return out


def e4m3_to_f32(b) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape, dtype=np.float32)
    lib().vfo_e4m3_to_f32_array(_p(b), _p(out), b.size)
    return out


def f32_to_f16_bits(x) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().vfo_f32_to_f16_array(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(h) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().vfo_f16_to_f32_array(_p(h), _p(out), h.size)
    return out


# ---- append / expansion --------------------------------------------------------------------
def kv_store_fp8(src, dst_bytes: np.ndarray, n: int, dst_byte_offset: int) -> int:
    src = np.ascontiguousarray(src, dtype=np.float32)
    assert dst_bytes.dtype == np.uint8
    return int(lib().vfo_kv_store_fp8(_p(src), _p(dst_bytes), n, dst_byte_offset))


def kv_copy_fp16(src, dst_bytes: np.ndarray, n: int, dst_byte_offset: int) -> int:
    src = np.ascontiguousarray(src, dtype=np.float32)
    assert dst_bytes.dtype == np.uint8
    return int(lib().vfo_kv_copy_fp16(_p(src), _p(dst_bytes), n, dst_byte_offset))


def kv_fp8_to_f16(src_bytes) -> np.ndarray:
    src = np.ascontiguousarray(src_bytes, dtype=np.uint8)
    out = np.empty(src.shape, dtype=np.uint16)
    lib().vfo_kv_fp8_to_f16(_p(src), _p(out), src.size)
    return out


# ---- layout --------------------------------------------------------------------------------
def layout_offsets(n_layers, n_kv_heads, head_dim, max_seq, dtype, per_layer_head_dim=None,
                   per_layer_n_kv_heads=None):
    """Cumulative byte-offset table (n_layers+1 entries) or None on overflow."""
    out = np.zeros(n_layers + 1, dtype=np.uint64)
    _a, pa = _opt_u32(per_layer_head_dim)
    _b, pb = _opt_u32(per_layer_n_kv_heads)
    rc = lib().vfo_layout_offsets(n_layers, n_kv_heads, head_dim, max_seq, pa, pb, dtype, _p(out))
    return None if rc != 0 else out


def kv_bytes_per_token(n_layers, n_kv_heads, head_dim, elem_size, per_layer_head_dim=None,
                       per_layer_n_kv_heads=None) -> int:
    _a, pa = _opt_u32(per_layer_head_dim)
    _b, pb = _opt_u32(per_layer_n_kv_heads)
    return int(lib().vfo_kv_bytes_per_token(n_layers, n_kv_heads, head_dim, pa, pb, elem_size))


def kv_start_decode(position: int, window: int) -> int:
    return int(lib().vfo_kv_start_decode(position, window))


def kv_start_batch(base_pos: int, seq_len: int, window: int) -> int:
    return int(lib().vfo_kv_start_batch(base_pos, seq_len, window))


# ---- attention -----------------------------------------------------------------------------
def _kv(a: np.ndarray, dtype: int) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == NP_DTYPE[dtype], (a.dtype, dtype)
    return a


def attn_decode_ref(q, k, v, dtype, n_heads, n_kv_heads, head_dim, seq_len, scale, kv_start=0,
                    softcap=0.0, threads=None) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.float32)
    k, v = _kv(k, dtype), _kv(v, dtype)
    out = np.zeros((n_heads, head_dim), dtype=np.float32)
    lib().vfo_attn_decode_ref(_p(q), _p(k), _p(v), dtype, n_heads, n_kv_heads, head_dim, seq_len,
                              kv_start, scale, softcap, _p(out), threads or default_threads())
    return out


def attn_split(q, k, v, dtype, n_heads, n_kv_heads, head_dim, seq_len, scale, tile=64, kv_start=0,
               softcap=0.0, threads=None):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k, v = _kv(k, dtype), _kv(v, dtype)
    n_tiles = (seq_len + tile - 1) // tile
    so = np.zeros((n_heads, n_tiles, head_dim), dtype=np.float32)
    sm = np.zeros((n_heads, n_tiles), dtype=np.float32)
    ss = np.zeros((n_heads, n_tiles), dtype=np.float32)
    lib().vfo_attn_split(_p(q), _p(k), _p(v), dtype, n_heads, n_kv_heads, head_dim, seq_len, kv_start,
                         scale, softcap, tile, n_tiles, _p(so), _p(sm), _p(ss),
                         threads or default_threads())
    return so, sm, ss


def attn_reduce(so, sm, ss) -> np.ndarray:
    n_heads, n_tiles, head_dim = so.shape
    so = np.ascontiguousarray(so, dtype=np.float32)
    sm = np.ascontiguousarray(sm, dtype=np.float32)
    ss = np.ascontiguousarray(ss, dtype=np.float32)
    out = np.zeros((n_heads, head_dim), dtype=np.float32)
    lib().vfo_attn_reduce(_p(so), _p(sm), _p(ss), n_heads, head_dim, n_tiles, _p(out))
    return out


def _batch(fn, q, k, v, dtype, m, n_kv, n_heads, n_kv_heads, head_dim, q_start, scale, kv_start,
           softcap, threads):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k, v = _kv(k, dtype), _kv(v, dtype)
    out = np.zeros((m, n_heads, head_dim), dtype=np.float32)
    fn(_p(q), _p(k), _p(v), dtype, m, n_kv, n_heads, n_kv_heads, head_dim, q_start, kv_start, scale,
       softcap, _p(out), threads or default_threads())
    return out


def attn_batch_ref(q, k, v, dtype, m, n_kv, n_heads, n_kv_heads, head_dim, q_start, scale, kv_start=0,
                   softcap=0.0, threads=None) -> np.ndarray:
    return _batch(lib().vfo_attn_batch_ref, q, k, v, dtype, m, n_kv, n_heads, n_kv_heads, head_dim,
                  q_start, scale, kv_start, softcap, threads)


def attn_batch_shader(q, k, v, dtype, m, n_kv, n_heads, n_kv_heads, head_dim, q_start, scale,
                      kv_start=0, softcap=0.0, threads=None) -> np.ndarray:
    return _batch(lib().vfo_attn_batch_shader, q, k, v, dtype, m, n_kv, n_heads, n_kv_heads, head_dim,
                  q_start, scale, kv_start, softcap, threads)


ROPE_NORM, ROPE_NEOX = 0, 2


def rope_theta_scale(freq_base: float, rotary_dim: int) -> np.float32:
    """(1 / freq_base)^(2 / rotary_dim) in f32 (forward/layer_plan.rs:532)."""
    return np.float32(np.float32(1.0) / np.float32(freq_base)) ** np.float32(np.float32(2.0) / np.float32(rotary_dim))


def rms_norm_rope(x, pos, head_dim, n_dims, theta_scale, mode=ROPE_NEOX, weight=None, ff=None, freq_scale=1.0,
                  attn_factor=1.0, eps=1e-6) -> np.ndarray:
    """x: [m, heads, head_dim] f32, pos: [m] int32 -> rotated (optionally RMS-normed * weight) copy."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, heads = x.shape[0], x.shape[1]
    assert x.shape[2] == head_dim
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    assert pos.shape == (m,)
    w = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
    f = None if ff is None else np.ascontiguousarray(ff, dtype=np.float32)
    out = np.empty_like(x)
    lib().vfo_rms_norm_rope(_p(x), _p(w) if w is not None else None, _p(pos), _p(f) if f is not None else None,
                            _p(out), m, heads, head_dim, mode, n_dims, float(theta_scale), float(freq_scale),
                            float(attn_factor), float(eps))
    return out


def sigmoid_mul(gate, data, chunk, stride, gate_offset) -> np.ndarray:
    """data[i] * sigmoid(gate[(i // chunk) * stride + gate_offset + i % chunk]) as a new array (flat index i)."""
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    out = np.array(data, dtype=np.float32, order="C", copy=True)
    if out.size:
        last = (out.size - 1) // chunk * stride + gate_offset + (out.size - 1) % chunk
        assert last < gate.size, "gate buffer too small"
    lib().vfo_sigmoid_mul(_p(gate), _p(out), out.size, chunk, stride, gate_offset)
    return out
