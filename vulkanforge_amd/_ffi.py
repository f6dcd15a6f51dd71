"""ctypes binding of ``libvfkv.so`` (declarations follow ``include/vfkv.h`` one to one)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libvfkv.so")

OK = 0
STATUS_NAMES = {0: "VFKV_OK", -1: "VFKV_ERR_INVALID_ARG", -2: "VFKV_ERR_OVERFLOW", -3: "VFKV_ERR_ALIGNMENT",
                -4: "VFKV_ERR_UNSUPPORTED", -5: "VFKV_ERR_HIP", -6: "VFKV_ERR_NO_DEVICE", -7: "VFKV_ERR_WORKSPACE"}


class VfkvError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


class CacheConfig(C.Structure):
    _fields_ = [("n_layers", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("max_seq_len", C.c_uint32), ("per_layer_head_dim", C.POINTER(C.c_uint32)),
                ("per_layer_n_kv_heads", C.POINTER(C.c_uint32)), ("dtype", C.c_uint32)]


class SplitParams(C.Structure):
    _fields_ = [("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("seq_len", C.c_uint32), ("max_seq", C.c_uint32), ("scale", C.c_float),
                ("n_tiles", C.c_uint32), ("kv_start", C.c_uint32)]


class BatchParams(C.Structure):
    _fields_ = [("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("m", C.c_uint32), ("n_kv", C.c_uint32), ("q_start", C.c_uint32), ("scale", C.c_float),
                ("kv_start", C.c_uint32)]


class RopeParams(C.Structure):
    _fields_ = [("rope_mode", C.c_uint32), ("rotary_dim", C.c_uint32), ("theta_scale", C.c_float),
                ("freq_scale", C.c_float), ("attn_factor", C.c_float), ("eps", C.c_float)]


class Gate(C.Structure):
    """SigmoidMulPushConstants (forward/runs.rs:2667) plus the gate buffer."""
    _fields_ = [("gate", C.c_void_p), ("chunk", C.c_uint32), ("stride", C.c_uint32), ("gate_offset", C.c_uint32)]


PREFILL_F16_WEIGHTS, PREFILL_FP8_SCORES, PREFILL_F16_QUERIES = 1, 2, 4   # the VFKV_PREFILL_* option bits
ROPE_NORM, ROPE_NEOX = 0, 2   # GGML_ROPE_TYPE_NORMAL / _NEOX (rms_norm.comp:25-26)

assert C.sizeof(SplitParams) == 32 and C.sizeof(BatchParams) == 32  # pipeline.rs:569,611

_u32, _u64, _vp, _f = C.c_uint32, C.c_uint64, C.c_void_p, C.c_float
_u32p = C.POINTER(C.c_uint32)

# name -> (restype, argtypes); every symbol declared in include/vfkv.h
SIGNATURES = {
    "vfkv_status_string": (C.c_char_p, [C.c_int]),
    "vfkv_last_error": (C.c_char_p, []),
    "vfkv_last_note": (C.c_char_p, []),
    "vfkv_abi_version": (_u32, []),
    "vfkv_device_count": (C.c_int, []),
    "vfkv_cache_create": (C.c_int, [C.POINTER(CacheConfig), C.POINTER(_vp)]),
    "vfkv_cache_create_external": (C.c_int, [C.POINTER(CacheConfig), _vp, _vp, C.POINTER(_vp)]),
    "vfkv_cache_kv_alignment_note": (C.c_char_p, [_vp]),
    "vfkv_cache_destroy": (None, [_vp]),
    "vfkv_cache_zero_fill": (C.c_int, [_vp, _vp]),
    "vfkv_cache_zero_layer": (C.c_int, [_vp, _u32, _vp]),
    "vfkv_cache_current_seq_len": (_u32, [_vp]),
    "vfkv_cache_set_current_seq_len": (None, [_vp, _u32]),
    "vfkv_cache_reset": (None, [_vp]),
    "vfkv_cache_k_ptr": (_vp, [_vp]),
    "vfkv_cache_v_ptr": (_vp, [_vp]),
    "vfkv_cache_dtype": (_u32, [_vp]),
    "vfkv_cache_bytes_per_buffer": (_u64, [_vp]),
    "vfkv_cache_head_dim_for": (_u32, [_vp, _u32]),
    "vfkv_cache_kv_heads_for": (_u32, [_vp, _u32]),
    "vfkv_cache_layer_offset_elems": (_u64, [_vp, _u32]),
    "vfkv_cache_pos_offset_bytes": (_u64, [_vp, _u32, _u32]),
    "vfkv_cache_row_bytes": (_u64, [_vp, _u32]),
    "vfkv_cache_layer_offset_bytes": (_u64, [_vp, _u32]),
    "vfkv_cache_layer_size_bytes": (_u64, [_vp, _u32]),
    "vfkv_kv_bytes_per_token": (_u64, [_u32, _u32, _u32, _u32p, _u32p, _u64]),
    "vfkv_guard_kv_precision": (C.c_int, [C.c_int, _u32, C.c_int]),
    "vfkv_kv_start_decode": (_u32, [_u32, _u32]),
    "vfkv_kv_start_batch": (_u32, [_u32, _u32, _u32]),
    "vfkv_kv_read_layer": (_u32, [_u32p, _u32, _u32]),
    "vfkv_build_kv_sources": (None, [C.POINTER(C.c_uint8), _u32, _u32, _u32, _u32p]),
    "vfkv_prefix_reuse_start": (_u32, [_u32p, _u32, _u32p, _u32]),
    "vfkv_store_fp8": (C.c_int, [_vp, _vp, _u32, _u64, _vp]),
    "vfkv_copy_fp16": (C.c_int, [_vp, _vp, _u32, _u64, _vp]),
    "vfkv_fp8_to_f16": (C.c_int, [_vp, _vp, _u64, _vp]),
    "vfkv_kv_write": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _vp]),
    "vfkv_rms_norm_mul_rope": (C.c_int, [_vp, _vp, _vp, _u32, _u32, _u32, _vp, _u32, _vp, C.POINTER(RopeParams), _vp]),
    "vfkv_qk_rope_kv_write": (C.c_int, [_vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                        C.POINTER(RopeParams), _vp, _vp]),
    "vfkv_k_rope_kv_write": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, C.POINTER(RopeParams), _vp, _vp]),
    "vfkv_flash_attn_split": (C.c_int, [_vp, _vp, _vp, _u32, _vp, _vp, _vp, C.POINTER(SplitParams), _u32, _f, _vp]),
    "vfkv_flash_attn_split_interleaved": (C.c_int, [_vp, _vp, _vp, _u32, _vp, _vp, _vp, C.POINTER(SplitParams), _u32, _f, _vp]),
    "vfkv_flash_attn_reduce": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp]),
    "vfkv_workspace_create": (C.c_int, [_u32, _u32, _u32, C.POINTER(_vp)]),
    "vfkv_workspace_destroy": (None, [_vp]),
    "vfkv_kv_write_decode_attention": (C.c_int, [_vp, _u32, _u32, _vp, _vp, _vp, _vp, _u32, _u32, _f, _f, _vp, _vp]),
    "vfkv_qk_rope_kv_write_decode_attention": (C.c_int, [_vp, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _f, _f,
                                                        _vp, _vp]),
    "vfkv_decode_tile_for": (_u32, [_u32, _u32, _u32, _u32, _u32]),
    "vfkv_decode_attention": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _f, _f, _vp, _vp]),
    "vfkv_decode_attention_static": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _f, _f, _vp]),
    "vfkv_flash_attn_batch": (C.c_int, [_vp, _vp, _vp, _u32, _vp, C.POINTER(BatchParams), _f, _vp]),
    "vfkv_flash_attn_batch_opt": (C.c_int, [_vp, _vp, _vp, _u32, _vp, C.POINTER(BatchParams), _f, _u32, _vp]),
    "vfkv_prefill_attention_opt": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _u32, _f, _f, _u32, _vp, _vp]),
    "vfkv_prefill_attention": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _u32, _f, _f, _vp]),
    "vfkv_prefill_attention_ws": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _u32, _f, _f, _vp, _vp]),
    "vfkv_sigmoid_mul": (C.c_int, [C.POINTER(Gate), _vp, _u32, _vp]),
    "vfkv_decode_attention_gated": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _u32, _u32, _f, _f, C.POINTER(Gate),
                                              _vp, _vp]),
    "vfkv_prefill_attention_gated": (C.c_int, [_vp, _u32, _u32, _u32, _vp, _vp, _u32, _u32, _u32, _f, _f, C.POINTER(Gate), _vp]),
}

_lib = None


def lib_path() -> str:
    return _SO


def lib() -> C.CDLL:
    """Loads the built library; raises if it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise ImportError(f"{_SO} is missing: build it with `make -C vulkanforge_amd/csrc` "
                              "(or `python -c 'import __graft_entry__ as g; g.build()'`)")
        # Callers hand in PyTorch device memory and streams, so the library must bind to the HIP
        # runtime PyTorch has loaded (same SONAME); importing torch first guarantees there is only
        # one runtime in the process.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(_SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status: int) -> None:
    if status != OK:
        raise VfkvError(status, lib().vfkv_last_error().decode("utf-8", "replace"))
