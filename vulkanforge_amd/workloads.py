"""The benchmark configurations of this path (geometry and synthetic-input recipes) and their
algorithmic work, so tests and the benchmark agree on shapes and byte counts."""
from __future__ import annotations

from dataclasses import dataclass

from .kv_cache import KvDtype


@dataclass(frozen=True)
class DecodeWorkload:
    name: str
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    context: int            # keys visible to the decode query (after the append, if any)
    dtype: KvDtype
    append: bool            # append one token per layer inside the step
    softcap: float = 0.0
    window: int = 0         # sliding window of the sliding layers (0 = none)
    sliding_pattern: int = 0  # k sliding layers followed by one global layer, repeated
    gated: bool = False     # the output is multiplied by sigmoid(gate), the gate sitting behind Q (Qwen3.6 full attention)
    rope: bool = False      # the step also RMS-normalises and rotates the token's Q and K rows (QNormRope + KNormRope + KvWrite + attention)

    def layer_window(self, layer: int) -> int:
        if not self.window or not self.sliding_pattern:
            return 0
        return 0 if (layer % (self.sliding_pattern + 1)) == self.sliding_pattern else self.window

    def kv_bytes_layer(self, layer: int) -> int:
        win = self.layer_window(layer)
        keys = min(self.context, win) if win else self.context
        return 2 * keys * self.n_kv_heads * self.head_dim * self.dtype.element_size()

    def kv_bytes_step(self) -> int:
        """Algorithmic KV bytes one decode step must read (K and V of every visible key once)."""
        return sum(self.kv_bytes_layer(i) for i in range(self.n_layers))


@dataclass(frozen=True)
class PrefillWorkload:
    name: str
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    base_pos: int
    m: int
    dtype: KvDtype
    workspace: bool = False   # attention through vfkv_prefill_attention_ws (key chunks over workgroups)
    gated: bool = False       # the output is multiplied by sigmoid(gate), per (token, head) the gate follows Q (Qwen3.6)

    def pairs_per_head(self) -> int:
        return sum(self.base_pos + i + 1 for i in range(self.m))

    def flops_layer(self) -> int:
        """4 * head_dim flop per (query, key) pair and head, causal-exact."""
        return self.pairs_per_head() * self.n_heads * 4 * self.head_dim

    def kv_bytes_layer(self) -> int:
        return 2 * (self.base_pos + self.m) * self.n_kv_heads * self.head_dim * self.dtype.element_size()


DECODE = {
    "decode_f16_2k_1layer": DecodeWorkload("decode_f16_2k_1layer", 1, 32, 8, 128, 2049, KvDtype.F16, True),
    "decode_fp8_8k_32layers": DecodeWorkload("decode_fp8_8k_32layers", 32, 32, 8, 128, 8193, KvDtype.F8, True),
    "decode_fp8_32k_32layers": DecodeWorkload("decode_fp8_32k_32layers", 32, 32, 8, 128, 32768, KvDtype.F8, False),
    # configuration 2 with the Q / K norm + RoPE of the token in front of the append, as a Qwen3-style decode layer issues it
    # (QNormRope, KNormRope, KvWrite, attention: executor/attention.rs:360-625); not a reference configuration
    "decode_fp8_8k_32layers_rope": DecodeWorkload("decode_fp8_8k_32layers_rope", 32, 32, 8, 128, 8193, KvDtype.F8, True, rope=True),
    # configuration 2 without the append (what the append inside the attention launch costs; not a reference configuration)
    "decode_fp8_8k_32layers_no_append": DecodeWorkload("decode_fp8_8k_32layers_no_append", 32, 32, 8, 128, 8193, KvDtype.F8, False),
    "decode_fp8_8192_32layers_no_append": DecodeWorkload("decode_fp8_8192_32layers_no_append", 32, 32, 8, 128, 8192, KvDtype.F8, False),
    # the headline geometry over an F16 cache (not one of the reference configurations; used to tune the F16 variant)
    "decode_f16_32k_32layers": DecodeWorkload("decode_f16_32k_32layers", 32, 32, 8, 128, 32768, KvDtype.F16, False),
    # the headline geometry with the gated output of the Qwen3.6 full-attention layers (not a reference configuration)
    "decode_fp8_32k_32layers_gated": DecodeWorkload("decode_fp8_32k_32layers_gated", 32, 32, 8, 128, 32768, KvDtype.F8, False,
                                                    gated=True),
    # the configuration-2 geometry over an F32 cache (the reference's VULKANFORGE_FP16_KV=0 mode; not a reference configuration):
    # the same bytes per layer as the headline workload
    "decode_f32_8k_32layers": DecodeWorkload("decode_f32_8k_32layers", 32, 32, 8, 128, 8193, KvDtype.F32, True),
    # Phi-3-mini geometry (32 heads, no grouping, head_dim 96, F16 cache; not a reference configuration): a head width between
    # the tiled ones, served by the worker for 128 with its tail masked off
    "decode_f16_hd96_4k_32layers": DecodeWorkload("decode_f16_hd96_4k_32layers", 32, 32, 32, 96, 4097, KvDtype.F16, True),
    "decode_f16_hd256_sliding_12layers": DecodeWorkload("decode_f16_hd256_sliding_12layers", 12, 16, 8, 256, 16384,
                                                        KvDtype.F16, False, softcap=50.0, window=4096,
                                                        sliding_pattern=5),
}
PREFILL = {
    "prefill_fp8_512x4608_32layers": PrefillWorkload("prefill_fp8_512x4608_32layers", 32, 32, 8, 128, 4096, 512,
                                                     KvDtype.F8),
    # the same with the gated output of the Qwen3.6 full-attention layers (not a reference configuration)
    "prefill_fp8_512x4608_32layers_gated": PrefillWorkload("prefill_fp8_512x4608_32layers_gated", 32, 32, 8, 128, 4096,
                                                           512, KvDtype.F8, gated=True),
    # Gemma-style geometry (16 query heads, 8 KV heads, head_dim 256): not a reference configuration
    "prefill_f16_hd256_512x4608_12layers": PrefillWorkload("prefill_f16_hd256_512x4608_12layers", 12, 16, 8, 256, 4096,
                                                           512, KvDtype.F16),
    "prefill_fp8_hd256_512x4608_12layers": PrefillWorkload("prefill_fp8_hd256_512x4608_12layers", 12, 16, 8, 256, 4096,
                                                           512, KvDtype.F8),
    # Phi-3-mini geometry (head_dim 96, F16 cache; not a reference configuration): the padded form of the f16 kernel
    "prefill_f16_hd96_512x4608_32layers": PrefillWorkload("prefill_f16_hd96_512x4608_32layers", 32, 32, 32, 96, 4096, 512,
                                                          KvDtype.F16),
    # the suffix of a request that reuses its prefix: 64 new tokens over 16 k resident rows, with and without the workspace
    "prefill_fp8_suffix64_over_16k_32layers": PrefillWorkload("prefill_fp8_suffix64_over_16k_32layers", 32, 32, 8, 128,
                                                              16384, 64, KvDtype.F8, workspace=True),
    "prefill_fp8_suffix64_over_16k_32layers_plain": PrefillWorkload("prefill_fp8_suffix64_over_16k_32layers_plain", 32, 32,
                                                                    8, 128, 16384, 64, KvDtype.F8),
    # the headline prefill geometry over an F32 cache (the reference's VULKANFORGE_FP16_KV=0 mode), 4 layers
    "prefill_f32_512x4608_4layers": PrefillWorkload("prefill_f32_512x4608_4layers", 4, 32, 8, 128, 4096, 512, KvDtype.F32),
    # the headline prefill geometry over an F16 cache (not a reference configuration; used to tune the F16 variant)
    "prefill_f16_512x4608_32layers": PrefillWorkload("prefill_f16_512x4608_32layers", 32, 32, 8, 128, 4096, 512,
                                                     KvDtype.F16),
}



@dataclass(frozen=True)
class RopeAppendWorkload:
    """K RMS-norm * weight + RoPE + append of K and V, one launch per layer (the step in front of attention)."""
    name: str
    n_layers: int
    n_kv_heads: int
    head_dim: int
    n_tokens: int           # rows appended per layer and step (1 = decode, chunk length = prefill)
    base_pos: int
    dtype: KvDtype

    def bytes_step(self) -> int:
        """Algorithmic bytes: K and V rows read as f32, written once in the cache dtype."""
        return self.n_layers * 2 * self.n_tokens * self.n_kv_heads * self.head_dim * (4 + self.dtype.element_size())


ROPE_APPEND = {
    "k_rope_append_fp8_decode_32layers": RopeAppendWorkload("k_rope_append_fp8_decode_32layers", 32, 8, 128, 1, 8192,
                                                            KvDtype.F8),
    "k_rope_append_fp8_prefill_512_32layers": RopeAppendWorkload("k_rope_append_fp8_prefill_512_32layers", 32, 8, 128,
                                                                 512, 4096, KvDtype.F8),
}

assert DECODE["decode_f16_2k_1layer"].kv_bytes_step() == 8_392_704
assert DECODE["decode_fp8_8k_32layers"].kv_bytes_step() == 536_936_448
assert DECODE["decode_fp8_32k_32layers"].kv_bytes_step() == 2_147_483_648
assert DECODE["decode_f16_hd256_sliding_12layers"].kv_bytes_step() == 603_979_776
assert PREFILL["prefill_fp8_512x4608_32layers"].flops_layer() == 36_511_416_320
