"""MI355X-native ring / Ulysses attention hot path with the reference's entry points."""
from . import _lib
from .attention import attn_fwd, attn_delta, attn_bwd_accumulate, attn_plan, cast_to_bf16, block_attention
from .ring_attention import LocalRing, RingKVGrads, ring_attention_kernel, ring_attention_with_lse
from .parallel_cp import SeqAllToAll, _all_to_all, ContextParallelAttention, LocalCPGroup
from . import layers
from .layers import precompute_freqs_cis, apply_rotary_emb, rope_table, rope_one
from .model import Attention, repeat_kv

__all__ = ["attn_fwd", "attn_delta", "attn_bwd_accumulate", "attn_plan", "cast_to_bf16", "block_attention",
           "LocalRing", "RingKVGrads", "ring_attention_kernel", "ring_attention_with_lse",
           "SeqAllToAll", "_all_to_all", "ContextParallelAttention", "LocalCPGroup",
           "precompute_freqs_cis", "apply_rotary_emb", "rope_table", "rope_one", "Attention", "repeat_kv"]
