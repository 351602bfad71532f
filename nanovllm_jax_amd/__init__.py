"""MI355X-native paged-decode path: KV-cache store + split-K paged decode attention.

Importing the package does not load the HIP library; the first call does, and
fails loudly if it has not been built.
"""
from .layers.attention import Attention, store_kv_to_cache
from .layers.paged_attention import paged_attention
from .layers.prefill_attention import paged_prefill_attention, variable_length_attention_prefill
from .utils.context import AttentionContext, create_decode_context, create_prefill_context

__all__ = ["Attention", "store_kv_to_cache", "paged_attention",
           "variable_length_attention_prefill", "paged_prefill_attention", "AttentionContext", "create_decode_context",
           "create_prefill_context"]
