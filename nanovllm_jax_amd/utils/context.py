"""Attention metadata carrier for the decode path.

Host-side mirror of ``utils/context.py`` of the reference (``AttentionContext``
:35-81, ``create_decode_context`` :169-190): same field names and meaning, with
device tensors in place of JAX arrays, for the decode phase and (``create_prefill_context``)
the prefill phase.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

__all__ = ["AttentionContext", "create_decode_context", "create_prefill_context"]


def _bucket_to_power_of_2(value: int, min_bucket: int = 16, max_bucket: int = 8192) -> int:
    """``value`` rounded up to a power of two and clamped into [min_bucket,
    max_bucket]: what the reference's helper of this name returns
    (``utils/context.py:18-32``; it buckets the static max lengths to limit
    recompilation).  The HIP kernels never read these fields; the contexts carry
    them so that code written against the reference sees the same values."""
    return max(min_bucket, min(max_bucket, 1 << max(int(value) - 1, 0).bit_length()))


@dataclass
class AttentionContext:
    """Metadata one attention call needs.

    is_prefill          False for decode, True for prefill.
    context_lens        [batch] int32, length of every sequence including the
                        position being decoded.
    slot_mapping        [num_tokens] int32, cache slot of every new K/V row;
                        -1 means "do not store".
    block_tables        [batch, max_blocks] int32, logical -> physical page,
                        padded with -1.
    decode_split        how the decode kernel divides the positions of the batch
                        (``chunk`` of ``paged_attention``): 0 = balanced on the
                        device from ``context_lens``; the filler, which knows
                        the lengths on the host, may ask for the whole-sequence
                        mode instead (``layers.paged_attention.choose_split``).
                        Not a field of the reference's dataclass.
    """
    is_prefill: bool = False
    cu_seqlens_q: Any = None
    cu_seqlens_k: Any = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    context_lens: Any = None
    slot_mapping: Any = None
    block_tables: Any = None
    last_token_indices: Any = None
    decode_split: int = 0


def create_decode_context(context_lens, slot_mapping, block_tables,
                          decode_split: int = 0) -> AttentionContext:
    """Context for one decode step (every token is a sequence's last token, so
    ``last_token_indices`` stays None)."""
    return AttentionContext(is_prefill=False, context_lens=context_lens,
                            slot_mapping=slot_mapping, block_tables=block_tables,
                            last_token_indices=None, decode_split=decode_split)


def create_prefill_context(cu_seqlens_q, cu_seqlens_k, max_seqlen_q: int, max_seqlen_k: int,
                           slot_mapping, block_tables=None) -> AttentionContext:
    """Context for a prefill step (``utils/context.py:129-166``):
    ``last_token_indices = cu_seqlens_q[1:] - 1``, max lengths bucketed."""
    return AttentionContext(is_prefill=True, cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k,
                            max_seqlen_q=_bucket_to_power_of_2(max_seqlen_q),
                            max_seqlen_k=_bucket_to_power_of_2(max_seqlen_k),
                            slot_mapping=slot_mapping, block_tables=block_tables,
                            last_token_indices=cu_seqlens_q[1:] - 1)
