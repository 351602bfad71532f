"""Fused QK-RMSNorm + rotary embedding + KV-cache store.

Host-side entry to ``nvj_qk_norm_rope_store_launch``: one launch for what the
reference runs as separate XLA ops between the fused QKV projection and the
attention call (``models/qwen3.py:157-166``: ``q_norm``/``k_norm``,
``rotary_emb``, then ``store_kv_to_cache`` inside ``Attention.__call__``,
``layers/attention.py:457-475``).  ``build_cos_sin_cache`` restates the table of
``RotaryEmbedding.__init__`` (``layers/rotary_embedding.py:60-76``).
"""
from __future__ import annotations

import torch

from .. import _lib

__all__ = ["qk_norm_rope_store", "build_cos_sin_cache"]


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def build_cos_sin_cache(head_dim: int, max_position: int, base: float, device) -> torch.Tensor:
    """``[max_position, head_dim]`` float32: cos of the head_dim/2 frequencies,
    then sin (the reference's cache without its singleton head axis)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(max_position, dtype=torch.float32), inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(device)


def qk_norm_rope_store(qkv, positions, cos_sin_cache, q_norm_weight, k_norm_weight, eps,
                       k_cache, v_cache, slot_mapping, num_heads, num_kv_heads, head_dim,
                       q_out=None):
    """Normalise and rotate q and k, write q out and K/V into the paged cache.

    qkv            [num_tokens, (num_heads + 2 * num_kv_heads) * head_dim] bf16
                   (rows may be strided)
    positions      [num_tokens] int32
    cos_sin_cache  [max_position, head_dim] float32
    q_norm_weight, k_norm_weight  [head_dim] float32, or both None
    k_cache, v_cache  bf16 caches (3-D flat or 4-D paged view), updated in place
    slot_mapping   [num_tokens] int32 (``< 0`` skips, ``>= num_slots`` drops)

    Returns q ``[num_tokens, num_heads, head_dim]`` bf16, ready for
    ``paged_attention``.
    """
    lib = _lib.load()
    tensors = [("qkv", qkv), ("positions", positions), ("cos_sin_cache", cos_sin_cache),
               ("k_cache", k_cache), ("v_cache", v_cache), ("slot_mapping", slot_mapping)]
    if q_norm_weight is not None or k_norm_weight is not None:
        _require(q_norm_weight is not None and k_norm_weight is not None,
                 "q_norm_weight and k_norm_weight must both be given or both be None")
        tensors += [("q_norm_weight", q_norm_weight), ("k_norm_weight", k_norm_weight)]
    for name, t in tensors:
        _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
        _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                            "this op has no CPU implementation")
        _require(t.device == qkv.device, f"{name} is on {t.device}, qkv on {qkv.device}")
    heads_total = num_heads + 2 * num_kv_heads
    _require(qkv.dtype == torch.bfloat16 and qkv.dim() == 2 and qkv.stride(1) == 1
             and qkv.shape[1] == heads_total * head_dim,
             f"qkv must be bf16 [num_tokens, {heads_total * head_dim}] with unit inner stride")
    num_tokens = qkv.shape[0]
    row_stride = qkv.stride(0) if num_tokens > 1 else qkv.shape[1]
    _require(positions.dtype == torch.int32 and positions.shape == (num_tokens,)
             and positions.is_contiguous(), "positions must be contiguous int32 [num_tokens]")
    _require(slot_mapping.dtype == torch.int32 and slot_mapping.shape == (num_tokens,)
             and slot_mapping.is_contiguous(), "slot_mapping must be contiguous int32 [num_tokens]")
    _require(cos_sin_cache.dtype == torch.float32 and cos_sin_cache.dim() == 2
             and cos_sin_cache.shape[1] == head_dim and cos_sin_cache.is_contiguous(),
             "cos_sin_cache must be contiguous float32 [max_position, head_dim]")
    for name, wt in (("q_norm_weight", q_norm_weight), ("k_norm_weight", k_norm_weight)):
        if wt is not None:
            _require(wt.dtype == torch.float32 and wt.shape == (head_dim,) and wt.is_contiguous(),
                     f"{name} must be contiguous float32 [head_dim]")
    _require(k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
             and k_cache.shape == v_cache.shape and k_cache.is_contiguous()
             and v_cache.is_contiguous(), "caches must be contiguous bf16 of equal shape")
    _require(tuple(k_cache.shape[-2:]) == (num_kv_heads, head_dim), "cache row shape mismatch")
    num_slots = k_cache.numel() // (num_kv_heads * head_dim)
    if q_out is None:
        q_out = torch.empty((num_tokens, num_heads, head_dim), dtype=torch.bfloat16,
                            device=qkv.device)
    else:
        _require(q_out.is_cuda and q_out.dtype == torch.bfloat16 and q_out.is_contiguous()
                 and q_out.shape == (num_tokens, num_heads, head_dim), "bad q_out")
    with torch.cuda.device(qkv.device):
        stream = torch.cuda.current_stream(qkv.device).cuda_stream
        code = lib.nvj_qk_norm_rope_store_launch(
            stream, qkv.data_ptr(), row_stride, positions.data_ptr(), cos_sin_cache.data_ptr(),
            cos_sin_cache.shape[0],
            q_norm_weight.data_ptr() if q_norm_weight is not None else None,
            k_norm_weight.data_ptr() if k_norm_weight is not None else None, float(eps),
            slot_mapping.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), q_out.data_ptr(),
            num_tokens, num_heads, num_kv_heads, head_dim, num_slots)
    _lib.check(code, "nvj_qk_norm_rope_store_launch")
    return q_out
