"""Variable-length causal prefill attention entry point.

Host-side mirror of ``variable_length_attention_prefill``
(``layers/attention.py:135-279`` of the reference): same argument list and
result, one dispatch target: ``nvj_prefill_attention_launch``.  The static
``max_seqlen_q / max_seqlen_k / batch_size`` arguments are accepted for
signature compatibility; the HIP kernel pads nothing and does not need them.
"""
from __future__ import annotations

import torch

from .. import _lib

__all__ = ["variable_length_attention_prefill", "paged_prefill_attention"]

_DTYPE_CODE = {torch.bfloat16: _lib.NVJ_DTYPE_BF16, torch.float16: _lib.NVJ_DTYPE_F16}


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def variable_length_attention_prefill(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q=0,
                                      max_seqlen_k=0, num_heads=None, num_kv_heads=None,
                                      scale=None, batch_size=None, *, out=None):
    """q [total_tokens, num_heads, head_dim], k/v [total_k_tokens, num_kv_heads,
    head_dim] packed rows, all bf16 or all float16; cu_seqlens_q / cu_seqlens_k
    [batch + 1] int32 on the device.  Query position p of a sequence attends key
    positions <= p of the same sequence.  Returns [total_tokens, num_heads,
    head_dim] in q's dtype."""
    lib = _lib.load()
    _require(isinstance(q, torch.Tensor) and q.dtype in _DTYPE_CODE,
             "q must be a bf16 or float16 torch.Tensor")
    for name, t, dt, nd in (("q", q, q.dtype, 3), ("k", k, q.dtype, 3), ("v", v, q.dtype, 3),
                            ("cu_seqlens_q", cu_seqlens_q, torch.int32, 1),
                            ("cu_seqlens_k", cu_seqlens_k, torch.int32, 1)):
        _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
        _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                            "prefill attention has no CPU implementation")
        _require(t.dtype == dt and t.dim() == nd and t.is_contiguous(),
                 f"{name} must be contiguous {dt} with {nd} dims")
        _require(t.device == q.device, f"{name} is on {t.device}, q on {q.device}")
    total, hq, d = q.shape
    _require(k.shape == v.shape and k.shape[2] == d, "k and v must share [tokens, kv_heads, head_dim]")
    hkv = k.shape[1]
    _require(num_heads in (None, hq) and num_kv_heads in (None, hkv), "head counts disagree with q/k")
    _require(hq % hkv == 0, "num_heads must be a multiple of num_kv_heads")
    batch = cu_seqlens_q.shape[0] - 1
    _require(batch >= 0 and cu_seqlens_k.shape[0] == batch + 1, "cu_seqlens shapes disagree")
    _require(batch_size in (None, batch), "batch_size disagrees with cu_seqlens")
    if scale is None:
        scale = d ** -0.5
    if out is None:
        out = torch.empty_like(q)
    else:
        _require(out.is_cuda and out.dtype == q.dtype and out.shape == q.shape
                 and out.is_contiguous(), "out must match q")
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        code = lib.nvj_prefill_attention_launch(
            stream, q.data_ptr(), k.data_ptr(), v.data_ptr(), cu_seqlens_q.data_ptr(),
            cu_seqlens_k.data_ptr(), out.data_ptr(), total, batch, hq, hkv, d, float(scale),
            _DTYPE_CODE[q.dtype])
    _lib.check(code, "nvj_prefill_attention_launch")
    return out


def paged_prefill_attention(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k,
                            scale=None, *, out=None):
    """Prefill attention behind a cached prefix: the keys and values of every
    sequence (``cu_seqlens_k[i+1] - cu_seqlens_k[i]`` of them, cached and new
    together) are read from the block-paged cache through ``block_tables``; the
    query rows of a sequence are its last ``len_q`` positions.  This is the call
    the reference's prefill context describes when ``cu_seqlens_k >
    cu_seqlens_q`` (``engine/model_runner.py:286-312``); run it after the new
    rows have been stored.

    q [total_tokens, num_heads, head_dim] bf16 or float16; k_cache, v_cache
    [num_blocks, block_size, num_kv_heads, head_dim] of the same dtype;
    block_tables [batch, max_blocks] int32; cu_seqlens_* [batch + 1] int32, all on
    the GPU.  Returns [total_tokens, num_heads, head_dim] in q's dtype."""
    lib = _lib.load()
    _require(isinstance(q, torch.Tensor) and q.dtype in _DTYPE_CODE,
             "q must be a bf16 or float16 torch.Tensor")
    for name, t, dt, nd in (("q", q, q.dtype, 3), ("k_cache", k_cache, q.dtype, 4),
                            ("v_cache", v_cache, q.dtype, 4),
                            ("block_tables", block_tables, torch.int32, 2),
                            ("cu_seqlens_q", cu_seqlens_q, torch.int32, 1),
                            ("cu_seqlens_k", cu_seqlens_k, torch.int32, 1)):
        _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
        _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                            "prefill attention has no CPU implementation")
        _require(t.dtype == dt and t.dim() == nd and t.is_contiguous(),
                 f"{name} must be contiguous {dt} with {nd} dims")
        _require(t.device == q.device, f"{name} is on {t.device}, q on {q.device}")
    total, hq, d = q.shape
    num_blocks, bs, hkv, d2 = k_cache.shape
    _require(v_cache.shape == k_cache.shape and d2 == d, "caches must share one shape and q's head_dim")
    _require(hq % hkv == 0, "num_heads must be a multiple of num_kv_heads")
    batch = cu_seqlens_q.shape[0] - 1
    _require(batch >= 0 and cu_seqlens_k.shape[0] == batch + 1 and block_tables.shape[0] == batch,
             "cu_seqlens / block_tables shapes disagree")
    if scale is None:
        scale = d ** -0.5
    if out is None:
        out = torch.empty_like(q)
    else:
        _require(out.is_cuda and out.dtype == q.dtype and out.shape == q.shape
                 and out.is_contiguous(), "out must match q")
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        code = lib.nvj_paged_prefill_attention_launch(
            stream, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
            cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), out.data_ptr(), total, batch, hq,
            hkv, d, bs, block_tables.shape[1], num_blocks, float(scale), _DTYPE_CODE[q.dtype])
    _lib.check(code, "nvj_paged_prefill_attention_launch")
    return out
