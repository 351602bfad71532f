"""Attention layer over a block-paged KV cache: store, then decode.

Host-side mirror of ``layers/attention.py`` of the reference for the decode
phase: ``store_kv_to_cache`` (:42-77) and ``Attention`` (:282-480) keep their
names, argument order and return shapes, for the decode phase and for the
prefill phase (:331-364).  Everything runs on the HIP library only; there is no
alternate dispatch.

Differences a caller can observe, both deliberate:
* the cache is updated in place and the very same tensors are returned (the
  reference returns new arrays that alias the donated inputs);
* a negative slot stores nothing (the reference's docstring, :57-58; its code
  writes row 0 instead).
"""
from __future__ import annotations

import torch

from .. import _lib
from ..utils.context import AttentionContext
from .paged_attention import paged_attention
from .prefill_attention import paged_prefill_attention, variable_length_attention_prefill

__all__ = ["store_kv_to_cache", "Attention"]

_DTYPE_CODE = {torch.bfloat16: _lib.NVJ_DTYPE_BF16, torch.float32: _lib.NVJ_DTYPE_F32,
               torch.float16: _lib.NVJ_DTYPE_F16}
_CACHE_DTYPES = (torch.bfloat16, torch.float16)


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _raw_stream(device_index: int) -> int:
    """The current HIP stream of a device as an integer handle."""
    try:
        return torch._C._cuda_getCurrentRawStream(device_index)
    except AttributeError:      # a torch without the raw accessor
        return torch.cuda.current_stream(device_index).cuda_stream


# the current device without the bookkeeping of torch.cuda.current_device()
_current_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device
_store_launch = None    # the library's entry point, looked up at the first call


# What a call signature (shapes, dtypes, devices of the five tensors) was validated
# to: the integer arguments of the launch.  Validation is by far the larger part of
# an eager call of this 3-microsecond kernel, so it runs once per signature.
_store_plans: dict = {}


def _plan_store(key, value, k_cache, v_cache, slot_mapping):
    for name, t in (("key", key), ("value", value), ("k_cache", k_cache),
                    ("v_cache", v_cache), ("slot_mapping", slot_mapping)):
        _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
        _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                            "the KV-cache store has no CPU implementation")
        _require(t.device == key.device, f"{name} is on {t.device}, key on {key.device}")
    _require(key.dim() == 3 and value.shape == key.shape,
             "key and value must both be [num_tokens, num_kv_heads, head_dim]")
    _require(key.dtype in _DTYPE_CODE, f"key dtype {key.dtype} not supported")
    _require(value.dtype in _DTYPE_CODE, f"value dtype {value.dtype} not supported")
    _require(k_cache.dtype in _CACHE_DTYPES and v_cache.dtype == k_cache.dtype,
             "caches must both be bf16 or both be float16")
    for name, t in (("key", key), ("value", value)):
        _require(t.dtype in (k_cache.dtype, torch.float32),
                 f"{name} must be {k_cache.dtype} (the cache dtype) or float32, got {t.dtype}")
    _require(k_cache.shape == v_cache.shape and k_cache.dim() in (3, 4),
             "caches must have equal 3-D or 4-D shapes")
    num_tokens, num_kv_heads, head_dim = key.shape
    _require(tuple(k_cache.shape[-2:]) == (num_kv_heads, head_dim),
             f"cache rows {tuple(k_cache.shape[-2:])} != key rows {(num_kv_heads, head_dim)}")
    _require(slot_mapping.dtype == torch.int32 and slot_mapping.shape == (num_tokens,),
             "slot_mapping must be int32 [num_tokens]")
    num_slots = k_cache.numel() // (num_kv_heads * head_dim)
    return (key.device.index, num_tokens, num_kv_heads, head_dim, num_slots,
            _DTYPE_CODE[key.dtype], _DTYPE_CODE[value.dtype], _DTYPE_CODE[k_cache.dtype])


def store_kv_to_cache(key, value, k_cache, v_cache, slot_mapping):
    """Scatter new K/V rows into the paged cache through ``slot_mapping``.

    key, value   [num_tokens, num_kv_heads, head_dim], the cache dtype or float32
                 (float32 rows are rounded to nearest even, as ``astype`` does)
    k_cache, v_cache
                 [num_slots, num_kv_heads, head_dim] bf16 or float16, or the 4-D
                 [num_blocks, block_size, num_kv_heads, head_dim] view of the
                 same memory
    slot_mapping [num_tokens] int32; ``slot < 0`` skips the token, ``slot >=
                 num_slots`` drops it

    Returns ``(k_cache, v_cache)``: the tensors passed in, updated in place.
    """
    try:
        sig = (key.shape, key.dtype, key.device, value.shape, value.dtype, value.device,
               k_cache.shape, k_cache.dtype, k_cache.device, v_cache.shape, v_cache.dtype,
               v_cache.device, slot_mapping.shape, slot_mapping.dtype, slot_mapping.device)
    except AttributeError as e:
        raise ValueError("store_kv_to_cache takes torch tensors") from e
    plan = _store_plans.get(sig)
    if plan is None:
        plan = _plan_store(key, value, k_cache, v_cache, slot_mapping)
        if len(_store_plans) < 256:
            _store_plans[sig] = plan
    # layout is a property of the tensor, not of the signature
    if not (key.is_contiguous() and value.is_contiguous() and k_cache.is_contiguous()
            and v_cache.is_contiguous() and slot_mapping.is_contiguous()):
        raise ValueError("key, value, k_cache, v_cache and slot_mapping must be contiguous")
    dev, num_tokens, num_kv_heads, head_dim, num_slots, kd, vd, cd = plan
    global _store_launch
    launch = _store_launch
    if launch is None:
        launch = _store_launch = _lib.load().nvj_store_kvcache_launch
    if _current_device() == dev:
        code = launch(_raw_stream(dev), key.data_ptr(), value.data_ptr(), k_cache.data_ptr(),
                      v_cache.data_ptr(), slot_mapping.data_ptr(), num_tokens, num_kv_heads,
                      head_dim, num_slots, kd, vd, cd)
    else:
        with torch.cuda.device(dev):
            code = launch(_raw_stream(dev), key.data_ptr(), value.data_ptr(), k_cache.data_ptr(),
                          v_cache.data_ptr(), slot_mapping.data_ptr(), num_tokens, num_kv_heads,
                          head_dim, num_slots, kd, vd, cd)
    if code != 0:
        _lib.check(code, "nvj_store_kvcache_launch")
    return k_cache, v_cache


class Attention:
    """Multi-head attention with a paged KV cache, decode phase.

    Same constructor and call contract as the reference's ``Attention``
    (``layers/attention.py:307-329, 436-480``): ``set_kv_cache`` hands over the
    per-layer ``[num_blocks, block_size, num_kv_heads, head_dim]`` bf16 caches;
    ``__call__(q, k, v, context)`` first stores the new K/V rows, then attends
    over the cache (the new row included: ``context_lens`` already counts it).
    """

    def __init__(self, num_heads: int, head_dim: int, scale: float, num_kv_heads: int,
                 block_size: int = 256):
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.block_size = block_size
        self.k_cache = None
        self.v_cache = None
        # optional caller-owned split workspace (a DecodeWorkspace, or a uint8
        # device tensor) shared by the calls of one stream; None = a fresh one per call
        self.workspace = None

    def set_kv_cache(self, k_cache, v_cache):
        self.k_cache = k_cache
        self.v_cache = v_cache

    def _prefill_attention(self, q, k, v, context: AttentionContext):
        """Variable-length causal attention over the packed prompt rows
        (layers/attention.py:331-364)."""
        dt = self.k_cache.dtype           # the model dtype: bf16 or float16
        if context.block_tables is not None:
            # prompt rows behind a cached prefix: the reference's filler sets
            # block_tables exactly then (engine/model_runner.py:309-312); keys and
            # values, the rows just stored included, come from the paged cache
            k_cache, v_cache = self.k_cache, self.v_cache
            if k_cache.dim() == 3:
                shape = (-1, self.block_size, self.num_kv_heads, self.head_dim)
                k_cache, v_cache = k_cache.view(shape), v_cache.view(shape)
            return paged_prefill_attention(q.to(dt).contiguous(), k_cache, v_cache,
                                           context.block_tables, context.cu_seqlens_q,
                                           context.cu_seqlens_k, self.scale)
        return variable_length_attention_prefill(
            q.to(dt).contiguous(), k.to(dt).contiguous(), v.to(dt).contiguous(),
            context.cu_seqlens_q, context.cu_seqlens_k, context.max_seqlen_q,
            context.max_seqlen_k, self.num_heads, self.num_kv_heads, self.scale)

    def _decode_attention(self, q, context: AttentionContext):
        q = q.to(self.k_cache.dtype)      # layers/attention.py:386-387
        return paged_attention(q, self.k_cache, self.v_cache, context.block_tables,
                               context.context_lens, self.scale, self.block_size,
                               chunk=context.decode_split, workspace=self.workspace)

    def __call__(self, q, k, v, context: AttentionContext):
        if self.k_cache is None or self.v_cache is None:
            raise RuntimeError("set_kv_cache() must be called before the first decode step")
        store_kv_to_cache(k, v, self.k_cache, self.v_cache, context.slot_mapping)
        if context.is_prefill:
            return self._prefill_attention(q, k, v, context)
        return self._decode_attention(q, context)
