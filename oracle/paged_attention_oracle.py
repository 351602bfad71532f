"""NumPy restatement of the reference's KV-cache store and paged decode attention.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and ``bench.py``'s ``cpu_baseline`` leg as the checker; never by the product
package, which has no CPU path.

bf16 tensors are carried as ``uint16`` bit patterns (NumPy has no bf16), fp32
tensors as ``float32``.  Every function names the reference lines it follows
(paths relative to the reference checkout).

What pins each function (see tests/test_oracle_pinning.py):

* ``f32_to_bf16_bits``          - IEEE round-to-nearest-even; cross-checked
                                  against ``torch.Tensor.to(torch.bfloat16)``.
* ``f32_to_f16_bits``           - NumPy's IEEE conversion; cross-checked against
                                  ``torch.Tensor.to(torch.float16)``.
* ``store_kv_to_cache_ref``     - brute-force per-token Python loop; untouched
                                  rows unchanged; idempotence; K/V independence.
* ``paged_decode_attention_vectorized_ref`` and ``..._per_seq``
                                - fp64 textbook softmax(qK^T)V on small shapes,
                                  ``torch.nn.functional.scaled_dot_product_attention``
                                  with ``enable_gqa`` on gathered pages,
                                  closed forms (ctx=1 -> V row, equal keys ->
                                  mean of V, ctx=0 -> zeros), permutation and
                                  padding invariance.
* ``qk_norm_rope_ref`` / ``qk_norm_rope_store_ref`` / ``build_cos_sin_cache_ref``
                                - float64 RMSNorm and rotation; closed forms
                                  (position 0 is the identity, unit weight gives
                                  unit RMS, rotation preserves each pair's norm,
                                  q.k depends on the position difference only).
                                  The fp32 summation order of the mean is this
                                  oracle's choice (the reference leaves it to
                                  XLA): PARITY UNPINNED at the level of fp32
                                  round-off of that sum.
* ``variable_length_attention_prefill_ref``
                                - fp64 brute force per (sequence, head, row);
                                  torch ``scaled_dot_product_attention`` with
                                  ``is_causal`` and ``enable_gqa``; row 0 is the
                                  first V row; packing invariance (a batch equals
                                  its sequences run one by one).  Same unpinned
                                  bf16 rounding of probabilities as the fallback.
* ``add_rms_norm_ref``          - float64 RMSNorm of the float64 sum (closed form),
                                  ``torch.nn.functional.rms_norm`` in float32; unit
                                  weight gives unit RMS; the residual output is
                                  the bf16 rounding of the exact sum.  The fp32
                                  summation order of the mean is this oracle's
                                  choice (the reference leaves it to XLA): PARITY
                                  UNPINNED at the level of fp32 round-off of that
                                  sum.
* ``silu_and_mul_ref``          - float64 ``g / (1 + exp(-g)) * u`` and torch's
                                  ``silu`` in float64; silu(0) = 0, large gates
                                  pass ``up`` through, large negative gates give 0.
                                  Evaluated in float64 and rounded once to bf16;
                                  where XLA rounds inside the reference's bf16
                                  expression is PARITY UNPINNED (at most one bf16
                                  ulp per rounding point).
* ``paged_attention_fallback_ref``
                                - the checks of the decode restatements above
                                  (float64 brute force, torch SDPA with
                                  ``enable_gqa``, ctx 0 / 1, equal keys, group
                                  mapping, page permutation, padding and garbage,
                                  one position more, out-of-range metadata), and a
                                  float64 computation that rounds the
                                  probabilities to bf16 at the same place, to one
                                  bf16 ulp, on lengths 1 to 5 and across a page
                                  boundary.  The rounding of the probabilities
                                  inside ``jax.nn.dot_product_attention``
                                  (third-party jax, not under the reference
                                  tree, ``requirements.txt`` pins ``jax>=0.4.20``)
                                  is restated from its published XLA
                                  implementation: PARITY UNPINNED at bit level
                                  for that one rounding step; it is covered by
                                  the 1e-2 tolerance, not by a vector.
"""
from __future__ import annotations

import numpy as np

__all__ = [
    "f32_to_bf16_bits",
    "bf16_bits_to_f32",
    "f32_to_f16_bits",
    "f16_bits_to_f32",
    "store_kv_to_cache_ref",
    "gather_kv_from_cache_ref",
    "paged_decode_attention_vectorized_ref",
    "paged_decode_attention_per_seq_ref",
    "paged_attention_fallback_ref",
    "textbook_attention_f64",
    "build_cos_sin_cache_ref",
    "qk_norm_rope_ref",
    "qk_norm_rope_store_ref",
    "variable_length_attention_prefill_ref",
    "textbook_prefill_f64",
    "prepare_decode_ref",
    "advance_decode_ref",
    "add_rms_norm_ref",
    "silu_and_mul_ref",
]


# ---------------------------------------------------------------------------
# bf16 <-> fp32 on bit patterns
# ---------------------------------------------------------------------------

def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern, round-to-nearest-even (what ``astype(bfloat16)``
    does in ``layers/attention.py:70-71`` and ``pallas_attention.py:238``).
    NaN stays a quiet NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounding_bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    r = ((u + rounding_bias) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    """bf16 bit pattern -> fp32 (exact)."""
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> IEEE half, round to nearest even, as uint16 bit patterns
    (NumPy's ``astype(float16)``; what ``astype(cache.dtype)`` of
    ``layers/attention.py:70-71`` does for a float16 cache)."""
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    """IEEE half bit pattern -> fp32 (exact)."""
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def _codec(dtype: str):
    """(bits -> fp32, fp32 -> bits) of a 16-bit cache dtype, "bf16" or "f16"."""
    if dtype == "bf16":
        return bf16_bits_to_f32, f32_to_bf16_bits
    if dtype == "f16":
        return f16_bits_to_f32, f32_to_f16_bits
    raise ValueError(dtype)


def _as_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Accept fp32 values or uint16 bf16 bits; return bf16 bits."""
    if x.dtype == np.uint16:
        return x
    if x.dtype == np.float32:
        return f32_to_bf16_bits(x)
    raise TypeError(f"expected float32 values or uint16 bf16 bits, got {x.dtype}")


# ---------------------------------------------------------------------------
# KV-cache store
# ---------------------------------------------------------------------------

def store_kv_to_cache_ref(key, value, k_cache, v_cache, slot_mapping,
                          negative_slots: str = "reference", dtype: str = "bf16"):
    """Restates ``store_kv_to_cache`` (``layers/attention.py:42-77``).

    key, value : [T, Hkv, D] float32 values or uint16 bits of the cache dtype
    k_cache, v_cache : [num_slots, Hkv, D] uint16 bits of the cache dtype
                 (``dtype``: "bf16" or "f16"; flattened cache,
                 ``layers/attention.py:458-463``)
    slot_mapping : [T] int32

    Returns new ``(k_cache, v_cache)``; inputs are not modified (the reference
    is functional).

    ``negative_slots``:
      "reference" - what the code does: ``safe = where(slot >= 0, slot, 0)``
                    (:64-67) then ``.at[safe].set(x, mode='drop')`` (:74-75),
                    i.e. a negative slot WRITES ROW 0; slots >= num_slots are
                    dropped.  Duplicate targets have no defined winner in XLA;
                    here the last writer wins.
      "skip"      - what the docstring (:57-58) and ``utils/context.py:57-58``
                    promise ("-1 indicates skip"): negative slots write nothing.
                    This is the contract of the HIP kernel.
    """
    if negative_slots not in ("reference", "skip"):
        raise ValueError(negative_slots)
    to_bits = _codec(dtype)[1]
    key, value = np.asarray(key), np.asarray(value)
    kb = key if key.dtype == np.uint16 else to_bits(key)          # :70  key.astype(cache.dtype)
    vb = value if value.dtype == np.uint16 else to_bits(value)    # :71
    if kb.dtype != np.uint16 or vb.dtype != np.uint16:
        raise TypeError("key / value must be float32 values or uint16 bit patterns")
    slots = np.asarray(slot_mapping, dtype=np.int64)
    k_new = np.array(k_cache, dtype=np.uint16, copy=True)
    v_new = np.array(v_cache, dtype=np.uint16, copy=True)
    num_slots = k_new.shape[0]
    valid = slots >= 0                           # :64
    if negative_slots == "reference":
        safe = np.where(valid, slots, 0)         # :67
        keep = safe < num_slots                  # mode='drop' (:74)
    else:
        safe = slots
        keep = valid & (slots < num_slots)
    idx = safe[keep]
    k_new[idx] = kb[keep]                        # :74
    v_new[idx] = vb[keep]                        # :75
    return k_new, v_new


# ---------------------------------------------------------------------------
# Paged decode attention
# ---------------------------------------------------------------------------

def gather_kv_from_cache_ref(k_cache, v_cache, block_tables, context_lens, block_size):
    """Restates ``gather_kv_from_cache`` (``layers/attention.py:80-122``):
    clip tables (:107), gather pages (:111-112), flatten to
    [B, MB*bs, Hkv, D] (:115-116), mask = pos < ctx (:119-120)."""
    bt = np.asarray(block_tables)
    B, MB = bt.shape
    S = MB * block_size
    Hkv, D = k_cache.shape[2], k_cache.shape[3]
    safe = np.clip(bt, 0, k_cache.shape[0] - 1)
    k = k_cache[safe].reshape(B, S, Hkv, D)
    v = v_cache[safe].reshape(B, S, Hkv, D)
    mask = np.arange(S)[None, :] < np.asarray(context_lens)[:, None]
    return k, v, mask


def paged_decode_attention_vectorized_ref(q, k_cache, v_cache, block_tables,
                                          context_lens, scale, block_size):
    """Literal restatement of ``paged_decode_attention_vectorized``
    (``layers/pallas_attention.py:146-238``), whole batch at once.

    q : [B, Hq, D] bf16 bits;  k_cache, v_cache : [NB, bs, Hkv, D] bf16 bits;
    block_tables : [B, MB] int32 (-1 padded);  context_lens : [B] int32.
    Returns [B, Hq, D] bf16 bits.

    Materialises [B, MB*bs, Hq, D] fp32 twice, like the reference: use
    ``paged_decode_attention_per_seq_ref`` for large shapes.
    """
    q = np.asarray(q)
    B, Hq, D = q.shape
    NB, bs, Hkv, _ = k_cache.shape
    assert bs == block_size
    MB = block_tables.shape[1]
    S = MB * block_size
    G = Hq // Hkv                                                    # :181
    safe = np.clip(np.asarray(block_tables), 0, NB - 1)             # :185
    k_flat = k_cache[safe].reshape(B, S, Hkv, D)                     # :188-192
    v_flat = v_cache[safe].reshape(B, S, Hkv, D)
    k_f32 = bf16_bits_to_f32(np.repeat(k_flat, G, axis=2))           # :197, :202
    v_f32 = bf16_bits_to_f32(np.repeat(v_flat, G, axis=2))           # :198, :203
    q_f32 = bf16_bits_to_f32(q)                                      # :201
    scale = np.float32(scale)
    # scores[b,h,s] = (q[b,h,:] . k[b,s,h,:]) * scale                  :208-214
    scores = np.einsum("bhd,bshd->bhs", q_f32, k_f32, dtype=np.float32) * scale
    mask = (np.arange(S)[None, None, :]
            < np.asarray(context_lens)[:, None, None])               # :216-217
    scores = np.where(mask, scores, np.float32(-1e9))                # :220
    smax = scores.max(axis=-1, keepdims=True)                        # :223
    e = np.exp(scores - smax, dtype=np.float32)                      # :224
    e = np.where(mask, e, np.float32(0.0))                           # :225
    ssum = e.sum(axis=-1, keepdims=True, dtype=np.float32)           # :226
    w = e / (ssum + np.float32(1e-9))                                # :227
    out = np.einsum("bhs,bshd->bhd", w, v_f32, dtype=np.float32)     # :231-236
    return f32_to_bf16_bits(out)                                     # :238


def paged_decode_attention_per_seq_ref(q, k_cache, v_cache, block_tables,
                                       context_lens, scale, block_size,
                                       return_f32: bool = False, dtype: str = "bf16"):
    """Same arithmetic as ``paged_decode_attention_vectorized_ref``
    (``layers/pallas_attention.py:146-238``), evaluated one sequence at a time
    over that sequence's own ceil(ctx/bs) pages so memory stays bounded at the
    32k-context configs.  Positions >= ctx carry weight exactly 0 in the
    reference (:225), so restricting to the live pages changes nothing but
    fp32 summation order.  ctx == 0 gives zeros (0 / (0 + 1e-9), :227).
    ``dtype`` ("bf16" or "f16") is the 16-bit type of q, the caches and the result.
    """
    q = np.asarray(q)
    B, Hq, D = q.shape
    NB, bs, Hkv, _ = k_cache.shape
    assert bs == block_size
    G = Hq // Hkv
    bt = np.asarray(block_tables)
    ctx = np.asarray(context_lens)
    scale = np.float32(scale)
    to_f32, to_bits = _codec(dtype)
    out = np.zeros((B, Hq, D), dtype=np.float32)
    for b in range(B):
        # the reference masks over the MB * bs gathered positions (:216-217): a
        # length beyond them means all of them, a negative one none
        n = min(int(ctx[b]), bt.shape[1] * block_size)
        if n <= 0:
            continue
        nblk = -(-n // block_size)
        pages = np.clip(bt[b, :nblk], 0, NB - 1)                     # :185
        k = to_f32(k_cache[pages].reshape(nblk * bs, Hkv, D)[:n])
        v = to_f32(v_cache[pages].reshape(nblk * bs, Hkv, D)[:n])
        qb = to_f32(q[b]).reshape(Hkv, G, D)               # head h -> kv h // G (:197)
        s = np.einsum("kgd,skd->kgs", qb, k, dtype=np.float32) * scale
        smax = s.max(axis=-1, keepdims=True)
        e = np.exp(s - smax, dtype=np.float32)
        w = e / (e.sum(axis=-1, keepdims=True, dtype=np.float32) + np.float32(1e-9))
        out[b] = np.einsum("kgs,skd->kgd", w, v, dtype=np.float32).reshape(Hq, D)
    if return_f32:
        return out
    return to_bits(out)


def paged_attention_fallback_ref(q, k_cache, v_cache, block_tables,
                                 context_lens, scale, block_size):
    """Restates the gather + ``jax.nn.dot_product_attention`` fallback
    (``layers/attention.py:399-434``; twin ``_paged_attention_fallback``
    ``layers/pallas_attention.py:510-550``).

    ``jax.nn.dot_product_attention`` is third-party (jax, not in the reference
    tree).  Its XLA implementation, as published, computes logits from the
    bf16 operands with fp32 accumulation, scales, masks, takes the softmax in
    fp32, casts the probabilities to the value dtype (bf16) and contracts with
    V with fp32 accumulation, rounding the result to bf16.  GQA maps query
    head h to kv head h // G.  Fully masked rows (ctx == 0) are not defined by
    the reference's callers; here they return zeros.
    """
    q = np.asarray(q)
    B, Hq, D = q.shape
    Hkv = k_cache.shape[2]
    G = Hq // Hkv
    kg, vg, mask = gather_kv_from_cache_ref(k_cache, v_cache, block_tables,
                                            context_lens, block_size)
    out = np.zeros((B, Hq, D), dtype=np.float32)
    scale = np.float32(scale)
    for b in range(B):
        n = int(mask[b].sum())
        if n == 0:
            continue
        k = bf16_bits_to_f32(kg[b, :n])
        v = bf16_bits_to_f32(vg[b, :n])
        qb = bf16_bits_to_f32(q[b]).reshape(Hkv, G, D)
        s = np.einsum("kgd,skd->kgs", qb, k, dtype=np.float32) * scale
        s = s - s.max(axis=-1, keepdims=True)
        e = np.exp(s, dtype=np.float32)
        p = e / e.sum(axis=-1, keepdims=True, dtype=np.float32)
        p = bf16_bits_to_f32(f32_to_bf16_bits(p))        # probs.astype(value.dtype)
        out[b] = np.einsum("kgs,skd->kgd", p, v, dtype=np.float32).reshape(Hq, D)
    return f32_to_bf16_bits(out)


def textbook_attention_f64(q, k_cache, v_cache, block_tables, context_lens,
                           scale, block_size):
    """softmax(q K^T * scale) V in float64 with plain Python loops over
    (sequence, head, position): the independent brute-force statement the
    restatements above are pinned against on small shapes.  Returns float64
    [B, Hq, D] (not rounded)."""
    q = np.asarray(q)
    B, Hq, D = q.shape
    NB, bs, Hkv, _ = k_cache.shape
    G = Hq // Hkv
    qf = bf16_bits_to_f32(q).astype(np.float64)
    kf = bf16_bits_to_f32(k_cache).astype(np.float64)
    vf = bf16_bits_to_f32(v_cache).astype(np.float64)
    out = np.zeros((B, Hq, D), dtype=np.float64)
    for b in range(B):
        n = int(context_lens[b])
        for h in range(Hq):
            kvh = h // G
            logits = np.empty(n, dtype=np.float64)
            for pos in range(n):
                page = int(block_tables[b, pos // block_size])
                logits[pos] = float(scale) * float(qf[b, h] @ kf[page, pos % block_size, kvh])
            if n == 0:
                continue
            w = np.exp(logits - logits.max())
            w /= w.sum()
            acc = np.zeros(D, dtype=np.float64)
            for pos in range(n):
                page = int(block_tables[b, pos // block_size])
                acc += w[pos] * vf[page, pos % block_size, kvh]
            out[b, h] = acc
    return out


# ---------------------------------------------------------------------------
# QK-RMSNorm + rotary embedding (+ store): the ops in front of the path
# ---------------------------------------------------------------------------

def build_cos_sin_cache_ref(head_dim: int, max_position: int, base: float) -> np.ndarray:
    """``RotaryEmbedding.__init__`` (``layers/rotary_embedding.py:60-76``):
    ``inv_freq = 1 / base ** (arange(0, D, 2) / D)``, ``freqs = outer(t, inv_freq)``,
    cache = ``[cos(freqs) | sin(freqs)]`` as float32 ``[max_position, D]``."""
    inv_freq = (1.0 / (np.float32(base) ** (np.arange(0, head_dim, 2, dtype=np.float32)
                                            / np.float32(head_dim)))).astype(np.float32)
    t = np.arange(max_position, dtype=np.float32)
    freqs = np.einsum("i,j->ij", t, inv_freq).astype(np.float32)
    return np.concatenate([np.cos(freqs), np.sin(freqs)], axis=-1).astype(np.float32)


def _butterfly_sum_128(sq1: np.ndarray, sq2: np.ndarray) -> np.ndarray:
    """Sum of 128 squares in the order the HIP kernel uses: lane l starts from
    x[l]^2 + x[l+64]^2, then adds its xor partner for masks 32, 16, .., 1.
    fp32 throughout; every lane ends with the same value, lane 0 is returned."""
    s = (sq1 + sq2).astype(np.float32)                  # [..., 64]
    lanes = np.arange(64)
    for m in (32, 16, 8, 4, 2, 1):
        s = (s + s[..., lanes ^ m]).astype(np.float32)
    return s[..., :1]


def qk_norm_rope_ref(x, positions, cos_sin_cache, weight, eps):
    """RMSNorm over the head dimension, then rotary embedding, for q or k.

    x : [T, H, 128] bf16 bits.  Follows ``RMSNorm._rms_forward``
    (``layers/layernorm.py:31-48``: fp32, ``x * rsqrt(mean(x^2) + eps) * weight``,
    cast back to the input dtype) and ``apply_rotary_emb``
    (``layers/rotary_embedding.py:13-37``: halves ``x1, x2``; ``y1 = x1 cos - x2
    sin``, ``y2 = x2 cos + x1 sin`` with float32 cos/sin, so the result is
    float32), with ``cos_sin = cache[positions]`` (:96-106).  ``weight`` None
    skips the norm (``models/qwen3.py:157``).  Returns float32 ``[T, H, 128]``.

    The reference leaves the fp32 summation order of the mean to XLA; this
    restatement fixes it to the xor-butterfly order of the HIP kernel so that
    the two agree bit for bit.  Any other order differs by fp32 round-off only.
    """
    xf = bf16_bits_to_f32(np.asarray(x))
    T, H, D = xf.shape
    assert D == 128
    x1, x2 = xf[..., :64], xf[..., 64:]
    if weight is not None:
        w = np.asarray(weight, dtype=np.float32)
        s = _butterfly_sum_128(x1 * x1, x2 * x2)
        var = s * np.float32(1.0 / 128.0) + np.float32(eps)
        r = (np.float32(1.0) / np.sqrt(var, dtype=np.float32)).astype(np.float32)
        x1 = bf16_bits_to_f32(f32_to_bf16_bits((x1 * r) * w[:64]))
        x2 = bf16_bits_to_f32(f32_to_bf16_bits((x2 * r) * w[64:]))
    pos = np.clip(np.asarray(positions, dtype=np.int64), 0, cos_sin_cache.shape[0] - 1)
    cs = np.asarray(cos_sin_cache, dtype=np.float32)[pos][:, None, :]
    cos, sin = cs[..., :64], cs[..., 64:]
    y1 = (x1 * cos).astype(np.float32) - (x2 * sin).astype(np.float32)
    y2 = (x2 * cos).astype(np.float32) + (x1 * sin).astype(np.float32)
    return np.concatenate([y1, y2], axis=-1).astype(np.float32)


def qk_norm_rope_store_ref(qkv, positions, cos_sin_cache, q_weight, k_weight, eps, k_cache,
                           v_cache, slot_mapping, num_heads, num_kv_heads,
                           negative_slots: str = "skip"):
    """The chain ``models/qwen3.py:150-166`` + ``layers/attention.py:386-387, 457-475``
    for packed ``qkv`` [T, (Hq + 2 Hkv) * 128] bf16 bits: split, QK norm, RoPE,
    q cast to bf16, K (float32 after RoPE) and V stored through
    ``store_kv_to_cache_ref``.  Returns ``(q_bits, k_cache, v_cache)``."""
    qkv = np.asarray(qkv)
    T = qkv.shape[0]
    D = 128
    qs, ks = num_heads * D, num_kv_heads * D
    q = qkv[:, :qs].reshape(T, num_heads, D)
    k = qkv[:, qs:qs + ks].reshape(T, num_kv_heads, D)
    v = qkv[:, qs + ks:qs + 2 * ks].reshape(T, num_kv_heads, D)
    q_rot = qk_norm_rope_ref(q, positions, cos_sin_cache, q_weight, eps)
    k_rot = qk_norm_rope_ref(k, positions, cos_sin_cache, k_weight, eps)
    kc, vc = store_kv_to_cache_ref(k_rot, np.ascontiguousarray(v), k_cache, v_cache,
                                   slot_mapping, negative_slots=negative_slots)
    return f32_to_bf16_bits(q_rot), kc, vc


# ---------------------------------------------------------------------------
# Decode metadata: the filler of the contract
# ---------------------------------------------------------------------------

def prepare_decode_ref(last_tokens, seq_lens, block_tables, block_size):
    """``ModelRunner._prepare_decode`` + ``_prepare_block_tables``
    (``engine/model_runner.py:334-376, 225-246``) for sequences given as
    (last token, length, list of page numbers): per sequence
    ``input_ids = last_token``, ``positions = len - 1``, ``context_lens = len``,
    ``slot = block_table[-1] * block_size + last_block_num_tokens - 1`` with
    ``last_block_num_tokens = len - (num_blocks - 1) * block_size``
    (``engine/sequence.py``), tables padded with -1 to the longest.  All int32."""
    n = len(seq_lens)
    input_ids = np.empty(n, np.int32)
    positions = np.empty(n, np.int32)
    context_lens = np.empty(n, np.int32)
    slot_mapping = np.empty(n, np.int32)
    width = max(len(t) for t in block_tables)
    tables = np.full((n, width), -1, np.int32)                     # :240
    for i in range(n):
        length, table = int(seq_lens[i]), list(block_tables[i])
        input_ids[i] = last_tokens[i]                              # :358
        positions[i] = length - 1                                  # :359
        context_lens[i] = length                                   # :360
        last_block_num_tokens = length - (len(table) - 1) * block_size
        slot_mapping[i] = table[-1] * block_size + last_block_num_tokens - 1   # :361
        tables[i, :len(table)] = table
    return input_ids, positions, context_lens, slot_mapping, tables


def advance_decode_ref(next_tokens, input_ids, positions, context_lens, slot_mapping,
                       block_tables, block_size):
    """What the arrays of ``prepare_decode_ref`` become once every active
    sequence has appended ``next_tokens[i]`` (``Sequence.append_token``, then the
    next ``_prepare_decode``), computed from the padded table instead of the
    Python lists: the page of position ``len - 1`` is column
    ``(len - 1) // block_size`` of the row.  Rows with ``context_lens <= 0`` are
    inactive (slot -1, nothing else changes); a row whose next page is missing
    (-1, or beyond the table) is left as it is with slot -1.  Returns new arrays."""
    ids = np.array(input_ids, np.int32, copy=True)
    pos = np.array(positions, np.int32, copy=True)
    ctx = np.array(context_lens, np.int32, copy=True)
    slots = np.array(slot_mapping, np.int32, copy=True)
    bt = np.asarray(block_tables)
    for i in range(len(ctx)):
        if ctx[i] <= 0:
            slots[i] = -1
            continue
        length = int(ctx[i]) + 1
        page_idx = (length - 1) // block_size
        page = int(bt[i, page_idx]) if page_idx < bt.shape[1] else -1
        if page < 0:
            slots[i] = -1
            continue
        ids[i] = next_tokens[i]
        pos[i] = length - 1
        ctx[i] = length
        slots[i] = page * block_size + (length - 1) % block_size
    return ids, pos, ctx, slots


# ---------------------------------------------------------------------------
# Variable-length causal prefill attention
# ---------------------------------------------------------------------------

def variable_length_attention_prefill_ref(q, k, v, cu_seqlens_q, cu_seqlens_k, scale,
                                          return_f32: bool = False, dtype: str = "bf16"):
    """Restates ``variable_length_attention_prefill`` (``layers/attention.py:135-279``)
    without its padding: for sequence i, q rows [cu_q[i], cu_q[i+1]) attend k/v
    rows [cu_k[i], cu_k[i+1]) under ``q_pos >= k_pos`` (:232-236, positions counted
    from the start of the sequence) and the validity masks (:238-243).  Padding
    rows exist only to make XLA shapes static (:186-222) and are scattered away
    (:263-277), so leaving them out changes nothing.  The attention itself is
    ``jax.nn.dot_product_attention`` (:247-251): fp32 logits from the bf16
    operands, fp32 softmax, probabilities cast to bf16, fp32-accumulated PV,
    bf16 result; GQA by head broadcast (h -> h // G).  A query row with no
    visible key is not defined by the reference; zeros here.

    q [T, Hq, D], k/v [Tk, Hkv, D] bit patterns of ``dtype`` ("bf16" or "f16").
    Returns [T, Hq, D] bits of the same type."""
    decode, encode = _codec(dtype)
    q = np.asarray(q)
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    cu_q = np.asarray(cu_seqlens_q, dtype=np.int64)
    cu_k = np.asarray(cu_seqlens_k, dtype=np.int64)
    out = np.zeros((T, Hq, D), dtype=np.float32)
    scale = np.float32(scale)
    for i in range(len(cu_q) - 1):
        lq, lk = int(cu_q[i + 1] - cu_q[i]), int(cu_k[i + 1] - cu_k[i])
        if lq <= 0 or lk <= 0:
            continue
        qs = decode(q[cu_q[i]:cu_q[i + 1]]).reshape(lq, Hkv, G, D)
        ks = decode(k[cu_k[i]:cu_k[i + 1]])
        vs = decode(v[cu_k[i]:cu_k[i + 1]])
        mask = np.arange(lq)[:, None] >= np.arange(lk)[None, :]           # :232-236
        s = np.einsum("qhgd,khd->hgqk", qs, ks, dtype=np.float32) * scale
        s = np.where(mask[None, None], s, np.float32(-1e30))
        s = s - s.max(axis=-1, keepdims=True)
        e = np.where(mask[None, None], np.exp(s, dtype=np.float32), np.float32(0))
        p = e / e.sum(axis=-1, keepdims=True, dtype=np.float32)
        p = decode(encode(p))                                            # probs -> value dtype
        o = np.einsum("hgqk,khd->qhgd", p, vs, dtype=np.float32)
        out[cu_q[i]:cu_q[i + 1]] = o.reshape(lq, Hq, D)
    return out if return_f32 else encode(out)


def paged_prefill_attention_ref(q, k_cache, v_cache, block_tables, cu_seqlens_q, cu_seqlens_k,
                                scale, return_f32: bool = False, dtype: str = "bf16"):
    """Prefill attention behind a cached prefix.  The reference prepares this case
    (``engine/model_runner.py:286-312``: ``seqlen_k = len(seq)``, ``seqlen_q`` without
    the cached tokens, ``block_tables`` set) but its attention call never reads the
    cached keys, so there is no reference behaviour to restate beyond the
    mathematics: the ``len_q`` query rows of a sequence are its last ``len_q``
    positions, row j attends the keys at positions ``<= len_k - len_q + j``, all
    ``len_k`` keys and values gathered from the pages (``layers/attention.py:80-122``),
    and the attention itself as in ``variable_length_attention_prefill_ref``."""
    decode, encode = _codec(dtype)
    q = np.asarray(q)
    T, Hq, D = q.shape
    NB, bs, Hkv, _ = k_cache.shape
    G = Hq // Hkv
    cu_q = np.asarray(cu_seqlens_q, dtype=np.int64)
    cu_k = np.asarray(cu_seqlens_k, dtype=np.int64)
    bt = np.asarray(block_tables)
    out = np.zeros((T, Hq, D), dtype=np.float32)
    scale = np.float32(scale)
    for i in range(len(cu_q) - 1):
        lq = int(cu_q[i + 1] - cu_q[i])
        lk = min(max(int(cu_k[i + 1] - cu_k[i]), 0), bt.shape[1] * bs)
        if lq <= 0 or lk <= 0:
            continue
        pages = np.clip(bt[i, :-(-lk // bs)], 0, NB - 1)
        ks = decode(k_cache[pages].reshape(-1, Hkv, D)[:lk])
        vs = decode(v_cache[pages].reshape(-1, Hkv, D)[:lk])
        qs = decode(q[cu_q[i]:cu_q[i + 1]]).reshape(lq, Hkv, G, D)
        off = max(lk - lq, 0)
        mask = (off + np.arange(lq))[:, None] >= np.arange(lk)[None, :]
        s = np.einsum("qhgd,khd->hgqk", qs, ks, dtype=np.float32) * scale
        s = np.where(mask[None, None], s, np.float32(-1e30))
        s = s - s.max(axis=-1, keepdims=True)
        e = np.where(mask[None, None], np.exp(s, dtype=np.float32), np.float32(0))
        p = e / e.sum(axis=-1, keepdims=True, dtype=np.float32)
        p = decode(encode(p))
        o = np.einsum("hgqk,khd->qhgd", p, vs, dtype=np.float32)
        out[cu_q[i]:cu_q[i + 1]] = o.reshape(lq, Hq, D)
    return out if return_f32 else encode(out)


def textbook_prefill_f64(q, k, v, cu_seqlens_q, cu_seqlens_k, scale):
    """Causal softmax(q K^T scale) V per (sequence, head, query row) in float64
    with plain loops: the brute force the restatement above is pinned against."""
    q = np.asarray(q)
    T, Hq, D = q.shape
    G = Hq // k.shape[1]
    qf = bf16_bits_to_f32(q).astype(np.float64)
    kf = bf16_bits_to_f32(np.asarray(k)).astype(np.float64)
    vf = bf16_bits_to_f32(np.asarray(v)).astype(np.float64)
    out = np.zeros((T, Hq, D))
    for i in range(len(cu_seqlens_q) - 1):
        q0, q1 = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        k0, k1 = int(cu_seqlens_k[i]), int(cu_seqlens_k[i + 1])
        for row in range(q1 - q0):
            n = min(row + 1, k1 - k0)
            if n <= 0:
                continue
            for h in range(Hq):
                logits = np.array([float(scale) * (qf[q0 + row, h] @ kf[k0 + j, h // G])
                                   for j in range(n)])
                w = np.exp(logits - logits.max())
                w /= w.sum()
                out[q0 + row, h] = sum(w[j] * vf[k0 + j, h // G] for j in range(n))
    return out


# ---------------------------------------------------------------------------
# RMSNorm (+ residual) and SiLU-and-multiply
# ---------------------------------------------------------------------------
def add_rms_norm_ref(x, weight, eps, residual=None):
    """``RMSNorm._rms_forward`` / ``_add_rms_forward`` (layers/layernorm.py:31-79).

    ``x``, ``residual``: ``[T, hidden]`` bf16 bit patterns (uint16); ``weight``
    ``[hidden]`` float32.  Returns ``y`` bits, or ``(y, new_residual)`` bits.

    fp32 throughout as the reference (:41, :66); the order of the sum of squares
    is this oracle's choice: the row is cut into 8-element pieces, accumulator
    ``l`` (of 64) takes pieces ``l, l + 64, ...`` in row order, then the 64
    accumulators are folded pairwise at distances 32, 16, ..., 1.
    """
    xb = _as_bf16_bits(np.asarray(x))
    t, hidden = xb.shape
    assert hidden % 8 == 0
    s = bf16_bits_to_f32(xb)
    new_res = None
    if residual is not None:
        s = (s + bf16_bits_to_f32(_as_bf16_bits(np.asarray(residual)))).astype(np.float32)
        new_res = f32_to_bf16_bits(s)                          # :68-69
    pieces = hidden // 8
    sq = (s * s).astype(np.float32).reshape(t, pieces, 8)
    acc = np.zeros((t, 64), np.float32)
    for p in range(pieces):
        lane = p % 64
        for e in range(8):
            acc[:, lane] = (acc[:, lane] + sq[:, p, e]).astype(np.float32)
    m = 32
    while m >= 1:
        idx = np.arange(64) ^ m
        acc = (acc + acc[:, idx]).astype(np.float32)
        m >>= 1
    total = acc[:, :1]
    inv_hidden = np.float32(1.0) / np.float32(hidden)
    r = (np.float32(1.0) / np.sqrt((total * inv_hidden + np.float32(eps)).astype(np.float32))
         ).astype(np.float32)                                  # :72-73
    w = np.asarray(weight, np.float32)[None, :]
    y = f32_to_bf16_bits(((s * r).astype(np.float32) * w).astype(np.float32))   # :76
    return y if residual is None else (y, new_res)


def silu_and_mul_ref(x):
    """``SiluAndMul.__call__`` (layers/activation.py:22-33): ``x`` ``[T, 2*I]`` bf16
    bits -> ``[T, I]`` bf16 bits, ``silu(gate) * up`` evaluated in float64 from the
    bf16 inputs and rounded once (via float32) to bf16."""
    xb = _as_bf16_bits(np.asarray(x))
    inter = xb.shape[-1] // 2
    g = bf16_bits_to_f32(xb[..., :inter]).astype(np.float64)
    u = bf16_bits_to_f32(xb[..., inter:]).astype(np.float64)
    with np.errstate(over="ignore"):
        out = g / (1.0 + np.exp(-g)) * u
    return f32_to_bf16_bits(out.astype(np.float32))
