"""Seeded synthetic decode workloads (block tables, context lengths, slots).

The five shapes are the ones the path is specified and measured on; C1..C4 are
single-layer paged decode calls, C5 is the whole-model decode step.  Only the
integer metadata is built here (NumPy, ``PCG64(seed)``); K/V/q values are
N(0,1) rounded to bf16 and are drawn by the caller either on the host
(``draw_bf16_bits``) or on the device.

Metadata follows the formulas of the reference's filler:
``slot = block_table[-1] * block_size + last_block_num_tokens - 1``
(``engine/model_runner.py:361``), ``context_lens = len(seq)`` (:360), block
tables padded with -1 (:240).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

__all__ = ["DecodeWorkload", "make_workload", "draw_bf16_bits", "algorithmic_bytes",
           "WORKLOADS"]


@dataclass
class DecodeWorkload:
    name: str
    batch: int
    num_heads: int          # Hq
    num_kv_heads: int       # Hkv
    head_dim: int
    block_size: int
    num_blocks: int         # pool size NB
    context_lens: np.ndarray    # [B] int32 (already counts the token being decoded)
    block_tables: np.ndarray    # [B, MB] int32, -1 padded
    slot_mapping: np.ndarray    # [B] int32, slot of the token being decoded
    q_gain: float = 1.0
    seed: int = 0
    extra: dict = field(default_factory=dict)

    @property
    def max_blocks(self) -> int:
        return int(self.block_tables.shape[1])

    @property
    def scale(self) -> float:
        return 1.0 / float(np.sqrt(self.head_dim))


def _slots(block_tables, context_lens, block_size):
    ctx = context_lens.astype(np.int64)
    last = np.maximum(ctx - 1, 0)
    page = block_tables[np.arange(len(ctx)), last // block_size].astype(np.int64)
    slot = page * block_size + last % block_size
    return np.where(ctx > 0, slot, -1).astype(np.int32)


def _tables_from_counts(rng, nblk, num_blocks, max_blocks):
    """Each sequence gets ``nblk[b]`` distinct pages drawn without replacement
    from the pool; the rest of its row is -1."""
    total = int(nblk.sum())
    assert total <= num_blocks, (total, num_blocks)
    pages = rng.permutation(num_blocks)[:total].astype(np.int32)
    bt = np.full((len(nblk), max_blocks), -1, dtype=np.int32)
    off = 0
    for b, n in enumerate(nblk):
        bt[b, :n] = pages[off:off + n]
        off += n
    return bt


def make_workload(name: str, seed: int | None = None) -> DecodeWorkload:
    name = name.upper()
    if name == "C1":     # Qwen3-0.6B shape, CPU-runnable
        seed = 1001 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs, NB, MB = 8, 16, 8, 128, 256, 64, 8
        ctx = rng.integers(128, 2049, size=B).astype(np.int32)
        bt = rng.permutation(NB).astype(np.int32).reshape(B, MB)
        nblk = -(-ctx // bs)
        bt[np.arange(MB)[None, :] >= nblk[:, None]] = -1
        gain = 1.0
    elif name == "C2":   # Qwen3-8B shape, the headline
        seed = 1002 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs, NB, MB = 64, 32, 8, 128, 256, 1024, 16
        ctx = np.full(B, 4096, dtype=np.int32)
        bt = rng.permutation(NB).astype(np.int32).reshape(B, MB)
        gain = 1.0
    elif name == "C3":   # ragged stress
        seed = 1003 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs = 256, 32, 8, 128, 256
        ctx = np.rint(np.exp(rng.uniform(np.log(16.0), np.log(32768.0), size=B)))
        ctx = np.clip(ctx, 16, 32768).astype(np.int32)
        nblk = -(-ctx // bs)
        NB = int(np.ceil(1.1 * nblk.sum()))
        MB = int(nblk.max())
        bt = _tables_from_counts(rng, nblk, NB, MB)
        gain = 1.0
    elif name == "C4":   # Qwen3-32B shape, long context, sharpened softmax
        seed = 1004 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs, NB, MB = 16, 64, 8, 128, 256, 2048, 128
        ctx = np.full(B, 32768, dtype=np.int32)
        bt = rng.permutation(NB).astype(np.int32).reshape(B, MB)
        gain = 4.0
    elif name == "C5":   # one layer of the whole-model decode step
        seed = 1005 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs, NB, MB = 128, 16, 8, 128, 256, 512, 4
        ctx = np.full(B, 1024, dtype=np.int32)
        bt = rng.permutation(NB).astype(np.int32).reshape(B, MB)
        gain = 1.0
    elif name == "R1":   # the shape the reference itself times (profile_attention.py:19-34)
        # MHA cache (32 KV heads), identity block tables, context lengths uniform in
        # [200, 2048); the reference draws fp16 with jax.random, here bf16 from this seed
        seed = 1101 if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        B, Hq, Hkv, D, bs, NB, MB = 64, 32, 32, 128, 256, 512, 8
        ctx = rng.integers(200, 2048, size=B).astype(np.int32)
        bt = np.arange(NB, dtype=np.int32).reshape(B, MB)
        gain = 1.0
    elif name in ("C2_JITTER", "C2_SPREAD", "RAGGED_SHORT"):
        # batches as a serving loop really sees them (the reference's filler hands over
        # whatever lengths the running sequences have, engine/model_runner.py:357-361):
        # C2 with lengths a few percent apart, C2 with lengths from half to one and a
        # half times 4096, and 256 short sequences of 200 to 2048 positions
        seed = {"C2_JITTER": 1012, "C2_SPREAD": 1022, "RAGGED_SHORT": 1032}[name] \
            if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        Hq, Hkv, D, bs = 32, 8, 128, 256
        if name == "C2_JITTER":
            B, ctx = 64, rng.integers(3840, 4097, size=64)
        elif name == "C2_SPREAD":
            B, ctx = 64, rng.integers(2048, 6145, size=64)
        else:
            B, ctx = 256, rng.integers(200, 2049, size=256)
        ctx = ctx.astype(np.int32)
        nblk = -(-ctx // bs)
        NB = int(np.ceil(1.1 * nblk.sum()))
        MB = int(nblk.max())
        bt = _tables_from_counts(rng, nblk, NB, MB)
        gain = 1.0
    elif name.startswith("UNIFORM:") or name.startswith("LOGUNIFORM:"):
        # UNIFORM:<batch>:<lo>:<hi>[:<kv heads>[:<query heads>]]: lengths uniform in
        # [lo, hi] (LOGUNIFORM: their logarithms are), Qwen3-8B heads unless given; a
        # measuring aid (bench.py --workload)
        f = [int(x) for x in name.split(":")[1:]]
        B, lo, hi = f[0], f[1], f[2]
        Hkv = f[3] if len(f) > 3 else 8
        Hq = f[4] if len(f) > 4 else 4 * Hkv
        D, bs = 128, 256
        seed = 2000 + B if seed is None else seed
        rng = np.random.Generator(np.random.PCG64(seed))
        if name.startswith("LOG"):
            ctx = np.rint(np.exp(rng.uniform(np.log(lo), np.log(hi), size=B))).astype(np.int32)
        else:
            ctx = rng.integers(lo, hi + 1, size=B).astype(np.int32)
        nblk = -(-ctx // bs)
        NB = int(np.ceil(1.1 * nblk.sum())) + 1
        MB = max(int(nblk.max()), 1)
        bt = _tables_from_counts(rng, nblk, NB, MB)
        gain = 1.0
    else:
        raise KeyError(name)
    return DecodeWorkload(name=name, batch=B, num_heads=Hq, num_kv_heads=Hkv,
                          head_dim=D, block_size=bs, num_blocks=NB,
                          context_lens=ctx, block_tables=bt,
                          slot_mapping=_slots(bt, ctx, bs), q_gain=gain, seed=seed)


WORKLOADS = ("C1", "C2", "C3", "C4", "C5", "R1", "C2_JITTER", "C2_SPREAD", "RAGGED_SHORT")


def draw_bf16_bits(rng: np.random.Generator, shape, gain: float = 1.0) -> np.ndarray:
    """N(0,1) * gain drawn in fp32, rounded to nearest-even bf16, returned as
    uint16 bit patterns."""
    x = rng.standard_normal(size=shape, dtype=np.float32)
    if gain != 1.0:
        x *= np.float32(gain)
    u = x.view(np.uint32)
    return ((u + (((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)))
            >> np.uint32(16)).astype(np.uint16)


def algorithmic_bytes(context_lens, batch, num_heads, num_kv_heads, head_dim,
                      max_blocks) -> int:
    """Bytes one decode call must move: K and V rows of every live position
    (bf16), q in and out (bf16), block tables and context lengths (int32).
    Split-K partials are overhead and are not counted."""
    total_ctx = int(np.asarray(context_lens, dtype=np.int64).sum())
    return (total_ctx * num_kv_heads * head_dim * 2 * 2
            + 2 * batch * num_heads * head_dim * 2
            + batch * max_blocks * 4 + batch * 4)
