"""Writes tests/golden/paged_decode_small.npz: seeded inputs and the expected
outputs of the CPU oracle for one small decode step (store, then attention).

The reference holds no vectors for this path (its only numeric check draws its
inputs from jax.random and stores nothing), so these come from the oracle,
after the oracle itself has been pinned (tests/test_oracle_pinning.py).  They
guard the oracle and the HIP path against silent drift.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from nanovllm_jax_amd.workloads import draw_bf16_bits  # noqa: E402
from oracle.paged_attention_oracle import (paged_decode_attention_per_seq_ref,  # noqa: E402
                                           store_kv_to_cache_ref)


def main():
    rng = np.random.Generator(np.random.PCG64(20240607))
    B, Hq, Hkv, D, bs, NB = 5, 8, 2, 128, 32, 10
    ctx = np.array([1, 33, 64, 100, 0], np.int32)
    nblk = -(-ctx // bs)
    MB = int(nblk.max())
    pages = rng.permutation(NB)
    bt = np.full((B, MB), -1, np.int32)
    off = 0
    for b in range(B):
        bt[b, :nblk[b]] = pages[off:off + nblk[b]]
        off += nblk[b]
    q = draw_bf16_bits(rng, (B, Hq, D))
    kc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    vc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    k_new = rng.standard_normal((B, Hkv, D), dtype=np.float32)
    v_new = draw_bf16_bits(rng, (B, Hkv, D))
    last = np.maximum(ctx - 1, 0)
    slots = np.where(ctx > 0, bt[np.arange(B), last // bs] * bs + last % bs, -1).astype(np.int32)
    flat = (NB * bs, Hkv, D)
    kc2, vc2 = store_kv_to_cache_ref(k_new, v_new, kc.reshape(flat), vc.reshape(flat), slots,
                                     negative_slots="skip")
    scale = np.float32(1.0 / np.sqrt(D))
    out = paged_decode_attention_per_seq_ref(q, kc2.reshape(kc.shape), vc2.reshape(vc.shape), bt,
                                             ctx, scale, bs)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "paged_decode_small.npz")
    np.savez_compressed(path, q=q, k_cache=kc, v_cache=vc, block_tables=bt, context_lens=ctx,
                        slot_mapping=slots, k_new=k_new, v_new=v_new, scale=scale,
                        block_size=np.int32(bs), k_cache_after=kc2.reshape(kc.shape),
                        v_cache_after=vc2.reshape(vc.shape), out=out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
