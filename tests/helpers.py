"""Shared helpers for the tests: bf16 bit patterns <-> torch tensors, seeded
small problems, the tolerance of the attention parity bar."""
from __future__ import annotations

import numpy as np

# attention parity bar: bf16 output, fp32 accumulate
ATOL = 1e-2
RTOL = 1e-2


def bits_to_torch(bits: np.ndarray, device="cpu"):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)
    return t.to(device)


def torch_to_bits(t) -> np.ndarray:
    import torch
    assert t.dtype in (torch.bfloat16, torch.float16)
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def make_problem(seed, B, Hq, Hkv, D, bs, NB, ctx, q_gain=1.0, shuffle=True):
    """Random bf16 q / caches and a block table for the given context lengths.
    Pages are drawn without replacement; table padding is -1."""
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = np.asarray(ctx, dtype=np.int32)
    assert len(ctx) == B
    nblk = -(-ctx // bs)
    MB = max(int(nblk.max()), 1)
    assert int(nblk.sum()) <= NB
    pages = rng.permutation(NB) if shuffle else np.arange(NB)
    bt = np.full((B, MB), -1, dtype=np.int32)
    off = 0
    for b in range(B):
        bt[b, :nblk[b]] = pages[off:off + nblk[b]]
        off += nblk[b]
    q = draw_bf16_bits(rng, (B, Hq, D), q_gain)
    kc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    vc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    return q, kc, vc, bt, ctx


def assert_close_bf16(got_bits, want_bits, atol=ATOL, rtol=RTOL, what=""):
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    got = bf16_bits_to_f32(got_bits).astype(np.float64)
    want = bf16_bits_to_f32(want_bits).astype(np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    bound = atol + rtol * np.abs(want)
    bad = ~(err <= bound)
    if bad.any():
        idx = np.unravel_index(np.argmax(np.where(bad, err, -1)), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.size} outside atol={atol} rtol={rtol}; "
            f"worst at {idx}: got {got[idx]} want {want[idx]} (max abs err {np.nanmax(err):.3e})")
    return float(err.max())
