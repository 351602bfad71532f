"""Pins the CPU oracle (NumPy and C restatements) without the reference:
brute force in fp64, a library routine, closed forms and invariants, each
chosen so that a plausible slip (wrong head mapping, missing scale, mask off by
one, transposed operand, wrong rounding) fails at least one of them."""
import numpy as np
import pytest
import torch

from helpers import bits_to_torch, make_problem, torch_to_bits
from oracle import c_oracle
from oracle.paged_attention_oracle import (bf16_bits_to_f32, f32_to_bf16_bits,
                                           paged_attention_fallback_ref,
                                           paged_decode_attention_per_seq_ref,
                                           paged_decode_attention_vectorized_ref,
                                           store_kv_to_cache_ref, textbook_attention_f64)

IMPLS = {
    "vectorized": lambda *a: bf16_bits_to_f32(paged_decode_attention_vectorized_ref(*a)),
    "per_seq": lambda *a: paged_decode_attention_per_seq_ref(*a, return_f32=True),
    "c": lambda *a: c_oracle.paged_decode(*a, return_f32=True),
}


# ---------------------------------------------------------------- bf16 rounding
def test_bf16_rounding_matches_torch_on_all_interesting_patterns():
    rng = np.random.Generator(np.random.PCG64(1))
    u = rng.integers(0, 2**32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    # every exponent with tie / just-below / just-above mantissas
    exps = np.arange(256, dtype=np.uint32) << 23
    tails = np.array([0x0000, 0x7FFF, 0x8000, 0x8001, 0x18000, 0x17FFF, 0x7F8000, 0x7FFFFF],
                     dtype=np.uint32)
    special = (exps[:, None] | tails[None, :]).ravel()
    u = np.concatenate([u, special, special | np.uint32(0x80000000)])
    x = u.view(np.float32)
    got = f32_to_bf16_bits(x)
    want = torch_to_bits(torch.from_numpy(x.copy()).to(torch.bfloat16))
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(bf16_bits_to_f32(got[nan])).all()


def test_bf16_round_trip_is_exact():
    b = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = bf16_bits_to_f32(b)
    keep = ~np.isnan(f)
    assert np.array_equal(f32_to_bf16_bits(f)[keep], b[keep])
    assert np.array_equal(f[keep], bits_to_torch(b).float().numpy()[keep])


# ---------------------------------------------------------------- store
def _store_problem(seed, T=9, Hkv=2, D=8, slots_n=32):
    rng = np.random.Generator(np.random.PCG64(seed))
    kc = rng.integers(0, 65536, (slots_n, Hkv, D)).astype(np.uint16)
    vc = rng.integers(0, 65536, (slots_n, Hkv, D)).astype(np.uint16)
    key = rng.standard_normal((T, Hkv, D), dtype=np.float32)
    val = rng.integers(0, 65536, (T, Hkv, D)).astype(np.uint16)
    slots = rng.permutation(slots_n)[:T].astype(np.int32)
    return key, val, kc, vc, slots


@pytest.mark.parametrize("impl", [store_kv_to_cache_ref, c_oracle.store_kvcache])
def test_store_against_per_token_loop(impl):
    key, val, kc, vc, slots = _store_problem(3)
    slots[2] = -1
    slots[5] = 32          # out of range -> dropped
    slots[6] = 10**6
    for mode in ("reference", "skip"):
        wk, wv = kc.copy(), vc.copy()
        for t in range(len(slots)):        # brute force
            s = int(slots[t])
            if s < 0:
                if mode == "skip":
                    continue
                s = 0
            if s >= kc.shape[0]:
                continue
            wk[s] = torch_to_bits(torch.from_numpy(key[t]).to(torch.bfloat16))
            wv[s] = val[t]
        gk, gv = impl(key, val, kc, vc, slots, negative_slots=mode)
        assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
    # the two modes differ exactly in row 0 (the reference's code clobbers it)
    rk, _ = impl(key, val, kc, vc, slots, negative_slots="reference")
    sk, _ = impl(key, val, kc, vc, slots, negative_slots="skip")
    assert np.array_equal(rk[1:], sk[1:]) and not np.array_equal(rk[0], sk[0])
    assert np.array_equal(sk[0], kc[0])


@pytest.mark.parametrize("impl", [store_kv_to_cache_ref, c_oracle.store_kvcache])
def test_store_invariants(impl):
    key, val, kc, vc, slots = _store_problem(4)
    k0, v0 = kc.copy(), vc.copy()
    gk, gv = impl(key, val, kc, vc, slots)
    assert np.array_equal(kc, k0) and np.array_equal(vc, v0), "inputs must not be modified"
    untouched = np.ones(kc.shape[0], bool); untouched[slots] = False
    assert np.array_equal(gk[untouched], kc[untouched]) and np.array_equal(gv[untouched], vc[untouched])
    gk2, gv2 = impl(key, val, gk, gv, slots)                 # idempotent
    assert np.array_equal(gk2, gk) and np.array_equal(gv2, gv)
    gk3, _ = impl(key, np.zeros_like(val), kc, vc, slots)    # K independent of V
    assert np.array_equal(gk3, gk)
    e = np.zeros((0,) + key.shape[1:], np.float32)           # no tokens
    ek, ev = impl(e, e.astype(np.uint16), kc, vc, np.zeros(0, np.int32))
    assert np.array_equal(ek, kc) and np.array_equal(ev, vc)


# ---------------------------------------------------------------- attention
@pytest.mark.parametrize("impl", sorted(IMPLS))
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (4, 2), (8, 2), (8, 1)])
def test_attention_against_fp64_brute_force(impl, Hq, Hkv):
    B, D, bs, NB = 3, 16, 8, 12
    q, kc, vc, bt, ctx = make_problem(21 + Hq + Hkv, B, Hq, Hkv, D, bs, NB, [1, 13, 24])
    scale = 0.37
    want = textbook_attention_f64(q, kc, vc, bt, ctx, scale, bs)
    got = IMPLS[impl](q, kc, vc, bt, ctx, scale, bs)
    tol = 1e-2 if impl == "vectorized" else 2e-5      # vectorized returns bf16-rounded values
    np.testing.assert_allclose(got, want, atol=tol, rtol=tol)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_attention_against_torch_sdpa_gqa(impl):
    """Library special case: gather the pages densely and call torch's
    scaled_dot_product_attention with enable_gqa on the CPU."""
    B, Hq, Hkv, D, bs, NB = 2, 8, 2, 32, 16, 10
    q, kc, vc, bt, ctx = make_problem(31, B, Hq, Hkv, D, bs, NB, [40, 57])
    scale = 1.0 / np.sqrt(D)
    got = IMPLS[impl](q, kc, vc, bt, ctx, scale, bs)
    for b in range(B):
        n = int(ctx[b]); nblk = -(-n // bs)
        k = bits_to_torch(kc[bt[b, :nblk]].reshape(-1, Hkv, D)[:n]).float()
        v = bits_to_torch(vc[bt[b, :nblk]].reshape(-1, Hkv, D)[:n]).float()
        qq = bits_to_torch(q[b]).float()
        o = torch.nn.functional.scaled_dot_product_attention(
            qq[None, :, None, :], k.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None],
            scale=float(scale), enable_gqa=True)[0, :, 0, :].numpy()
        tol = 1e-2 if impl == "vectorized" else 2e-5
        np.testing.assert_allclose(got[b], o, atol=tol, rtol=tol)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_attention_closed_forms(impl):
    B, Hq, Hkv, D, bs, NB = 4, 8, 2, 16, 8, 16
    q, kc, vc, bt, ctx = make_problem(41, B, Hq, Hkv, D, bs, NB, [0, 1, 20, 16])
    G = Hq // Hkv
    # all keys of sequence 2 equal -> uniform weights -> mean of V over ctx
    nblk = -(-int(ctx[2]) // bs)
    kc[bt[2, :nblk]] = kc[bt[2, 0], 0][None, None]
    scale = 0.5
    got = IMPLS[impl](q, kc, vc, bt, ctx, scale, bs)
    assert not got[0].any()                                           # ctx = 0 -> zeros
    v0 = bf16_bits_to_f32(vc[bt[1, 0], 0])                            # ctx = 1 -> V row
    np.testing.assert_allclose(got[1], np.repeat(v0, G, axis=0), rtol=1e-6, atol=0)
    v = bf16_bits_to_f32(vc[bt[2, :nblk]].reshape(-1, Hkv, D)[: ctx[2]]).astype(np.float64)
    tol = 1e-2 if impl == "vectorized" else 1e-5
    np.testing.assert_allclose(got[2], np.repeat(v.mean(axis=0), G, axis=0), atol=tol, rtol=tol)
    # identical queries inside a group -> identical outputs
    q2 = q.copy(); q2[3, 1] = q2[3, 0]
    got2 = IMPLS[impl](q2, kc, vc, bt, ctx, scale, bs)
    assert np.array_equal(got2[3, 0], got2[3, 1])
    # doubling the scale is the same as doubling q (power of two: exact in bf16)
    qd = f32_to_bf16_bits(bf16_bits_to_f32(q) * 2)
    np.testing.assert_allclose(IMPLS[impl](qd, kc, vc, bt, ctx, scale, bs),
                               IMPLS[impl](q, kc, vc, bt, ctx, 2 * scale, bs), atol=tol, rtol=tol)


@pytest.mark.parametrize("impl", sorted(IMPLS))
def test_attention_layout_invariances(impl):
    B, Hq, Hkv, D, bs, NB = 3, 4, 2, 16, 8, 20
    q, kc, vc, bt, ctx = make_problem(51, B, Hq, Hkv, D, bs, NB, [5, 17, 32])
    scale = 0.3
    base = IMPLS[impl](q, kc, vc, bt, ctx, scale, bs)
    # physical page permutation
    perm = np.random.Generator(np.random.PCG64(2)).permutation(NB)
    kc2 = np.empty_like(kc); vc2 = np.empty_like(vc); kc2[perm] = kc; vc2[perm] = vc
    bt2 = np.where(bt >= 0, perm[np.clip(bt, 0, NB - 1)], -1).astype(np.int32)
    np.testing.assert_array_equal(IMPLS[impl](q, kc2, vc2, bt2, ctx, scale, bs), base)
    # wider table with -1 padding, finite garbage past ctx and in unused pages
    bt3 = np.concatenate([bt, np.full((B, 3), -1, np.int32)], axis=1)
    kc3, vc3 = kc.copy(), vc.copy()
    for b in range(B):
        n = int(ctx[b]); last = (n - 1) // bs
        kc3[bt[b, last], n - last * bs:] = 0x4F00      # large finite
        vc3[bt[b, last], n - last * bs:] = 0xCF00
    np.testing.assert_allclose(IMPLS[impl](q, kc3, vc3, bt3, ctx, scale, bs), base,
                               atol=1e-6, rtol=1e-6)
    # one position more really changes the answer (mask is not off by one)
    ctx4 = ctx.copy(); ctx4[0] += 1
    assert not np.allclose(IMPLS[impl](q, kc, vc, bt, ctx4, scale, bs)[0], base[0])


def test_restatements_agree_with_each_other_at_c1():
    from nanovllm_jax_amd.workloads import draw_bf16_bits, make_workload
    w = make_workload("C1")
    rng = np.random.Generator(np.random.PCG64(5))
    shape = (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
    q = draw_bf16_bits(rng, (w.batch, w.num_heads, w.head_dim))
    kc, vc = draw_bf16_bits(rng, shape), draw_bf16_bits(rng, shape)
    args = (q, kc, vc, w.block_tables, w.context_lens, w.scale, w.block_size)
    a = paged_decode_attention_per_seq_ref(*args, return_f32=True)
    c = c_oracle.paged_decode(*args, return_f32=True)
    np.testing.assert_allclose(c, a, atol=2e-6, rtol=1e-5)
    v = bf16_bits_to_f32(paged_decode_attention_vectorized_ref(*args))
    np.testing.assert_allclose(v, a, atol=1e-6, rtol=2 ** -8)
    f = bf16_bits_to_f32(paged_attention_fallback_ref(*args))
    np.testing.assert_allclose(f, a, atol=1e-2, rtol=1e-2)     # the path's parity bar
