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
    "fallback": lambda *a: bf16_bits_to_f32(paged_attention_fallback_ref(*a)),
}
# these two return values rounded to bf16 (the fallback also rounds its probabilities)
ROUNDED = ("vectorized", "fallback")


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
    tol = 1e-2 if impl in ROUNDED else 2e-5
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
        tol = 1e-2 if impl in ROUNDED else 2e-5
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
    tol = 1e-2 if impl in ROUNDED else 1e-5
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


def _f64_attention_with_rounded_probabilities(q, kc, vc, bt, ctx, scale, bs):
    """float64 softmax, probabilities rounded to bf16, float64 P.V: what the fallback
    computes, with every step but the one rounding exact."""
    B, Hq, D = q.shape
    Hkv = kc.shape[2]
    G = Hq // Hkv
    out = np.zeros((B, Hq, D))
    for b in range(B):
        n = int(ctx[b])
        if n == 0:
            continue
        nblk = -(-n // bs)
        k = bf16_bits_to_f32(kc[bt[b, :nblk]].reshape(-1, Hkv, D)[:n]).astype(np.float64)
        v = bf16_bits_to_f32(vc[bt[b, :nblk]].reshape(-1, Hkv, D)[:n]).astype(np.float64)
        for h in range(Hq):
            s = k[:, h // G] @ bf16_bits_to_f32(q[b, h]).astype(np.float64) * scale
            p = np.exp(s - s.max())
            p /= p.sum()
            p = bf16_bits_to_f32(f32_to_bf16_bits(p.astype(np.float32))).astype(np.float64)
            out[b, h] = p @ v[:, h // G]
    return out


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2), (8, 1)])
def test_fallback_against_float64_with_the_same_rounding_step(Hq, Hkv):
    """Tighter than the 1e-2 bar: with the probabilities rounded to bf16 in an otherwise
    exact float64 computation, the fallback restatement must agree to one bf16 ulp of the
    result (its own final rounding) plus fp32 round-off.  Lengths 1 to 5 and a page
    boundary: a mask off by one moves such a short row by far more."""
    B, D, bs, NB = 8, 16, 8, 20
    ctx = [1, 2, 3, 4, 5, 8, 9, 30]
    q, kc, vc, bt, ctx = make_problem(61 + Hq, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 0.41
    want = _f64_attention_with_rounded_probabilities(q, kc, vc, bt, ctx, scale, bs)
    got = bf16_bits_to_f32(paged_attention_fallback_ref(q, kc, vc, bt, ctx, scale, bs))
    # a probability that lands on the other side of a bf16 tie in fp32 moves the result by
    # at most 2^-9 of that probability's share: allow 2^-7 relative, 2^-9 absolute
    np.testing.assert_allclose(got, want, rtol=2.0 ** -7, atol=2.0 ** -9)
    # and without the rounding step the agreement is visibly worse at these sizes
    exact = textbook_attention_f64(q, kc, vc, bt, ctx, scale, bs)
    assert np.abs(got - exact).max() > np.abs(got - want).max()


def _bad_metadata_problem():
    """Lengths beyond what the table describes and below zero, live table entries of -1
    and beyond the pool: the literal restatement defines the result (clip of the table,
    pallas_attention.py:185; mask over the MB * bs gathered positions, :216-217)."""
    B, Hq, Hkv, D, bs, NB = 5, 8, 2, 16, 8, 16
    q, kc, vc, bt, ctx = make_problem(71, B, Hq, Hkv, D, bs, NB, [24, 24, 9, 17, 24])
    ctx = ctx.copy(); bt = bt.copy()
    ctx[0] = 1000          # > MB * bs = 24: every gathered position is live
    ctx[1] = -5            # nothing is live: zeros
    bt[2, 0] = -1          # clipped to page 0
    bt[3, 1] = NB + 7      # clipped to page NB - 1
    bt[4, 2] = 2 ** 30
    return q, kc, vc, bt, ctx, 0.3, bs


@pytest.mark.parametrize("impl", ["per_seq", "c", "fallback"])
def test_out_of_range_metadata_follows_the_literal_restatement(impl):
    q, kc, vc, bt, ctx, scale, bs = _bad_metadata_problem()
    want = bf16_bits_to_f32(paged_decode_attention_vectorized_ref(q, kc, vc, bt, ctx, scale, bs))
    got = IMPLS[impl](q, kc, vc, bt, ctx, scale, bs)
    np.testing.assert_allclose(got, want, atol=1e-2, rtol=1e-2)
    assert not got[1].any()
    # and the literal restatement itself against float64 on the clipped, clamped problem
    NB = kc.shape[0]
    exact = textbook_attention_f64(q, kc, vc, np.clip(bt, 0, NB - 1),
                                   np.clip(ctx, 0, bt.shape[1] * bs), scale, bs)
    np.testing.assert_allclose(want, exact, atol=1e-2, rtol=1e-2)


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


# ---------------------------------------------------------------- QK norm + RoPE
def _rope_inputs(seed, T=6, H=3):
    from oracle.paged_attention_oracle import build_cos_sin_cache_ref
    rng = np.random.Generator(np.random.PCG64(seed))
    x = f32_to_bf16_bits(rng.standard_normal((T, H, 128), dtype=np.float32) * 3)
    w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    pos = rng.integers(0, 4096, T).astype(np.int32)
    return x, w, pos, build_cos_sin_cache_ref(128, 4096, 1e6)


def test_cos_sin_cache_against_float64():
    from oracle.paged_attention_oracle import build_cos_sin_cache_ref
    cs = build_cos_sin_cache_ref(128, 512, 1e6)
    inv = 1.0 / (1e6 ** (np.arange(0, 128, 2, dtype=np.float64) / 128))
    f = np.outer(np.arange(512, dtype=np.float64), inv)
    assert cs.shape == (512, 128) and cs.dtype == np.float32
    np.testing.assert_allclose(cs[:, :64], np.cos(f), atol=3e-5)
    np.testing.assert_allclose(cs[:, 64:], np.sin(f), atol=3e-5)
    assert np.array_equal(cs[0, :64], np.ones(64, np.float32)) and not cs[0, 64:].any()


def test_qk_norm_rope_against_float64_math():
    from oracle.paged_attention_oracle import qk_norm_rope_ref
    x, w, pos, cs = _rope_inputs(61)
    got = qk_norm_rope_ref(x, pos, cs, w, 1e-6)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    n = xf / np.sqrt((xf ** 2).mean(-1, keepdims=True) + 1e-6) * w
    c = cs[pos][:, None, :64].astype(np.float64); s = cs[pos][:, None, 64:].astype(np.float64)
    want = np.concatenate([n[..., :64] * c - n[..., 64:] * s, n[..., 64:] * c + n[..., :64] * s], -1)
    # the normalised value is rounded to bf16 before the rotation: 2^-8 relative
    np.testing.assert_allclose(got, want, atol=2e-2, rtol=2 ** -7)
    # without the norm only fp32 round-off remains
    got2 = qk_norm_rope_ref(x, pos, cs, None, 1e-6)
    want2 = np.concatenate([xf[..., :64] * c - xf[..., 64:] * s, xf[..., 64:] * c + xf[..., :64] * s], -1)
    np.testing.assert_allclose(got2, want2, atol=1e-5, rtol=1e-6)


def test_qk_norm_rope_closed_forms():
    from oracle.paged_attention_oracle import qk_norm_rope_ref
    x, w, pos, cs = _rope_inputs(62)
    ones = np.ones(128, np.float32)
    zero = np.zeros_like(pos)
    # position 0: cos = 1, sin = 0 -> rotation is the identity
    assert np.array_equal(qk_norm_rope_ref(x, zero, cs, None, 1e-6), bf16_bits_to_f32(x))
    # unit weight -> unit RMS (up to the bf16 rounding of the normalised value)
    y = qk_norm_rope_ref(x, pos, cs, ones, 1e-6)
    np.testing.assert_allclose(np.sqrt((y.astype(np.float64) ** 2).mean(-1)), 1.0, atol=3e-3)
    # the rotation preserves the norm of every (i, i + 64) pair
    y0 = qk_norm_rope_ref(x, pos, cs, None, 1e-6).astype(np.float64)
    xf = bf16_bits_to_f32(x).astype(np.float64)
    np.testing.assert_allclose(y0[..., :64] ** 2 + y0[..., 64:] ** 2,
                               xf[..., :64] ** 2 + xf[..., 64:] ** 2, rtol=1e-5, atol=1e-6)
    # q . k after rotation depends on the position difference only
    q = x[:1, :1]; k = x[1:2, :1]
    def dot(pq, pk):
        a = qk_norm_rope_ref(q, np.array([pq]), cs, None, 0).astype(np.float64)
        b = qk_norm_rope_ref(k, np.array([pk]), cs, None, 0).astype(np.float64)
        return float((a * b).sum())
    assert abs(dot(100, 40) - dot(1060, 1000)) < 1e-2 * (1 + abs(dot(100, 40)))
    assert abs(dot(100, 40) - dot(100, 41)) > 1e-3
    # out-of-range positions are clamped like a JAX gather
    big = np.array([10 ** 6] * len(pos))
    assert np.array_equal(qk_norm_rope_ref(x, big, cs, w, 1e-6),
                          qk_norm_rope_ref(x, np.full(len(pos), 4095), cs, w, 1e-6))


def test_qk_norm_rope_store_composes_the_pieces():
    from oracle.paged_attention_oracle import qk_norm_rope_ref, qk_norm_rope_store_ref
    rng = np.random.Generator(np.random.PCG64(63))
    T, Hq, Hkv = 5, 4, 2
    _, w, pos, cs = _rope_inputs(64, T=T)
    qkv = f32_to_bf16_bits(rng.standard_normal((T, (Hq + 2 * Hkv) * 128), dtype=np.float32))
    kc = rng.integers(0, 65536, (16, Hkv, 128)).astype(np.uint16)
    vc = rng.integers(0, 65536, (16, Hkv, 128)).astype(np.uint16)
    slots = np.array([3, -1, 15, 16, 0], np.int32)
    q, k2, v2 = qk_norm_rope_store_ref(qkv, pos, cs, w, w[::-1].copy(), 1e-6, kc, vc, slots, Hq, Hkv)
    qh = qkv[:, :Hq * 128].reshape(T, Hq, 128)
    kh = qkv[:, Hq * 128:(Hq + Hkv) * 128].reshape(T, Hkv, 128)
    vh = qkv[:, (Hq + Hkv) * 128:].reshape(T, Hkv, 128)
    assert np.array_equal(q, f32_to_bf16_bits(qk_norm_rope_ref(qh, pos, cs, w, 1e-6)))
    kr = f32_to_bf16_bits(qk_norm_rope_ref(kh, pos, cs, w[::-1].copy(), 1e-6))
    for t, s in enumerate(slots):
        if 0 <= s < 16:
            assert np.array_equal(k2[s], kr[t]) and np.array_equal(v2[s], vh[t])
    untouched = [i for i in range(16) if i not in (3, 15, 0)]
    assert np.array_equal(k2[untouched], kc[untouched]) and np.array_equal(v2[untouched], vc[untouched])


# ---------------------------------------------------------------- decode metadata
def test_prepare_and_advance_decode_against_a_sequence_simulation():
    """Brute force: keep Python-side sequences (token list + page list, a new page
    whenever the length crosses a page boundary, as BlockManager.may_append does)
    and rebuild the arrays from scratch every step; the in-place advance must give
    the same arrays."""
    from nanovllm_jax_amd.engine.decode_step import prepare_decode
    from oracle.paged_attention_oracle import advance_decode_ref, prepare_decode_ref
    bs = 4
    rng = np.random.Generator(np.random.PCG64(8))
    lens = [1, 3, 4, 5, 8, 11]
    free = list(range(100, 200))
    tables = [[free.pop() for _ in range(-(-n // bs))] for n in lens]
    last = rng.integers(0, 1000, len(lens)).tolist()
    ids, pos, ctx, slots, bt = prepare_decode_ref(last, lens, tables, bs)
    # the package's host filler is the same restatement
    for a, b in zip(prepare_decode(last, lens, tables, bs), (ids, pos, ctx, slots, bt)):
        assert np.array_equal(a, b)
    # hand-checked values: length 5, pages [p0, p1] -> slot p1*4 + 0; length 4 -> p0*4 + 3
    assert slots[3] == tables[3][1] * bs + 0 and slots[2] == tables[2][0] * bs + 3
    assert list(pos) == [n - 1 for n in lens] and list(ctx) == lens
    width = 6
    bt_dev = np.full((len(lens), width), -1, np.int32); bt_dev[:, :bt.shape[1]] = bt
    for step in range(9):
        nxt = rng.integers(0, 1000, len(lens))
        for i in range(len(lens)):                    # sequences append, pages are added on demand
            lens[i] += 1
            if lens[i] % bs == 1:
                tables[i].append(free.pop()); bt_dev[i, len(tables[i]) - 1] = tables[i][-1]
        want = prepare_decode_ref(nxt.tolist(), lens, tables, bs)
        ids, pos, ctx, slots = advance_decode_ref(nxt, ids, pos, ctx, slots, bt_dev, bs)
        assert np.array_equal(ids, want[0]) and np.array_equal(pos, want[1])
        assert np.array_equal(ctx, want[2]) and np.array_equal(slots, want[3])


def test_advance_decode_inactive_and_missing_page():
    from oracle.paged_attention_oracle import advance_decode_ref
    bs = 4
    ids = np.array([7, 8, 9], np.int32); pos = np.array([3, 0, 3], np.int32)
    ctx = np.array([4, 0, 4], np.int32); slots = np.array([19, 5, 23], np.int32)
    bt = np.array([[4, -1], [1, 2], [5, 6]], np.int32)
    i2, p2, c2, s2 = advance_decode_ref([70, 80, 90], ids, pos, ctx, slots, bt, bs)
    assert list(c2) == [4, 0, 5] and list(s2) == [-1, -1, 24]      # row 0: next page missing
    assert list(i2) == [7, 8, 90] and list(p2) == [3, 0, 4]


# ---------------------------------------------------------------- prefill attention
def _prefill_problem(seed, lens_q, lens_k, Hq, Hkv, D):
    rng = np.random.Generator(np.random.PCG64(seed))
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q = f32_to_bf16_bits(rng.standard_normal((cu_q[-1], Hq, D), dtype=np.float32))
    k = f32_to_bf16_bits(rng.standard_normal((cu_k[-1], Hkv, D), dtype=np.float32))
    v = f32_to_bf16_bits(rng.standard_normal((cu_k[-1], Hkv, D), dtype=np.float32))
    return q, k, v, cu_q, cu_k


@pytest.mark.parametrize("Hq,Hkv", [(2, 2), (4, 2), (4, 1)])
def test_prefill_against_fp64_brute_force(Hq, Hkv):
    from oracle.paged_attention_oracle import (textbook_prefill_f64,
                                               variable_length_attention_prefill_ref)
    lens = [1, 7, 12]
    q, k, v, cu_q, cu_k = _prefill_problem(71 + Hq, lens, lens, Hq, Hkv, 16)
    got = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, 0.4, return_f32=True)
    want = textbook_prefill_f64(q, k, v, cu_q, cu_k, 0.4)
    np.testing.assert_allclose(got, want, atol=1e-2, rtol=1e-2)   # probabilities are rounded to bf16
    # row 0 of every sequence sees one key: exactly its V row
    for i in range(len(lens)):
        np.testing.assert_allclose(got[cu_q[i]], np.repeat(bf16_bits_to_f32(v[cu_k[i]]), Hq // Hkv, 0),
                                   rtol=1e-6, atol=0)
    # unequal lengths: top-left aligned causal mask, keys beyond len_k never seen
    q2, k2, v2, cq2, ck2 = _prefill_problem(75, [6, 3], [4, 9], Hq, Hkv, 16)
    got2 = variable_length_attention_prefill_ref(q2, k2, v2, cq2, ck2, 0.4, return_f32=True)
    np.testing.assert_allclose(got2, textbook_prefill_f64(q2, k2, v2, cq2, ck2, 0.4), atol=1e-2, rtol=1e-2)


def test_prefill_against_torch_sdpa_causal_gqa_and_packing_invariance():
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    lens = [33, 5, 64]
    Hq, Hkv, D = 8, 2, 32
    q, k, v, cu_q, cu_k = _prefill_problem(81, lens, lens, Hq, Hkv, D)
    got = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, D ** -0.5, return_f32=True)
    for i, n in enumerate(lens):
        sl = slice(cu_q[i], cu_q[i + 1])
        qq = bits_to_torch(q[sl]).float().permute(1, 0, 2)[None]
        kk = bits_to_torch(k[sl]).float().permute(1, 0, 2)[None]
        vv = bits_to_torch(v[sl]).float().permute(1, 0, 2)[None]
        o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, is_causal=True,
                                                             enable_gqa=True)[0].permute(1, 0, 2)
        np.testing.assert_allclose(got[sl], o.numpy(), atol=1e-2, rtol=1e-2)
        # a batch is its sequences one by one
        alone = variable_length_attention_prefill_ref(q[sl], k[sl], v[sl], [0, n], [0, n],
                                                      D ** -0.5, return_f32=True)
        assert np.array_equal(alone, got[sl])


# ---------------------------------------------------------------------------
# RMSNorm (+ residual) and SiLU-and-multiply
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("hidden", [1024, 520, 4096])
def test_add_rms_norm_against_float64_and_torch(hidden):
    import torch
    from oracle.paged_attention_oracle import add_rms_norm_ref
    rng = np.random.Generator(np.random.PCG64(61))
    x = f32_to_bf16_bits(rng.standard_normal((5, hidden), dtype=np.float32) * 3)
    res = f32_to_bf16_bits(rng.standard_normal((5, hidden), dtype=np.float32))
    w = (1 + 0.3 * rng.standard_normal(hidden)).astype(np.float32)
    xf, rf = bf16_bits_to_f32(x).astype(np.float64), bf16_bits_to_f32(res).astype(np.float64)

    # closed form in float64 (layers/layernorm.py:41-48 and :66-76)
    def f64(s):
        return s / np.sqrt((s * s).mean(-1, keepdims=True) + 1e-6) * w

    y = bf16_bits_to_f32(add_rms_norm_ref(x, w, 1e-6))
    want = f64(xf)
    assert np.all(np.abs(y - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)       # one bf16 rounding
    y2, new_res = add_rms_norm_ref(x, w, 1e-6, res)
    want2 = f64(xf + rf)
    assert np.all(np.abs(bf16_bits_to_f32(y2) - want2) <= 2.0 ** -8 * np.abs(want2) + 1e-30)
    # the new residual is the rounding of the exact sum (a sum of two bf16 fits fp32 exactly
    # unless the exponents are far apart, where fp32 rounds first: compare through fp32)
    assert np.array_equal(new_res, f32_to_bf16_bits((xf + rf).astype(np.float32)))
    # library special case: torch's rms_norm in float32
    t = torch.nn.functional.rms_norm(torch.from_numpy(xf.astype(np.float32)), (hidden,),
                                     torch.from_numpy(w), 1e-6).numpy()
    assert np.all(np.abs(y - t) <= 2.0 ** -8 * np.abs(t) + 1e-30)
    # unit weight -> unit RMS (to bf16 precision)
    y1 = bf16_bits_to_f32(add_rms_norm_ref(x, np.ones(hidden, np.float32), 1e-6))
    assert np.allclose(np.sqrt((y1.astype(np.float64) ** 2).mean(-1)), 1.0, atol=3e-3)


def test_silu_and_mul_against_float64_torch_and_closed_forms():
    import torch
    from oracle.paged_attention_oracle import silu_and_mul_ref
    rng = np.random.Generator(np.random.PCG64(62))
    x = f32_to_bf16_bits(rng.standard_normal((4, 2 * 96), dtype=np.float32) * 4)
    g = torch.from_numpy(bf16_bits_to_f32(x[:, :96]).astype(np.float64))
    u = torch.from_numpy(bf16_bits_to_f32(x[:, 96:]).astype(np.float64))
    want = (torch.nn.functional.silu(g) * u).numpy()
    got = bf16_bits_to_f32(silu_and_mul_ref(x))
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)
    # closed forms: silu(0) = 0; a large gate passes `up` through; a large negative gate gives 0
    special = f32_to_bf16_bits(np.array([[0.0, 80.0, -200.0, 1.0, 1.5, -2.5, 3.0, 7.0]],
                                          np.float32))
    out = bf16_bits_to_f32(silu_and_mul_ref(special))
    assert out[0, 0] == 0.0
    assert out[0, 1] == np.float32(80.0 * -2.5)
    assert out[0, 2] == 0.0
    assert abs(out[0, 3] - 7.0 / (1 + np.exp(-1.0))) <= 2.0 ** -8 * 7


def test_f16_rounding_against_torch_and_special_values():
    from oracle.paged_attention_oracle import f16_bits_to_f32, f32_to_f16_bits
    rng = np.random.Generator(np.random.PCG64(63))
    x = np.concatenate([
        (rng.standard_normal(200_000) * np.exp(rng.uniform(-20, 12, 200_000))).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.9, 1e-8, 6.0e-8, 5.96e-8, 2.98e-8, 6.1e-5,
                  np.inf, -np.inf, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11], np.float32)])
    want = torch.from_numpy(x).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    got = f32_to_f16_bits(x)
    assert np.array_equal(got, want)
    # ties go to even; overflow to inf; the round trip of every finite half value is exact
    assert f32_to_f16_bits(np.array([1 + 2.0 ** -11], np.float32))[0] == 0x3C00
    assert f32_to_f16_bits(np.array([1 + 3 * 2.0 ** -11], np.float32))[0] == 0x3C02
    assert f32_to_f16_bits(np.array([65520.0], np.float32))[0] == 0x7C00
    all_bits = np.arange(0x7C00, dtype=np.uint16)
    assert np.array_equal(f32_to_f16_bits(f16_bits_to_f32(all_bits)), all_bits)


def test_c_oracle_float16_matches_the_numpy_restatement():
    """The C restatement with IEEE-half elements: store bit for bit (its f32 -> half
    rounding over subnormals, ties, overflow and NaN), decode within float32
    round-off of the NumPy restatement, same rounded output except at ties."""
    from oracle.paged_attention_oracle import (f16_bits_to_f32, f32_to_f16_bits,
                                               paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    rng = np.random.Generator(np.random.PCG64(77))
    T, Hkv, D, slots_n = 64, 2, 64, 200
    vals = (rng.standard_normal((2, T, Hkv, D)) * np.exp(rng.uniform(-20, 12, (2, T, Hkv, D)))
            ).astype(np.float32)
    vals[0, 0, 0, :8] = [65504.0, 65520.0, 65519.99, 1e-8, 6.0e-8, 2.98e-8, -0.0, np.nan]
    kc = rng.integers(0, 0x7C00, (slots_n, Hkv, D)).astype(np.uint16)
    slots = rng.permutation(slots_n)[:T].astype(np.int32)
    wk, wv = store_kv_to_cache_ref(vals[0], vals[1], kc, kc.copy(), slots, negative_slots="skip",
                                   dtype="f16")
    ck, cv = c_oracle.store_kvcache(vals[0], vals[1], kc, kc.copy(), slots, negative_slots="skip",
                                    dtype="f16")
    nan = np.isnan(f16_bits_to_f32(wk))
    assert np.array_equal(nan, np.isnan(f16_bits_to_f32(ck)))
    assert np.array_equal(np.where(nan, 0, wk), np.where(nan, 0, ck)) and np.array_equal(wv, cv)
    # every finite half value decodes to the same float in C: round trip through the store
    all_bits = np.arange(0x7C00, dtype=np.uint16).reshape(-1, 1, 64)
    allf = f16_bits_to_f32(all_bits)
    z = np.zeros_like(all_bits)
    rk, _ = c_oracle.store_kvcache(allf, allf, z, z.copy(), np.arange(all_bits.shape[0], dtype=np.int32),
                                   dtype="f16")
    assert np.array_equal(rk, all_bits)
    B, Hq, Hkv, D, bs, NB = 5, 8, 2, 128, 64, 24
    q, kc, vc, bt, ctx = make_problem(78, B, Hq, Hkv, D, bs, NB, [0, 1, 65, 200, 130])
    cv16 = lambda b: f32_to_f16_bits(bf16_bits_to_f32(b) * np.float32(1.01))
    q, kc, vc = cv16(q), cv16(kc), cv16(vc)
    want = paged_decode_attention_per_seq_ref(q, kc, vc, bt, ctx, 0.09, bs, return_f32=True,
                                              dtype="f16")
    got = c_oracle.paged_decode(q, kc, vc, bt, ctx, 0.09, bs, return_f32=True, dtype="f16")
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    got_bits = c_oracle.paged_decode(q, kc, vc, bt, ctx, 0.09, bs, dtype="f16")
    assert np.array_equal(got_bits, f32_to_f16_bits(got))


def test_paged_prefill_oracle_against_float64_and_the_packed_one():
    """The cached-prefix prefill restatement: equal to the packed one when nothing
    is cached, and to a float64 brute force (bottom-right aligned causal mask over
    the gathered pages) when a prefix is."""
    from oracle.paged_attention_oracle import (paged_prefill_attention_ref,
                                               variable_length_attention_prefill_ref)
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    rng = np.random.Generator(np.random.PCG64(91))
    Hq, Hkv, D, bs, NB = 4, 2, 128, 32, 12
    lens_k, lens_q = [70, 33, 5], [20, 33, 1]
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    kc, vc = draw_bf16_bits(rng, (NB, bs, Hkv, D)), draw_bf16_bits(rng, (NB, bs, Hkv, D))
    q = draw_bf16_bits(rng, (int(cu_q[-1]), Hq, D), 2.0)
    bt = np.full((3, 3), -1, np.int32)
    pages = rng.permutation(NB)
    used = 0
    for i, n in enumerate(lens_k):
        nb = -(-n // bs)
        bt[i, :nb] = pages[used:used + nb]
        used += nb
    got = paged_prefill_attention_ref(q, kc, vc, bt, cu_q, cu_k, 0.1, return_f32=True)
    qf = bf16_bits_to_f32(q).astype(np.float64)
    for i in range(3):
        lk, lq = lens_k[i], lens_q[i]
        kk = bf16_bits_to_f32(kc[bt[i, :-(-lk // bs)]].reshape(-1, Hkv, D)[:lk]).astype(np.float64)
        vv = bf16_bits_to_f32(vc[bt[i, :-(-lk // bs)]].reshape(-1, Hkv, D)[:lk]).astype(np.float64)
        for j in range(lq):
            n = lk - lq + j + 1
            for h in range(Hq):
                lg = 0.1 * (kk[:n, h // 2] @ qf[cu_q[i] + j, h])
                w = np.exp(lg - lg.max()); w /= w.sum()
                assert np.allclose(got[cu_q[i] + j, h], w @ vv[:n, h // 2], atol=1e-2), (i, j, h)
    # nothing cached: the packed restatement on the same rows
    lens = [40, 7]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k = draw_bf16_bits(rng, (47, Hkv, D)); v = draw_bf16_bits(rng, (47, Hkv, D))
    q = draw_bf16_bits(rng, (47, Hq, D))
    kc2 = np.zeros((4, bs, Hkv, D), np.uint16); vc2 = np.zeros_like(kc2)
    bt2 = np.array([[2, 0], [3, -1]], np.int32)
    for i, n in enumerate(lens):
        for p in range(n):
            kc2[bt2[i, p // bs], p % bs] = k[cu[i] + p]; vc2[bt2[i, p // bs], p % bs] = v[cu[i] + p]
    a = paged_prefill_attention_ref(q, kc2, vc2, bt2, cu, cu, 0.1)
    b = variable_length_attention_prefill_ref(q, k, v, cu, cu, 0.1)
    assert np.array_equal(a, b)
