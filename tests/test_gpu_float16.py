"""float16 caches (the reference's cache dtype is its model dtype, and its own
timing scripts use float16: profile_attention.py:27-30): KV store bit-exact,
decode attention within atol/rtol 1e-2 of the oracle, in every split mode."""
import numpy as np
import pytest

from helpers import make_problem

pytestmark = pytest.mark.gpu


def _to_f16(bits, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.float16).to(dev)


def _bits(t):
    import torch
    assert t.dtype == torch.float16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def _as_f16_problem(seed, B, Hq, Hkv, D, bs, NB, ctx, gain=1.0):
    """The bf16 generator's values re-rounded to float16 bit patterns."""
    from oracle.paged_attention_oracle import bf16_bits_to_f32, f32_to_f16_bits
    q, kc, vc, bt, ctx = make_problem(seed, B, Hq, Hkv, D, bs, NB, ctx, q_gain=gain)
    cv = lambda b: f32_to_f16_bits(bf16_bits_to_f32(b) * np.float32(1.001))   # not bf16-exact values
    return cv(q), cv(kc), cv(vc), bt, ctx


@pytest.mark.parametrize("chunk", [0, 64, -1])
@pytest.mark.parametrize("Hq,Hkv,D", [(32, 8, 128), (16, 8, 128), (8, 2, 64), (32, 1, 128)])
def test_decode_float16(Hq, Hkv, D, chunk):
    print(f"case f16 decode Hq={Hq} Hkv={Hkv} D={D} chunk={chunk}", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    from oracle.paged_attention_oracle import f16_bits_to_f32, paged_decode_attention_per_seq_ref
    B, bs, NB = 9, 64, 60
    ctx = [0, 1, 33, 64, 100, 257, 300, 31, 129]
    q, kc, vc, bt, ctx = _as_f16_problem(800 + Hq + D, B, Hq, Hkv, D, bs, NB, ctx, gain=2.0)
    dev = "cuda:0"
    scale = 1.0 / np.sqrt(D)
    out = paged_attention(_to_f16(q, dev), _to_f16(kc, dev), _to_f16(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), scale, bs,
                          chunk=chunk)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    got = f16_bits_to_f32(_bits(out)).astype(np.float64)
    want = f16_bits_to_f32(paged_decode_attention_per_seq_ref(q, kc, vc, bt, ctx, scale, bs,
                                                              dtype="f16")).astype(np.float64)
    err = np.abs(got - want)
    assert np.all(err <= 1e-2 + 1e-2 * np.abs(want)), f"max err {err.max():.3e}"
    assert not got[0].any()                                     # ctx = 0 -> zeros
    v_first = f16_bits_to_f32(vc[bt[1, 0], 0])                  # ctx = 1 -> the V row itself
    assert np.array_equal(got[1], np.repeat(v_first, Hq // Hkv, axis=0))


@pytest.mark.parametrize("k_f32,v_f32", [(True, False), (False, False), (True, True)])
def test_store_float16_bit_exact(k_f32, v_f32):
    print(f"case f16 store k_f32={k_f32} v_f32={v_f32}", flush=True)
    import torch
    from nanovllm_jax_amd import store_kv_to_cache
    from oracle.paged_attention_oracle import f32_to_f16_bits, store_kv_to_cache_ref
    rng = np.random.Generator(np.random.PCG64(820))
    T, Hkv, D, slots_n = 37, 8, 128, 500
    vals = (rng.standard_normal((2, T, Hkv, D)) * np.exp(rng.uniform(-18, 11, (2, T, Hkv, D)))
            ).astype(np.float32)
    vals[0, 0, 0, :6] = [65504.0, 65520.0, 1e-8, 6.0e-8, -0.0, 1 + 2.0 ** -11]   # edge values
    kc = rng.integers(0, 0x7C00, (slots_n, Hkv, D)).astype(np.uint16)
    vc = rng.integers(0, 0x7C00, (slots_n, Hkv, D)).astype(np.uint16)
    slots = rng.permutation(slots_n)[:T].astype(np.int32)
    slots[3], slots[5] = -1, slots_n + 7                          # skipped / dropped
    dev = "cuda:0"
    k_in = vals[0] if k_f32 else f32_to_f16_bits(vals[0])
    v_in = vals[1] if v_f32 else f32_to_f16_bits(vals[1])
    up = lambda a: torch.from_numpy(a).to(dev) if a.dtype == np.float32 else _to_f16(a, dev)
    kct, vct = _to_f16(kc, dev), _to_f16(vc, dev)
    store_kv_to_cache(up(k_in), up(v_in), kct, vct, torch.from_numpy(slots).to(dev))
    torch.cuda.synchronize()
    wk, wv = store_kv_to_cache_ref(k_in, v_in, kc, vc, slots, negative_slots="skip", dtype="f16")
    assert np.array_equal(_bits(kct), wk), "K cache not bit-exact"
    assert np.array_equal(_bits(vct), wv), "V cache not bit-exact"


def test_mixed_dtypes_are_refused():
    import torch
    from nanovllm_jax_amd import paged_attention, store_kv_to_cache
    dev = "cuda:0"
    q = torch.zeros((1, 8, 128), dtype=torch.float16, device=dev)
    kc = torch.zeros((2, 64, 8, 128), dtype=torch.bfloat16, device=dev)
    bt = torch.zeros((1, 1), dtype=torch.int32, device=dev)
    ctx = torch.ones(1, dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        paged_attention(q, kc, kc, bt, ctx, 0.1, 64)               # f16 q, bf16 cache
    k = torch.zeros((1, 8, 128), dtype=torch.float16, device=dev)
    with pytest.raises(ValueError):
        store_kv_to_cache(k, k, kc.view(-1, 8, 128), kc.view(-1, 8, 128),
                          torch.zeros(1, dtype=torch.int32, device=dev))   # f16 rows, bf16 cache


def test_prefill_float16():
    print("case f16 prefill", flush=True)
    import torch
    from nanovllm_jax_amd import variable_length_attention_prefill
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    from oracle.paged_attention_oracle import (bf16_bits_to_f32, f16_bits_to_f32, f32_to_f16_bits,
                                               variable_length_attention_prefill_ref)
    rng = np.random.Generator(np.random.PCG64(830))
    lens = [1, 33, 128, 300, 0, 517]
    Hq, Hkv, D = 16, 4, 128
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cv = lambda b: f32_to_f16_bits(bf16_bits_to_f32(b) * np.float32(1.001))
    q = cv(draw_bf16_bits(rng, (int(cu[-1]), Hq, D), 2.0))
    k = cv(draw_bf16_bits(rng, (int(cu[-1]), Hkv, D)))
    v = cv(draw_bf16_bits(rng, (int(cu[-1]), Hkv, D)))
    dev = "cuda:0"
    scale = D ** -0.5
    out = variable_length_attention_prefill(_to_f16(q, dev), _to_f16(k, dev), _to_f16(v, dev),
                                            torch.from_numpy(cu).to(dev),
                                            torch.from_numpy(cu).to(dev), scale=scale)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    got = f16_bits_to_f32(_bits(out)).astype(np.float64)
    want = f16_bits_to_f32(variable_length_attention_prefill_ref(q, k, v, cu, cu, scale,
                                                                 dtype="f16")).astype(np.float64)
    err = np.abs(got - want)
    assert np.all(err <= 1e-2 + 1e-2 * np.abs(want)), f"max err {err.max():.3e}"
    assert np.array_equal(got[0], np.repeat(f16_bits_to_f32(v[0]), Hq // Hkv, axis=0))  # 1 key


def test_attention_layer_with_float16_caches_prefill_then_decode():
    """The layer call of the reference (layers/attention.py:436-480) on a float16
    model: store + prefill attention, then store + decode attention over the
    same cache, every result float16."""
    print("case f16 Attention layer prefill then decode", flush=True)
    import torch
    from nanovllm_jax_amd import Attention, create_decode_context, create_prefill_context
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    from oracle.paged_attention_oracle import (bf16_bits_to_f32, f16_bits_to_f32, f32_to_f16_bits,
                                               paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref,
                                               variable_length_attention_prefill_ref)
    rng = np.random.Generator(np.random.PCG64(840))
    Hq, Hkv, D, bs, NB = 8, 2, 128, 64, 12
    lens = [70, 5, 129]
    B = len(lens)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    cv = lambda b: f32_to_f16_bits(bf16_bits_to_f32(b))
    q, k, v = (cv(draw_bf16_bits(rng, (T, h, D))) for h in (Hq, Hkv, Hkv))
    pages = rng.permutation(NB)
    bt = np.full((B, 3), -1, np.int32)
    slots = np.zeros(T, np.int32)
    used = 0
    for b, n in enumerate(lens):
        nb = -(-n // bs)
        bt[b, :nb] = pages[used:used + nb]
        used += nb
        pos = np.arange(n)
        slots[cu[b]:cu[b + 1]] = bt[b, pos // bs] * bs + pos % bs
    dev = "cuda:0"
    kc = torch.zeros((NB, bs, Hkv, D), dtype=torch.float16, device=dev)
    vc = torch.zeros_like(kc)
    attn = Attention(Hq, D, D ** -0.5, Hkv, bs)
    attn.set_kv_cache(kc, vc)
    ctx = create_prefill_context(torch.from_numpy(cu).to(dev), torch.from_numpy(cu).to(dev),
                                 max(lens), max(lens), torch.from_numpy(slots).to(dev))
    out = attn(_to_f16(q, dev), _to_f16(k, dev), _to_f16(v, dev), ctx)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    want = variable_length_attention_prefill_ref(q, k, v, cu, cu, D ** -0.5, dtype="f16")
    err = np.abs(f16_bits_to_f32(_bits(out)).astype(np.float64) - f16_bits_to_f32(want))
    assert np.all(err <= 1e-2 + 1e-2 * np.abs(f16_bits_to_f32(want))), f"prefill {err.max():.3e}"
    flat = (NB * bs, Hkv, D)
    zero = np.zeros(flat, np.uint16)
    wk, wv = store_kv_to_cache_ref(k, v, zero, zero.copy(), slots, negative_slots="skip",
                                   dtype="f16")
    assert np.array_equal(_bits(kc).reshape(flat), wk) and np.array_equal(_bits(vc).reshape(flat), wv)
    # one decode step on top
    q1, k1, v1 = (cv(draw_bf16_bits(rng, (B, h, D))) for h in (Hq, Hkv, Hkv))
    new_len = np.array(lens, np.int32) + 1
    slot1 = np.array([bt[b, (n - 1) // bs] * bs + (n - 1) % bs for b, n in enumerate(new_len)],
                     np.int32)
    dctx = create_decode_context(torch.from_numpy(new_len).to(dev), torch.from_numpy(slot1).to(dev),
                                 torch.from_numpy(bt).to(dev))
    out1 = attn(_to_f16(q1, dev), _to_f16(k1, dev), _to_f16(v1, dev), dctx)
    torch.cuda.synchronize()
    wk, wv = store_kv_to_cache_ref(k1, v1, wk, wv, slot1, negative_slots="skip", dtype="f16")
    want1 = paged_decode_attention_per_seq_ref(q1, wk.reshape(NB, bs, Hkv, D),
                                               wv.reshape(NB, bs, Hkv, D), bt, new_len, D ** -0.5,
                                               bs, dtype="f16")
    err = np.abs(f16_bits_to_f32(_bits(out1)).astype(np.float64) - f16_bits_to_f32(want1))
    assert np.all(err <= 1e-2 + 1e-2 * np.abs(f16_bits_to_f32(want1))), f"decode {err.max():.3e}"


def test_paged_prefill_float16():
    print("case f16 paged prefill", flush=True)
    import torch
    from nanovllm_jax_amd import paged_prefill_attention
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    from oracle.paged_attention_oracle import (bf16_bits_to_f32, f16_bits_to_f32, f32_to_f16_bits,
                                               paged_prefill_attention_ref)
    rng = np.random.Generator(np.random.PCG64(850))
    Hq, Hkv, D, bs = 8, 2, 128, 64
    lens_q, prefix = [40, 129, 1], [100, 0, 63]
    lens_k = [a + b for a, b in zip(lens_q, prefix)]
    nblk = [-(-n // bs) for n in lens_k]
    NB = sum(nblk) + 1
    cv = lambda b: f32_to_f16_bits(bf16_bits_to_f32(b) * np.float32(1.001))
    kc, vc = cv(draw_bf16_bits(rng, (NB, bs, Hkv, D))), cv(draw_bf16_bits(rng, (NB, bs, Hkv, D)))
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q = cv(draw_bf16_bits(rng, (int(cu_q[-1]), Hq, D), 2.0))
    bt = np.full((3, max(nblk)), -1, np.int32)
    pages = rng.permutation(NB)
    used = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = pages[used:used + n]
        used += n
    dev = "cuda:0"
    scale = D ** -0.5
    out = paged_prefill_attention(_to_f16(q, dev), _to_f16(kc, dev), _to_f16(vc, dev),
                                  torch.from_numpy(bt).to(dev), torch.from_numpy(cu_q).to(dev),
                                  torch.from_numpy(cu_k).to(dev), scale)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    got = f16_bits_to_f32(_bits(out)).astype(np.float64)
    want = f16_bits_to_f32(paged_prefill_attention_ref(q, kc, vc, bt, cu_q, cu_k, scale,
                                                       dtype="f16")).astype(np.float64)
    err = np.abs(got - want)
    assert np.all(err <= 1e-2 + 1e-2 * np.abs(want)), f"max err {err.max():.3e}"
