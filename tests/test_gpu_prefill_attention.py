"""GPU parity of the HIP variable-length causal prefill attention against the
CPU oracle (atol/rtol 1e-2, bf16 out, fp32 accumulate), through the C ABI."""
import numpy as np
import pytest

from helpers import assert_close_bf16, bits_to_torch, torch_to_bits

pytestmark = pytest.mark.gpu


def _problem(seed, lens_q, lens_k, Hq, Hkv, D=128, gain=1.0):
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    rng = np.random.Generator(np.random.PCG64(seed))
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q = draw_bf16_bits(rng, (int(cu_q[-1]), Hq, D), gain)
    k = draw_bf16_bits(rng, (max(int(cu_k[-1]), 1), Hkv, D))
    v = draw_bf16_bits(rng, (max(int(cu_k[-1]), 1), Hkv, D))
    return q, k, v, cu_q, cu_k


def run_hip(q, k, v, cu_q, cu_k, scale):
    import torch
    from nanovllm_jax_amd import variable_length_attention_prefill
    dev = "cuda:0"
    out = variable_length_attention_prefill(
        bits_to_torch(q, dev), bits_to_torch(k, dev), bits_to_torch(v, dev),
        torch.from_numpy(cu_q).to(dev), torch.from_numpy(cu_k).to(dev), scale=scale)
    torch.cuda.synchronize()
    return torch_to_bits(out)


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (16, 8), (32, 8), (8, 1)])
def test_prefill_ragged_batch(Hq, Hkv):
    print(f"case prefill ragged Hq={Hq} Hkv={Hkv}", flush=True)
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    lens = [1, 31, 32, 33, 127, 128, 129, 300, 17]
    q, k, v, cu_q, cu_k = _problem(10 + Hq, lens, lens, Hq, Hkv)
    scale = 128 ** -0.5
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, scale)
    got = run_hip(q, k, v, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what=f"prefill Hq={Hq} Hkv={Hkv}")
    G = Hq // Hkv
    for i in range(len(lens)):                    # first row of a sequence == its first V row
        assert np.array_equal(got[cu_q[i]], np.repeat(v[cu_k[i]], G, axis=0))


@pytest.mark.parametrize("batch", [65, 130, 300, 600])
def test_prefill_batches_of_many_short_prompts(batch):
    """More sequences than the 64 a wave looks at together, and than the 256 whose
    lengths it fetches in one go, when it finds the sequence of a query tile: short
    prompts, empty ones and a few longer than a tile among them."""
    print(f"case prefill many prompts batch={batch}", flush=True)
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    rng = np.random.Generator(np.random.PCG64(700 + batch))
    lens = rng.integers(0, 41, size=batch)
    lens[rng.integers(0, batch, size=5)] = [129, 257, 128, 1, 300]
    lens[[0, 63, 64, batch - 1]] = [3, 130, 0, 131]
    lens = [int(x) for x in lens]
    q, k, v, cu_q, cu_k = _problem(710 + batch, lens, lens, 4, 2)
    scale = 128 ** -0.5
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, scale)
    got = run_hip(q, k, v, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what=f"prefill {batch} prompts")
    for i in range(batch):                        # first row of a sequence == its first V row
        if lens[i] > 0:
            assert np.array_equal(got[cu_q[i]], np.repeat(v[cu_k[i]], 2, axis=0)), i


def test_prefill_reference_smoke_lengths():
    """Sequence lengths of the reference's prefill smoke test
    (test_mosaic_kernels.py:90-159): 512, 768, 1024, 1536; Hq=32, Hkv=8, D=128."""
    print("case prefill reference smoke lengths", flush=True)
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    lens = [512, 768, 1024, 1536]
    q, k, v, cu_q, cu_k = _problem(20, lens, lens, 32, 8)
    scale = 128 ** -0.5
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, scale)
    got = run_hip(q, k, v, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what="prefill smoke lengths")


def test_prefill_unequal_q_and_k_lengths_and_empty_sequences():
    print("case prefill unequal lengths / empty", flush=True)
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    lens_q = [40, 0, 5, 200, 64]
    lens_k = [12, 7, 90, 200, 0]
    q, k, v, cu_q, cu_k = _problem(30, lens_q, lens_k, 16, 8)
    scale = 128 ** -0.5
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, scale)
    got = run_hip(q, k, v, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what="prefill unequal")
    assert not got[cu_q[4]:cu_q[5]].any()         # no keys at all -> zeros


def test_prefill_sharp_softmax_and_packing_invariance():
    print("case prefill sharp softmax / packing", flush=True)
    from oracle.paged_attention_oracle import variable_length_attention_prefill_ref
    lens = [257, 100]
    q, k, v, cu_q, cu_k = _problem(40, lens, lens, 16, 8, gain=4.0)
    scale = 128 ** -0.5
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, scale)
    got = run_hip(q, k, v, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what="prefill sharp")
    alone = run_hip(q[cu_q[1]:], k[cu_k[1]:], v[cu_k[1]:], np.array([0, 100], np.int32),
                    np.array([0, 100], np.int32), scale)
    assert np.array_equal(alone, got[cu_q[1]:])


def test_attention_layer_prefill_then_decode():
    """Attention.__call__ in prefill mode stores the prompt's K/V through
    slot_mapping and attends over the packed rows; a decode step over the same
    cache then equals the last prefill row recomputed (same keys, same query)."""
    print("case Attention prefill then decode", flush=True)
    import torch
    from nanovllm_jax_amd import Attention, create_decode_context, create_prefill_context
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    from oracle.paged_attention_oracle import (store_kv_to_cache_ref,
                                               variable_length_attention_prefill_ref)
    Hq, Hkv, D, bs, NB = 16, 8, 128, 256, 8
    lens = [300, 77]
    q, k, v, cu_q, cu_k = _problem(50, lens, lens, Hq, Hkv)
    tables = [[3, 5], [6]]
    slots = np.concatenate([np.concatenate([np.arange(p * bs, p * bs + min(bs, n - j * bs))
                                            for j, p in enumerate(t)])
                            for t, n in zip(tables, lens)]).astype(np.int32)
    dev = "cuda:0"
    attn = Attention(Hq, D, D ** -0.5, Hkv, bs)
    kc = np.zeros((NB, bs, Hkv, D), np.uint16)
    attn.set_kv_cache(bits_to_torch(kc, dev), bits_to_torch(kc.copy(), dev))
    up = lambda a: torch.from_numpy(a).to(dev)
    ctx = create_prefill_context(up(cu_q), up(cu_k), max(lens), max(lens), up(slots))
    out = attn(bits_to_torch(q, dev), bits_to_torch(k, dev), bits_to_torch(v, dev), ctx)
    torch.cuda.synchronize()
    want = variable_length_attention_prefill_ref(q, k, v, cu_q, cu_k, D ** -0.5)
    assert_close_bf16(torch_to_bits(out), want, what="layer prefill")
    flat = (-1, Hkv, D)
    wk, wv = store_kv_to_cache_ref(k, v, kc.reshape(flat), kc.reshape(flat), slots, negative_slots="skip")
    assert np.array_equal(torch_to_bits(attn.k_cache).reshape(flat), wk)
    assert np.array_equal(torch_to_bits(attn.v_cache).reshape(flat), wv)
    # decode with the last prompt token as the query, its K/V already in the cache
    last = cu_q[1:] - 1
    bt = np.array([[3, 5], [6, -1]], np.int32)
    dctx = create_decode_context(up(np.array(lens, np.int32)),
                                 up(np.array([-1, -1], np.int32)), up(bt))
    dq = bits_to_torch(q[last], dev)
    dout = attn(dq, bits_to_torch(k[last], dev), bits_to_torch(v[last], dev), dctx)
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(dout), want[last], what="decode == last prefill row")


# ---- prefill behind a cached prefix: keys and values from the paged cache ----
def _paged_problem(seed, lens_k, lens_q, Hq, Hkv, bs, extra_pages=3):
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    rng = np.random.Generator(np.random.PCG64(seed))
    D = 128
    B = len(lens_k)
    nblk = [-(-n // bs) for n in lens_k]
    NB = sum(nblk) + extra_pages
    kc, vc = draw_bf16_bits(rng, (NB, bs, Hkv, D)), draw_bf16_bits(rng, (NB, bs, Hkv, D))
    cu_q = np.concatenate([[0], np.cumsum(lens_q)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)
    q = draw_bf16_bits(rng, (max(int(cu_q[-1]), 1), Hq, D), 2.0)[:int(cu_q[-1])]
    bt = np.full((B, max(max(nblk), 1) + 1), -1, np.int32)       # one padding column
    pages = rng.permutation(NB)
    used = 0
    for i, n in enumerate(nblk):
        bt[i, :n] = pages[used:used + n]
        used += n
    return q, kc, vc, bt, cu_q, cu_k


def run_hip_paged(q, kc, vc, bt, cu_q, cu_k, scale):
    import torch
    from nanovllm_jax_amd import paged_prefill_attention
    dev = "cuda:0"
    out = paged_prefill_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev),
                                  bits_to_torch(vc, dev), torch.from_numpy(bt).to(dev),
                                  torch.from_numpy(cu_q).to(dev), torch.from_numpy(cu_k).to(dev),
                                  scale)
    torch.cuda.synchronize()
    return torch_to_bits(out)


@pytest.mark.parametrize("Hq,Hkv,bs", [(8, 2, 32), (16, 8, 64), (32, 8, 256), (4, 4, 96)])
def test_paged_prefill_behind_a_cached_prefix(Hq, Hkv, bs):
    """Prompt chunks of many lengths behind prefixes of many lengths (none, shorter
    and longer than a page, ending on and off page and tile boundaries), pages in
    random order, padding table entries, garbage in unused pages."""
    print(f"case paged prefill Hq={Hq} Hkv={Hkv} bs={bs}", flush=True)
    from oracle.paged_attention_oracle import paged_prefill_attention_ref
    lens_q = [1, 33, 128, 129, 40, 300, 5, 64]
    prefix = [0, 31, 32, 500, 257, 0, 700, 64]
    lens_k = [a + b for a, b in zip(lens_q, prefix)]
    q, kc, vc, bt, cu_q, cu_k = _paged_problem(70 + Hq + bs, lens_k, lens_q, Hq, Hkv, bs)
    scale = 128 ** -0.5
    want = paged_prefill_attention_ref(q, kc, vc, bt, cu_q, cu_k, scale)
    got = run_hip_paged(q, kc, vc, bt, cu_q, cu_k, scale)
    assert_close_bf16(got, want, what="paged prefill")
    # poison everything no live key sits on: the result must not move
    live = np.zeros(kc.shape[:2], bool)
    for i, n in enumerate(lens_k):
        for p in range(n):
            live[bt[i, p // bs], p % bs] = True
    kc2, vc2 = kc.copy(), vc.copy()
    kc2[~live] = 0x7FC0
    vc2[~live] = 0x7FC0                                           # NaN
    bt2 = np.where(bt < 0, 10 ** 6, bt).astype(np.int32)          # padding entries out of range
    got2 = run_hip_paged(q, kc2, vc2, bt2, cu_q, cu_k, scale)
    assert np.array_equal(got, got2), "something outside the live keys was read"


def test_paged_prefill_without_prefix_equals_packed_prefill_bit_for_bit():
    print("case paged prefill == packed prefill", flush=True)
    lens = [300, 77, 1, 129]
    Hq, Hkv, bs = 16, 8, 64
    q, kc, vc, bt, cu_q, cu_k = _paged_problem(81, lens, lens, Hq, Hkv, bs)
    # the packed rows are the live cache rows in sequence order
    k = np.concatenate([kc[bt[i, p // bs], p % bs][None] for i, n in enumerate(lens) for p in range(n)])
    v = np.concatenate([vc[bt[i, p // bs], p % bs][None] for i, n in enumerate(lens) for p in range(n)])
    scale = 0.11
    packed = run_hip(q, k, v, cu_q, cu_k, scale)
    paged = run_hip_paged(q, kc, vc, bt, cu_q, cu_k, scale)
    assert np.array_equal(packed, paged)


def test_attention_layer_prefill_with_cached_prefix():
    """Attention.__call__ with a prefill context that carries block_tables (the
    reference's filler sets them when a prefix is cached): the chunk's K/V rows are
    stored, then the chunk attends over prefix + chunk from the cache; a decode step
    with the chunk's last token as the query sees the same keys."""
    print("case Attention prefill behind a cached prefix", flush=True)
    import torch
    from nanovllm_jax_amd import Attention, create_decode_context, create_prefill_context
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    from oracle.paged_attention_oracle import (paged_prefill_attention_ref,
                                               store_kv_to_cache_ref)
    Hq, Hkv, D, bs = 16, 8, 128, 64
    prefix, chunk = [100, 0, 64], [60, 130, 7]
    lens_k = [a + b for a, b in zip(prefix, chunk)]
    q, kc, vc, bt, cu_q, cu_k = _paged_problem(82, lens_k, chunk, Hq, Hkv, bs)
    rng = np.random.Generator(np.random.PCG64(83))
    k_new = draw_bf16_bits(rng, (int(cu_q[-1]), Hkv, D))
    v_new = draw_bf16_bits(rng, (int(cu_q[-1]), Hkv, D))
    slots = np.concatenate([bt[i, np.arange(prefix[i], lens_k[i]) // bs] * bs +
                            np.arange(prefix[i], lens_k[i]) % bs for i in range(3)]).astype(np.int32)
    dev = "cuda:0"
    up = lambda a: torch.from_numpy(a).to(dev)
    attn = Attention(Hq, D, D ** -0.5, Hkv, bs)
    attn.set_kv_cache(bits_to_torch(kc, dev), bits_to_torch(vc, dev))
    ctx = create_prefill_context(up(cu_q), up(cu_k), max(chunk), max(lens_k), up(slots),
                                 block_tables=up(bt))
    out = attn(bits_to_torch(q, dev), bits_to_torch(k_new, dev), bits_to_torch(v_new, dev), ctx)
    torch.cuda.synchronize()
    flat = (-1, Hkv, D)
    wk, wv = store_kv_to_cache_ref(k_new, v_new, kc.reshape(flat), vc.reshape(flat), slots,
                                   negative_slots="skip")
    assert np.array_equal(torch_to_bits(attn.k_cache).reshape(flat), wk)
    want = paged_prefill_attention_ref(q, wk.reshape(kc.shape), wv.reshape(vc.shape), bt, cu_q,
                                       cu_k, D ** -0.5)
    assert_close_bf16(torch_to_bits(out), want, what="layer prefill behind a prefix")
    last = cu_q[1:] - 1
    dctx = create_decode_context(up(np.array(lens_k, np.int32)), up(np.full(3, -1, np.int32)),
                                 up(bt))
    dout = attn(bits_to_torch(q[last], dev), bits_to_torch(k_new[last], dev),
                bits_to_torch(v_new[last], dev), dctx)
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(dout), want[last], what="decode == last chunk row")
