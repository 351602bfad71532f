"""GPU parity of the HIP KV-cache store against the CPU oracle: bit-exact."""
import numpy as np
import pytest

from helpers import bits_to_torch, torch_to_bits

pytestmark = pytest.mark.gpu


def run_store(key, value, kc, vc, slots):
    """key/value: float32 arrays or uint16 bf16 bits.  Returns new cache bits."""
    import torch
    from nanovllm_jax_amd import store_kv_to_cache
    dev = "cuda:0"

    def up(x):
        return bits_to_torch(x, dev) if x.dtype == np.uint16 else torch.from_numpy(x).to(dev)

    kct, vct = bits_to_torch(kc, dev), bits_to_torch(vc, dev)
    k2, v2 = store_kv_to_cache(up(key), up(value), kct, vct, torch.from_numpy(slots).to(dev))
    torch.cuda.synchronize()
    assert k2 is kct and v2 is vct, "store must update the caller's tensors in place"
    return torch_to_bits(kct), torch_to_bits(vct)


def _problem(seed, T, Hkv, D, num_slots, f32_k=True, f32_v=False):
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    rng = np.random.Generator(np.random.PCG64(seed))
    kc = draw_bf16_bits(rng, (num_slots, Hkv, D))
    vc = draw_bf16_bits(rng, (num_slots, Hkv, D))
    key = rng.standard_normal((T, Hkv, D), dtype=np.float32) if f32_k else draw_bf16_bits(rng, (T, Hkv, D))
    val = rng.standard_normal((T, Hkv, D), dtype=np.float32) if f32_v else draw_bf16_bits(rng, (T, Hkv, D))
    slots = rng.permutation(num_slots)[:T].astype(np.int32)
    return key, val, kc, vc, slots


@pytest.mark.parametrize("f32_k,f32_v", [(True, False), (False, False), (True, True), (False, True)])
@pytest.mark.parametrize("T", [1, 8, 257])
def test_store_bit_exact(T, f32_k, f32_v):
    print(f"case store T={T} f32_k={f32_k} f32_v={f32_v}", flush=True)
    from oracle.paged_attention_oracle import store_kv_to_cache_ref
    key, val, kc, vc, slots = _problem(3 + T, T, 8, 128, 2048, f32_k, f32_v)
    gk, gv = run_store(key, val, kc, vc, slots)
    wk, wv = store_kv_to_cache_ref(key, val, kc, vc, slots, negative_slots="skip")
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
    # with unique in-range slots the skip contract and the reference's literal code agree
    rk, rv = store_kv_to_cache_ref(key, val, kc, vc, slots, negative_slots="reference")
    assert np.array_equal(gk, rk) and np.array_equal(gv, rv)


def test_store_special_values_round_to_nearest_even():
    """Ties, subnormals, infinities, NaN, negative zero, largest finite."""
    print("case store special values", flush=True)
    from oracle.paged_attention_oracle import store_kv_to_cache_ref
    Hkv, D = 8, 128
    specials = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF, 0x7F800000,
                         0xFF800000, 0x7FC00000, 0x7F800001, 0x80000000, 0x00000001, 0x00008000,
                         0x00018000, 0x7F7F8000, 0xFFFFFFFF, 0x3EFFFFFF], dtype=np.uint32)
    key = np.resize(specials, Hkv * D).view(np.float32).reshape(1, Hkv, D).copy()
    val = key[..., ::-1].copy()
    kc = np.zeros((4, Hkv, D), np.uint16); vc = np.zeros((4, Hkv, D), np.uint16)
    slots = np.array([2], np.int32)
    gk, gv = run_store(key, val, kc, vc, slots)
    wk, wv = store_kv_to_cache_ref(key, val, kc, vc, slots, negative_slots="skip")
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)


def test_store_skip_drop_and_empty():
    print("case store skip/drop/empty", flush=True)
    from oracle.paged_attention_oracle import store_kv_to_cache_ref
    key, val, kc, vc, slots = _problem(5, 6, 8, 128, 64)
    slots = np.array([-1, 5, 64, 1 << 30, 0, -12345], np.int32)   # skip, ok, drop, drop, ok, skip
    gk, gv = run_store(key, val, kc, vc, slots)
    wk, wv = store_kv_to_cache_ref(key, val, kc, vc, slots, negative_slots="skip")
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
    touched = np.zeros(64, bool); touched[[5, 0]] = True
    assert np.array_equal(gk[~touched], kc[~touched]) and np.array_equal(gv[~touched], vc[~touched])
    # no tokens at all
    e = np.zeros((0, 8, 128), np.float32)
    gk, gv = run_store(e, e.copy(), kc, vc, np.zeros(0, np.int32))
    assert np.array_equal(gk, kc) and np.array_equal(gv, vc)


def test_store_idempotent_and_4d_cache():
    print("case store idempotent / 4-D cache", flush=True)
    import torch
    from nanovllm_jax_amd import store_kv_to_cache
    from oracle.paged_attention_oracle import store_kv_to_cache_ref
    key, val, kc, vc, slots = _problem(9, 16, 8, 128, 4 * 256)
    dev = "cuda:0"
    kct = bits_to_torch(kc, dev).view(4, 256, 8, 128); vct = bits_to_torch(vc, dev).view(4, 256, 8, 128)
    kt, vt, st = torch.from_numpy(key).to(dev), bits_to_torch(val, dev), torch.from_numpy(slots).to(dev)
    store_kv_to_cache(kt, vt, kct, vct, st)
    once = torch_to_bits(kct).reshape(-1, 8, 128), torch_to_bits(vct).reshape(-1, 8, 128)
    store_kv_to_cache(kt, vt, kct, vct, st)
    twice = torch_to_bits(kct).reshape(-1, 8, 128), torch_to_bits(vct).reshape(-1, 8, 128)
    wk, wv = store_kv_to_cache_ref(key, val, kc, vc, slots, negative_slots="skip")
    assert np.array_equal(once[0], wk) and np.array_equal(once[1], wv)
    assert np.array_equal(twice[0], wk) and np.array_equal(twice[1], wv)


def test_store_then_decode_sees_the_new_row():
    """Store before read inside one step (layers/attention.py:456-480): the
    decode call must attend over the row written by the store of the same step."""
    print("case store then decode (C1 layer call)", flush=True)
    import torch
    from nanovllm_jax_amd import Attention, create_decode_context
    from nanovllm_jax_amd.workloads import draw_bf16_bits, make_workload
    from oracle.paged_attention_oracle import (paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    from helpers import assert_close_bf16
    w = make_workload("C1")
    rng = np.random.Generator(np.random.PCG64(77))
    shape = (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
    kc, vc = draw_bf16_bits(rng, shape), draw_bf16_bits(rng, shape)
    q = draw_bf16_bits(rng, (w.batch, w.num_heads, w.head_dim))
    k_new = (rng.standard_normal((w.batch, w.num_kv_heads, w.head_dim), dtype=np.float32) * 3)
    v_new = draw_bf16_bits(rng, (w.batch, w.num_kv_heads, w.head_dim), gain=3.0)
    dev = "cuda:0"
    attn = Attention(w.num_heads, w.head_dim, w.scale, w.num_kv_heads, w.block_size)
    attn.set_kv_cache(bits_to_torch(kc, dev), bits_to_torch(vc, dev))
    ctx = create_decode_context(torch.from_numpy(w.context_lens).to(dev),
                                torch.from_numpy(w.slot_mapping).to(dev),
                                torch.from_numpy(w.block_tables).to(dev))
    out = attn(bits_to_torch(q, dev), torch.from_numpy(k_new).to(dev), bits_to_torch(v_new, dev), ctx)
    torch.cuda.synchronize()
    flat = (-1, w.num_kv_heads, w.head_dim)
    wk, wv = store_kv_to_cache_ref(k_new, v_new, kc.reshape(flat), vc.reshape(flat),
                                   w.slot_mapping, negative_slots="skip")
    assert np.array_equal(torch_to_bits(attn.k_cache).reshape(flat), wk)
    assert np.array_equal(torch_to_bits(attn.v_cache).reshape(flat), wv)
    want = paged_decode_attention_per_seq_ref(q, wk.reshape(shape), wv.reshape(shape),
                                              w.block_tables, w.context_lens, w.scale, w.block_size)
    assert_close_bf16(torch_to_bits(out), want, what="store+decode C1")
    stale = paged_decode_attention_per_seq_ref(q, kc, vc, w.block_tables, w.context_lens,
                                               w.scale, w.block_size)
    assert not np.array_equal(stale, want), "test is vacuous: new row does not change the output"
