"""GPU parity of the fused QK-RMSNorm + RoPE + KV-store kernel against the CPU
oracle: bit-exact (the kernel and the oracle run the same IEEE fp32 sequence)."""
import numpy as np
import pytest

from helpers import bits_to_torch, torch_to_bits

pytestmark = pytest.mark.gpu


def _run(seed, T, Hq, Hkv, with_norm=True, num_slots=2048, stride_pad=0, slots=None):
    import torch
    from nanovllm_jax_amd.layers.qk_rope_store import qk_norm_rope_store
    from oracle.paged_attention_oracle import (build_cos_sin_cache_ref, f32_to_bf16_bits,
                                               qk_norm_rope_store_ref)
    rng = np.random.Generator(np.random.PCG64(seed))
    width = (Hq + 2 * Hkv) * 128
    qkv_full = f32_to_bf16_bits(rng.standard_normal((T, width + stride_pad), dtype=np.float32) * 2)
    qkv = qkv_full[:, :width]
    cs = build_cos_sin_cache_ref(128, 4096, 1e6)
    qw = (1 + 0.2 * rng.standard_normal(128)).astype(np.float32) if with_norm else None
    kw = (1 + 0.2 * rng.standard_normal(128)).astype(np.float32) if with_norm else None
    pos = rng.integers(0, 4096, T).astype(np.int32)
    kc = rng.integers(0, 65536, (num_slots, Hkv, 128)).astype(np.uint16)
    vc = rng.integers(0, 65536, (num_slots, Hkv, 128)).astype(np.uint16)
    kc[(kc & 0x7F80) == 0x7F80] = 0; vc[(vc & 0x7F80) == 0x7F80] = 0      # no NaN patterns: compare bits
    if slots is None:
        slots = rng.permutation(num_slots)[:T].astype(np.int32)
    want_q, want_k, want_v = qk_norm_rope_store_ref(np.ascontiguousarray(qkv), pos, cs, qw, kw, 1e-6,
                                                    kc, vc, slots, Hq, Hkv)
    dev = "cuda:0"
    up = lambda a: None if a is None else torch.from_numpy(a).to(dev)
    qkv_t = bits_to_torch(qkv_full, dev)[:, :width]            # strided rows when stride_pad > 0
    kct, vct = bits_to_torch(kc, dev), bits_to_torch(vc, dev)
    q = qk_norm_rope_store(qkv_t, up(pos), up(cs), up(qw), up(kw), 1e-6, kct, vct, up(slots),
                           Hq, Hkv, 128)
    torch.cuda.synchronize()
    assert np.array_equal(torch_to_bits(q), want_q), "q not bit-exact"
    assert np.array_equal(torch_to_bits(kct), want_k), "K cache not bit-exact"
    assert np.array_equal(torch_to_bits(vct), want_v), "V cache not bit-exact"


@pytest.mark.parametrize("with_norm", [True, False])
@pytest.mark.parametrize("T,Hq,Hkv", [(1, 16, 8), (8, 16, 8), (64, 32, 8), (128, 16, 8), (257, 8, 2)])
def test_fused_bit_exact(T, Hq, Hkv, with_norm):
    print(f"case fused qk-rope-store T={T} Hq={Hq} Hkv={Hkv} norm={with_norm}", flush=True)
    _run(100 + T, T, Hq, Hkv, with_norm)


def test_fused_strided_rows_and_skip_drop():
    print("case fused strided / skip / drop", flush=True)
    slots = np.array([5, -1, 2048, 7, 0, -3, 2047, 1 << 30], np.int32)
    _run(7, 8, 16, 8, True, stride_pad=256, slots=slots)


def test_fused_feeds_paged_attention_like_the_unfused_chain():
    """Fused kernel, then decode attention == oracle chain end to end (C1 shape)."""
    print("case fused -> paged attention", flush=True)
    import torch
    from helpers import assert_close_bf16
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.qk_rope_store import qk_norm_rope_store
    from nanovllm_jax_amd.workloads import draw_bf16_bits, make_workload
    from oracle.paged_attention_oracle import (build_cos_sin_cache_ref,
                                               paged_decode_attention_per_seq_ref,
                                               qk_norm_rope_store_ref)
    w = make_workload("C1")
    rng = np.random.Generator(np.random.PCG64(31))
    shape = (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
    kc, vc = draw_bf16_bits(rng, shape), draw_bf16_bits(rng, shape)
    qkv = draw_bf16_bits(rng, (w.batch, (w.num_heads + 2 * w.num_kv_heads) * 128), gain=2.0)
    cs = build_cos_sin_cache_ref(128, 4096, 1e6)
    ones = np.ones(128, np.float32)
    pos = (w.context_lens - 1).astype(np.int32)
    flat = (-1, w.num_kv_heads, 128)
    q_ref, k_ref, v_ref = qk_norm_rope_store_ref(qkv, pos, cs, ones, ones, 1e-6, kc.reshape(flat),
                                                 vc.reshape(flat), w.slot_mapping, w.num_heads,
                                                 w.num_kv_heads)
    want = paged_decode_attention_per_seq_ref(q_ref, k_ref.reshape(shape), v_ref.reshape(shape),
                                              w.block_tables, w.context_lens, w.scale, w.block_size)
    dev = "cuda:0"
    up = lambda a: torch.from_numpy(a).to(dev)
    kct, vct = bits_to_torch(kc, dev), bits_to_torch(vc, dev)
    q = qk_norm_rope_store(bits_to_torch(qkv, dev), up(pos), up(cs), up(ones), up(ones), 1e-6, kct,
                           vct, up(w.slot_mapping), w.num_heads, w.num_kv_heads, 128)
    out = paged_attention(q, kct, vct, up(w.block_tables), up(w.context_lens), w.scale, w.block_size)
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(out), want, what="fused chain C1")
