"""The committed golden step (tests/golden/paged_decode_small.npz): the oracle
must reproduce it on the CPU, the HIP path on the GPU."""
import os

import numpy as np
import pytest

from helpers import assert_close_bf16, bits_to_torch, torch_to_bits

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "paged_decode_small.npz")


def load():
    return np.load(GOLDEN, allow_pickle=False)


def test_oracles_reproduce_golden():
    from oracle import c_oracle
    from oracle.paged_attention_oracle import (paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    g = load()
    bs = int(g["block_size"])
    flat = (-1,) + g["k_cache"].shape[2:]
    for store in (store_kv_to_cache_ref, c_oracle.store_kvcache):
        kc, vc = store(g["k_new"], g["v_new"], g["k_cache"].reshape(flat),
                       g["v_cache"].reshape(flat), g["slot_mapping"], negative_slots="skip")
        assert np.array_equal(kc.reshape(g["k_cache"].shape), g["k_cache_after"])
        assert np.array_equal(vc.reshape(g["v_cache"].shape), g["v_cache_after"])
    args = (g["q"], g["k_cache_after"], g["v_cache_after"], g["block_tables"], g["context_lens"],
            float(g["scale"]), bs)
    assert np.array_equal(paged_decode_attention_per_seq_ref(*args), g["out"])
    assert_close_bf16(c_oracle.paged_decode(*args), g["out"], atol=1e-6, rtol=2 ** -7,
                      what="C oracle vs golden")


@pytest.mark.gpu
def test_hip_reproduces_golden():
    print("case golden step", flush=True)
    import torch
    from nanovllm_jax_amd import Attention, create_decode_context
    g = load()
    dev = "cuda:0"
    B, Hq, D = g["q"].shape
    Hkv = g["k_cache"].shape[2]
    attn = Attention(Hq, D, float(g["scale"]), Hkv, int(g["block_size"]))
    attn.set_kv_cache(bits_to_torch(g["k_cache"], dev), bits_to_torch(g["v_cache"], dev))
    ctx = create_decode_context(torch.from_numpy(g["context_lens"]).to(dev),
                                torch.from_numpy(g["slot_mapping"]).to(dev),
                                torch.from_numpy(g["block_tables"]).to(dev))
    out = attn(bits_to_torch(g["q"], dev), torch.from_numpy(g["k_new"]).to(dev),
               bits_to_torch(g["v_new"], dev), ctx)
    torch.cuda.synchronize()
    assert np.array_equal(torch_to_bits(attn.k_cache), g["k_cache_after"])
    assert np.array_equal(torch_to_bits(attn.v_cache), g["v_cache_after"])
    assert_close_bf16(torch_to_bits(out), g["out"], what="golden step")
