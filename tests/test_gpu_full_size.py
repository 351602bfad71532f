"""Parity at the full sizes of the specified workloads (C2 headline, C3 ragged,
C4 long context, C5 layer shape): HIP output against the C oracle run on the
host cores over the very same device-drawn inputs, plus size-independent
properties (split invariance, store-then-read)."""
import os
import sys

import numpy as np
import pytest

from helpers import assert_close_bf16, bits_to_torch, torch_to_bits

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu


def _run(name, chunks, dtype="bf16"):
    import torch
    import bench
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.workloads import make_workload
    from oracle import c_oracle
    dev = torch.device("cuda:0")
    w = make_workload(name)
    dt = torch.float16 if dtype == "f16" else torch.bfloat16
    q, kc, vc, bt, ctx, slots, k_new, v_new = bench.device_inputs(w, torch, dev, dt)
    outs = []
    for ch in chunks:
        print(f"case {name} full size chunk={ch}", flush=True)
        out = paged_attention(q, kc, vc, bt, ctx, w.scale, w.block_size, chunk=ch)
        torch.cuda.synchronize()
        outs.append(torch_to_bits(out))
    want = c_oracle.paged_decode(torch_to_bits(q), torch_to_bits(kc), torch_to_bits(vc),
                                 w.block_tables, w.context_lens, w.scale, w.block_size,
                                 dtype=dtype)
    for ch, got in zip(chunks, outs):
        if dtype == "f16":
            from oracle.paged_attention_oracle import f16_bits_to_f32
            g, t = (f16_bits_to_f32(a).astype(np.float64) for a in (got, want))
            assert np.all(np.abs(g - t) <= 1e-2 + 1e-2 * np.abs(t)), f"{name} f16 chunk={ch}"
            err = float(np.abs(g - t).max())
        else:
            err = assert_close_bf16(got, want, what=f"{name} chunk={ch}")
        print(f"  {name} chunk={ch}: max abs err {err:.3e}", flush=True)
    del q, kc, vc
    torch.cuda.empty_cache()
    return w, outs, want


def test_c2_qwen3_8b_shape():
    _run("C2", [0, 256])


def test_c2_float16_caches():
    _run("C2", [0, -1], dtype="f16")


def test_c5_layer_shape():
    _run("C5", [0])


def test_c4_long_context_sharp_softmax():
    w, outs, want = _run("C4", [0, 4096])
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    # q * 4 sharpens the softmax: outputs are not the ~1/sqrt(ctx) averages of C2
    assert np.abs(bf16_bits_to_f32(want)).max() > 0.3


def test_c3_ragged_batch():
    w, outs, want = _run("C3", [0, 512])
    # sequences whose last page is partial must be present in this workload
    assert (w.context_lens % w.block_size != 0).sum() > w.batch // 2


def test_pool_larger_than_4_gib_per_tensor():
    """Pages near the top of a 5 GiB-per-tensor pool: every byte offset into the
    caches needs more than 32 bits (decode reads, plain store, fused store)."""
    print("case large pool addressing", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention, store_kv_to_cache
    from oracle.paged_attention_oracle import (f32_to_bf16_bits, paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    dev = "cuda:0"
    NB, bs, Hkv, D, Hq, B = 10240, 256, 8, 128, 32, 4          # 10240 pages x 512 KiB = 5 GiB
    kc = torch.zeros((NB, bs, Hkv, D), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros((NB, bs, Hkv, D), dtype=torch.bfloat16, device=dev)
    rng = np.random.Generator(np.random.PCG64(99))
    ctx = np.array([700, 256, 1, 513], np.int32)
    pages = [NB - 1 - i for i in range(8)]                      # all above the 4 GiB mark
    bt = np.full((B, 3), -1, np.int32)
    small_k = np.zeros((8, bs, Hkv, D), np.uint16)              # host copy of just those pages
    small_v = np.zeros((8, bs, Hkv, D), np.uint16)
    remap, nxt = {}, 0
    for b in range(B):
        for p in range(-(-int(ctx[b]) // bs)):
            page = pages[nxt]
            bt[b, p] = page
            remap[page] = nxt
            small_k[nxt] = draw_bf16_bits(rng, (bs, Hkv, D))
            small_v[nxt] = draw_bf16_bits(rng, (bs, Hkv, D))
            kc[page] = bits_to_torch(small_k[nxt], dev)
            vc[page] = bits_to_torch(small_v[nxt], dev)
            nxt += 1
    q = draw_bf16_bits(rng, (B, Hq, D))
    # store one new row per sequence at its last position, then read
    k_new = rng.standard_normal((B, Hkv, D), dtype=np.float32)
    v_new = draw_bf16_bits(rng, (B, Hkv, D))
    slots = np.array([bt[b, (ctx[b] - 1) // bs] * bs + (ctx[b] - 1) % bs for b in range(B)], np.int64)
    assert slots.min() * Hkv * D * 2 > 2 ** 32
    store_kv_to_cache(torch.from_numpy(k_new).to(dev), bits_to_torch(v_new, dev),
                      kc.view(-1, Hkv, D), vc.view(-1, Hkv, D),
                      torch.from_numpy(slots.astype(np.int32)).to(dev))
    small_bt = np.vectorize(lambda x: remap.get(int(x), -1))(bt).astype(np.int32)
    small_slots = np.array([small_bt[b, (ctx[b] - 1) // bs] * bs + (ctx[b] - 1) % bs
                            for b in range(B)], np.int32)
    wk, wv = store_kv_to_cache_ref(k_new, v_new, small_k.reshape(-1, Hkv, D),
                                   small_v.reshape(-1, Hkv, D), small_slots, negative_slots="skip")
    for page, i in remap.items():
        assert np.array_equal(torch_to_bits(kc[page]), wk.reshape(8, bs, Hkv, D)[i])
        assert np.array_equal(torch_to_bits(vc[page]), wv.reshape(8, bs, Hkv, D)[i])
    want = paged_decode_attention_per_seq_ref(q, wk.reshape(8, bs, Hkv, D), wv.reshape(8, bs, Hkv, D),
                                              small_bt, ctx, D ** -0.5, bs)
    for chunk in (0, 256, -1):
        out = paged_attention(bits_to_torch(q, dev), kc, vc, torch.from_numpy(bt).to(dev),
                              torch.from_numpy(ctx).to(dev), D ** -0.5, bs, chunk=chunk)
        torch.cuda.synchronize()
        assert_close_bf16(torch_to_bits(out), want, what=f"large pool chunk={chunk}")
    del kc, vc
    torch.cuda.empty_cache()
