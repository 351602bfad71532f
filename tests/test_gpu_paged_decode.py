"""GPU parity of the HIP paged decode attention against the CPU oracle,
through the C ABI (via the package's ctypes binding)."""
import numpy as np
import pytest

from helpers import ATOL, RTOL, assert_close_bf16, bits_to_torch, make_problem, torch_to_bits

pytestmark = pytest.mark.gpu


def run_hip(q, kc, vc, bt, ctx, scale, bs, chunk=0):
    import torch
    from nanovllm_jax_amd import paged_attention
    dev = "cuda:0"
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
                          scale, bs, chunk=chunk)
    torch.cuda.synchronize()
    return torch_to_bits(out)


def oracle(q, kc, vc, bt, ctx, scale, bs):
    from oracle.paged_attention_oracle import paged_decode_attention_per_seq_ref
    return paged_decode_attention_per_seq_ref(q, kc, vc, bt, ctx, scale, bs)


@pytest.mark.parametrize("chunk", [0, 32, 64, 256, 1024, -1])
@pytest.mark.parametrize("Hq,Hkv", [(16, 8), (32, 8), (64, 8), (8, 8), (8, 2), (4, 1)])
def test_small_random(Hq, Hkv, chunk):
    print(f"case small_random Hq={Hq} Hkv={Hkv} chunk={chunk}", flush=True)
    B, D, bs, NB = 5, 128, 64, 40
    ctx = [1, 31, 64, 97, 300]
    q, kc, vc, bt, ctx = make_problem(7 + Hq + chunk, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what=f"Hq={Hq} Hkv={Hkv} chunk={chunk}")


def test_c1_shape_vs_vectorized_oracle():
    """Config C1 (Qwen3-0.6B shape), against the literal whole-batch restatement."""
    print("case C1", flush=True)
    from nanovllm_jax_amd.workloads import draw_bf16_bits, make_workload
    from oracle.paged_attention_oracle import paged_decode_attention_vectorized_ref
    w = make_workload("C1")
    rng = np.random.Generator(np.random.PCG64(w.seed + 100))
    q = draw_bf16_bits(rng, (w.batch, w.num_heads, w.head_dim))
    kc = draw_bf16_bits(rng, (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim))
    vc = draw_bf16_bits(rng, (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim))
    got = run_hip(q, kc, vc, w.block_tables, w.context_lens, w.scale, w.block_size)
    want = paged_decode_attention_vectorized_ref(q, kc, vc, w.block_tables, w.context_lens,
                                                 w.scale, w.block_size)
    assert_close_bf16(got, want, what="C1")


def test_edge_context_lengths():
    """ctx = 0 -> zeros; ctx = 1 -> the V row itself, exactly; block boundary
    and one past it."""
    print("case edge_context_lengths", flush=True)
    B, Hq, Hkv, D, bs, NB = 6, 32, 8, 128, 256, 16
    ctx = [0, 1, 256, 257, 255, 512]
    q, kc, vc, bt, ctx = make_problem(11, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what="edge")
    assert not got[0].any(), "ctx=0 must give zeros"
    G = Hq // Hkv
    v_first = vc[bt[1, 0], 0]                       # [Hkv, D]
    assert np.array_equal(got[1], np.repeat(v_first, G, axis=0)), "ctx=1 must return V[0] exactly"


def test_padding_and_garbage_are_never_read():
    """Table entries past the live pages and cache rows past ctx must not
    matter: poison them (NaN bit patterns / wild page numbers)."""
    print("case padding_and_garbage", flush=True)
    B, Hq, Hkv, D, bs, NB = 4, 32, 8, 128, 256, 24
    ctx = [100, 300, 513, 1000]
    q, kc, vc, bt, ctx = make_problem(13, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    clean = run_hip(q, kc, vc, bt, ctx, scale, bs)
    kc2, vc2, bt2 = kc.copy(), vc.copy(), bt.copy()
    for b in range(B):
        n = int(ctx[b]); last = (n - 1) // bs
        page = bt[b, last]
        kc2[page, n - last * bs:] = 0x7FC0          # NaN
        vc2[page, n - last * bs:] = 0x7FC0
        bt2[b, last + 1:] = np.array([2**30, -7, -1, 123456][: bt.shape[1] - last - 1] +
                                     [-1] * max(0, bt.shape[1] - last - 1 - 4), dtype=np.int32)
    used = set(int(p) for b in range(B) for p in bt[b, : -(-int(ctx[b]) // bs)])
    for p in range(NB):
        if p not in used:
            kc2[p] = 0x7FC0; vc2[p] = 0x7FC0
    dirty = run_hip(q, kc2, vc2, bt2, ctx, scale, bs)
    assert np.array_equal(clean, dirty)


def test_split_invariance_and_page_permutation():
    print("case split_invariance", flush=True)
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    B, Hq, Hkv, D, bs, NB = 3, 32, 8, 128, 256, 20
    ctx = [1500, 777, 2048]
    q, kc, vc, bt, ctx = make_problem(17, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    outs = [bf16_bits_to_f32(run_hip(q, kc, vc, bt, ctx, scale, bs, ch)) for ch in (32, 128, 256, 2048)]
    for o in outs[1:]:
        np.testing.assert_allclose(o, outs[0], atol=ATOL, rtol=RTOL)
    # move every page somewhere else: same logical content, other physical layout
    perm = np.random.Generator(np.random.PCG64(5)).permutation(NB)
    kc2 = np.empty_like(kc); vc2 = np.empty_like(vc)
    kc2[perm] = kc; vc2[perm] = vc
    bt2 = np.where(bt >= 0, perm[np.clip(bt, 0, NB - 1)], -1).astype(np.int32)
    moved = run_hip(q, kc2, vc2, bt2, ctx, scale, bs, 256)
    assert np.array_equal(moved, run_hip(q, kc, vc, bt, ctx, scale, bs, 256))


def test_reference_smoke_shape_b64():
    """Shape of the reference's decode smoke test (test_mosaic_kernels.py:30-54):
    B=64, Hq=32, Hkv=8, D=128, 128 pages of 256, tables arange % 128,
    ctx = min(200 + 50 i, 2048)."""
    print("case reference_smoke_b64", flush=True)
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    B, Hq, Hkv, D, bs, NB, MB = 64, 32, 8, 128, 256, 128, 8
    rng = np.random.Generator(np.random.PCG64(42))
    q = draw_bf16_bits(rng, (B, Hq, D))
    kc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    vc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    bt = (np.arange(B * MB, dtype=np.int32).reshape(B, MB) % NB).astype(np.int32)
    ctx = np.minimum(200 + 50 * np.arange(B), 2048).astype(np.int32)
    scale = 1.0 / np.sqrt(D)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what="reference smoke shape")


def _fallback_case(name):
    from nanovllm_jax_amd.workloads import draw_bf16_bits, make_workload
    if name == "C1":
        w = make_workload("C1")
        rng = np.random.Generator(np.random.PCG64(w.seed + 200))
        shape = (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
        return (draw_bf16_bits(rng, (w.batch, w.num_heads, w.head_dim)),
                draw_bf16_bits(rng, shape), draw_bf16_bits(rng, shape), w.block_tables,
                w.context_lens, w.scale, w.block_size)
    if name == "parity_d64":      # layers/pallas_attention.py:622-647
        B, Hq, Hkv, D, bs, NB = 4, 8, 2, 64, 256, 32
        bt = np.arange(16, dtype=np.int32).reshape(4, 4)
        ctx = np.array([200, 512, 300, 100], np.int32)
    else:                         # test_mosaic_kernels.py:30-54
        B, Hq, Hkv, D, bs, NB = 64, 32, 8, 128, 256, 128
        bt = (np.arange(B * 8, dtype=np.int32).reshape(B, 8) % NB).astype(np.int32)
        ctx = np.minimum(200 + 50 * np.arange(B), 2048).astype(np.int32)
    rng = np.random.Generator(np.random.PCG64(4200 + B))
    return (draw_bf16_bits(rng, (B, Hq, D)), draw_bf16_bits(rng, (NB, bs, Hkv, D)),
            draw_bf16_bits(rng, (NB, bs, Hkv, D)), bt, ctx, float(1.0 / np.sqrt(D)), bs)


@pytest.mark.parametrize("chunk", [0, 256, -1])
@pytest.mark.parametrize("name", ["C1", "parity_d64", "smoke_b64"])
def test_against_the_fallback_oracle(name, chunk):
    """The reference's second dispatch target - gather + dot_product_attention
    (layers/attention.py:399-434), the one a jaxlib without Pallas takes - restated by
    paged_attention_fallback_ref: bf16 operands, fp32 softmax, probabilities rounded to
    bf16 before P.V.  Config C1, the shape of the reference's own parity check and the
    shape of its decode smoke test, in every split mode."""
    print(f"case fallback oracle {name} chunk={chunk}", flush=True)
    from oracle.paged_attention_oracle import paged_attention_fallback_ref
    q, kc, vc, bt, ctx, scale, bs = _fallback_case(name)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
    want = paged_attention_fallback_ref(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what=f"fallback oracle {name} chunk={chunk}")


@pytest.mark.parametrize("chunk", [0, 64, -1])
def test_out_of_range_metadata_is_clamped_like_the_reference(chunk):
    """A length beyond the table's reach means every described position, a negative one
    gives zeros, live table entries below 0 or beyond the pool are clipped into it
    (pallas_attention.py:185, :216-217): never a read outside the cache."""
    print(f"case out-of-range metadata chunk={chunk}", flush=True)
    from oracle.paged_attention_oracle import paged_decode_attention_vectorized_ref
    B, Hq, Hkv, D, bs, NB = 6, 16, 8, 128, 64, 40
    q, kc, vc, bt, ctx = make_problem(72, B, Hq, Hkv, D, bs, NB, [256, 256, 70, 200, 256, 100])
    ctx = ctx.copy(); bt = bt.copy()
    ctx[0] = 100000
    ctx[1] = -3
    bt[2, 0] = -1
    bt[3, 1] = NB + 5
    bt[4, 3] = 2 ** 30
    bt[5, 1] = -(2 ** 31)
    scale = float(1.0 / np.sqrt(D))
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
    want = paged_decode_attention_vectorized_ref(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what=f"out-of-range metadata chunk={chunk}")
    assert not got[1].any()


@pytest.mark.parametrize("B,seed", [(70, 1), (300, 2), (517, 3)])
def test_balanced_split_many_ragged_sequences(B, seed):
    """The balanced split (chunk=0) derives its cut from context_lens on the
    device: exercise runs that span many short sequences, empty sequences in
    between, batches beyond the 256 sequences whose prefix sums are kept in
    registers, and compare with a fixed split and the oracle."""
    print(f"case balanced ragged B={B}", flush=True)
    rng = np.random.Generator(np.random.PCG64(seed))
    Hq, Hkv, D, bs = 16, 8, 128, 32
    ctx = rng.integers(0, 200, size=B)
    ctx[rng.integers(0, B, size=B // 7)] = 0            # empty sequences
    ctx[rng.integers(0, B, size=3)] = rng.integers(900, 1500, size=3)   # a few long ones
    ctx[-1] = 0 if seed == 2 else 777                   # last sequence empty / long
    NB = int((-(-ctx // bs)).sum()) + 3
    q, kc, vc, bt, ctx = make_problem(100 + seed, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, 0)
    assert_close_bf16(got, want, what=f"balanced B={B}")
    assert not got[ctx == 0].any()
    fixed = run_hip(q, kc, vc, bt, ctx, scale, bs, 64)
    assert_close_bf16(fixed, want, what=f"fixed chunk B={B}")


@pytest.mark.parametrize("B,Hq,Hkv,D,lo,hi", [
    (2, 32, 8, 128, 0, 3000),      # 1 KV head x 8 parts per workgroup, rows over many workgroups
    (3, 32, 8, 128, 0, 3000),      # 2 x 4, rows over many workgroups
    (10, 32, 8, 128, 0, 900),      # 2 x 4, runs cross rows of different head groups
    (16, 16, 8, 128, 0, 1400),     # 4 x 2 because the table is wide
    (64, 32, 8, 128, 0, 900),      # 4 x 2
    (128, 16, 8, 128, 500, 512),   # 4 x 2, every row exactly one workgroup (no partials)
    (64, 16, 8, 128, 500, 512),    # equal step counts: the kernel takes 2 x 4 instead, as above
    (64, 16, 8, 128, 470, 512),    # 15 or 16 steps: stays 4 x 2, every row over two workgroups
    (64, 8, 8, 64, 250, 256),      # head_dim 64, equal step counts: 2 x 4 taken on the device
    (128, 8, 4, 128, 500, 512),    # 4 KV heads, equal step counts: 128 rows of 4, 256 of 2 -> 2 x 4
    (140, 8, 4, 64, 0, 300),       # head_dim 64, 4 x 2
    (90, 12, 6, 128, 0, 500),      # 6 KV heads: 2 per workgroup
    (40, 5, 5, 128, 0, 700),       # 5 KV heads: 1 per workgroup
    (300, 8, 8, 128, 0, 200)])     # 4 x 2, more sequences than workgroups
def test_balanced_split_every_workgroup_shape(B, Hq, Hkv, D, lo, hi):
    """chunk = 0 picks the KV heads per workgroup from the batch and head counts; every
    shape, with rows that are finished inside one workgroup, rows shared by parts of a
    workgroup (merged in LDS) and rows shared by workgroups (merged by the wave that
    completes them), against the oracle."""
    print(f"case balanced shapes B={B} Hq={Hq} Hkv={Hkv} D={D}", flush=True)
    rng = np.random.Generator(np.random.PCG64(B * 7 + Hkv))
    bs = 64
    ctx = rng.integers(lo, hi + 1, size=B)
    if lo == 0:
        ctx[rng.integers(0, B, size=max(1, B // 9))] = 0
        ctx[rng.integers(0, B)] = hi * 3            # one long sequence
    NB = int((-(-ctx // bs)).sum()) + 2
    q, kc, vc, bt, ctx = make_problem(900 + B, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, 0)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what=f"balanced shapes B={B} Hkv={Hkv}")
    assert not got[ctx == 0].any()


@pytest.mark.parametrize("odd_one", [None, 3, 100])
def test_balanced_split_layout_chosen_on_the_device(odd_one):
    """128 sequences x 4 KV heads of 8 steps each: the host plans 4 KV heads per
    workgroup (128 rows, each shared by two of the 256 workgroups); the kernel finds
    the step counts equal and takes 2 KV heads instead (256 rows, one whole row per
    workgroup, merged in LDS): nothing is written to the workspace.  With one
    shorter sequence it must stay with the host's plan, and partials appear.  Both
    against the oracle."""
    print(f"case device-chosen layout odd_one={odd_one}", flush=True)
    B, Hq, Hkv, D, bs = 128, 8, 4, 128, 64
    rng = np.random.Generator(np.random.PCG64(77))
    ctx = rng.integers(250, 257, size=B)        # 8 steps of 32 each
    if odd_one is not None:
        ctx[odd_one] = 100                      # 4 steps
    NB = int((-(-ctx // bs)).sum()) + 2
    q, kc, vc, bt, ctx = make_problem(4242, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    from nanovllm_jax_amd.layers.paged_attention import paged_decode_workspace_bytes
    dev = "cuda:0"
    # a workspace full of ones: whatever is still all ones afterwards was not written
    ws = torch.full((paged_decode_workspace_bytes(B, Hq, D, bt.shape[1], bs, Hkv, 0),), 0xFF,
                    dtype=torch.uint8, device=dev)
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), scale, bs,
                          chunk=0, workspace=ws)
    torch.cuda.synchronize()
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(torch_to_bits(out), want, what=f"device-chosen layout odd_one={odd_one}")
    counters = int(_lib.load().nvj_paged_decode_counter_bytes(B, Hq, Hkv))
    assert not ws[:counters].any(), "counters are zero after the call"
    partials_untouched = bool((ws[counters:] == 0xFF).all())
    assert partials_untouched == (odd_one is None), \
        "equal step counts: no partial is written; one odd sequence: some are"



@pytest.mark.parametrize("B,Hkv", [(6, 8), (64, 8), (300, 4)])
def test_balanced_split_is_one_launch_that_leaves_its_counters_zero(B, Hkv):
    """With a DecodeWorkspace (counters zero from the start) a chunk = 0 call is a single
    kernel that merges shared rows itself and puts every counter back to zero: 20 replays
    of one captured launch, the lengths changing before every replay (growing, shrinking,
    emptied, so the rows that are shared and the waves that merge them change too), each
    equal to an eager call on a fresh workspace and within the bar of the oracle."""
    print(f"case balanced one launch, 20 replays B={B} Hkv={Hkv}", flush=True)
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace
    Hq, D, bs = 2 * Hkv, 128, 64
    rng = np.random.Generator(np.random.PCG64(31 + B))
    cap = rng.integers(64, 1500, size=B)               # positions each sequence owns pages for
    q, kc, vc, bt, cap = make_problem(77 + B, B, Hq, Hkv, D, bs,
                                      int((-(-cap // bs)).sum()) + 1, cap)
    dev = "cuda:0"
    qt, kt, vt = bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev)
    btt, ct = torch.from_numpy(bt).to(dev), torch.from_numpy(cap).to(dev)
    out = torch.empty_like(qt)
    ws = DecodeWorkspace.for_shape(B, Hq, D, bt.shape[1], bs, Hkv, dev)
    counter_bytes = -(-B * Hkv * 4 // 256) * 256
    call = lambda: paged_attention(qt, kt, vt, btt, ct, 0.088, bs, chunk=0, out=out,
                                   workspace=ws, phases=_lib.NVJ_PHASE_SPLITK)
    s = torch.cuda.Stream(dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        call()
    torch.cuda.current_stream(dev).wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for step in range(20):
        new_ctx = (cap * rng.random(B)).astype(np.int32)
        new_ctx[rng.integers(0, B, size=2)] = 0
        if step % 5 == 0:
            new_ctx = cap.copy()
        ct.copy_(torch.from_numpy(new_ctx).to(dev))
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        replayed = torch_to_bits(out).copy()
        assert not ws.buffer[:counter_bytes].any(), f"replay {step} left a counter set"
        eager = paged_attention(qt, kt, vt, btt, ct, 0.088, bs, chunk=0)   # fresh workspace
        torch.cuda.synchronize()
        assert np.array_equal(replayed, torch_to_bits(eager)), f"replay {step} differs from eager"
        want = oracle(q, kc, vc, bt, new_ctx, 0.088, bs)
        assert_close_bf16(replayed, want, what=f"one-launch replay {step}")


def test_decode_workspace_reused_across_shapes():
    """One DecodeWorkspace serving calls of different shapes: the counters of a larger
    batch lie where a smaller batch left partials, which the binding knows and clears."""
    print("case DecodeWorkspace across shapes", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace
    dev, D, bs = "cuda:0", 128, 64
    ws = DecodeWorkspace(32 << 20, dev)
    for seed, B, Hq, Hkv, chunk in [(1, 3, 32, 8, 0), (2, 90, 16, 8, 0), (3, 5, 16, 8, 64),
                                    (4, 200, 8, 8, 0), (5, 2, 8, 2, 0)]:
        rng = np.random.Generator(np.random.PCG64(seed))
        ctx = rng.integers(0, 1200, size=B)
        q, kc, vc, bt, ctx = make_problem(seed, B, Hq, Hkv, D, bs,
                                          int((-(-ctx // bs)).sum()) + 1, ctx)
        out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev),
                              bits_to_torch(vc, dev), torch.from_numpy(bt).to(dev),
                              torch.from_numpy(ctx).to(dev), 0.088, bs, chunk=chunk, workspace=ws)
        torch.cuda.synchronize()
        assert_close_bf16(torch_to_bits(out), oracle(q, kc, vc, bt, ctx, 0.088, bs),
                          what=f"shared workspace, call {seed}")


def test_balanced_split_plain_entry_point_clears_dirty_counters():
    """nvj_paged_decode_launch promises that the workspace need not be initialised: it
    clears the counters itself.  Fill the workspace with ones and call it."""
    print("case balanced, dirty workspace", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.paged_attention import paged_decode_workspace_bytes
    B, Hq, Hkv, D, bs, NB = 10, 32, 8, 128, 64, 200
    ctx = [1000, 5, 0, 640, 77, 1200, 64, 333, 2, 900]
    q, kc, vc, bt, ctx = make_problem(91, B, Hq, Hkv, D, bs, NB, ctx)
    dev = "cuda:0"
    ws = torch.full((paged_decode_workspace_bytes(B, Hq, D, bt.shape[1], bs, Hkv, 0),), 0xFF,
                    dtype=torch.uint8, device=dev)
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), 0.088, bs,
                          chunk=0, workspace=ws)
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(out), oracle(q, kc, vc, bt, ctx, 0.088, bs),
                      what="dirty workspace")


def test_balanced_split_all_empty_and_single_position():
    print("case balanced all-empty / single position", flush=True)
    B, Hq, Hkv, D, bs, NB = 9, 32, 8, 128, 256, 12
    q, kc, vc, bt, ctx = make_problem(5, B, Hq, Hkv, D, bs, NB, [0] * B)
    got = run_hip(q, kc, vc, bt, ctx, 0.1, bs, 0)
    assert not got.any()
    ctx2 = np.zeros(B, np.int32); ctx2[4] = 1
    q, kc, vc, bt, ctx2 = make_problem(6, B, Hq, Hkv, D, bs, NB, ctx2)
    got = run_hip(q, kc, vc, bt, ctx2, 0.1, bs, 0)
    assert np.array_equal(got[4], np.repeat(vc[bt[4, 0], 0], Hq // Hkv, axis=0))
    assert not np.delete(got, 4, axis=0).any()


def test_reference_parity_check_shape_d64():
    """Shape of the reference's only numeric parity check
    (layers/pallas_attention.py:622-647): B=4, Hq=8, Hkv=2, D=64, 32 pages of 256,
    4 pages per sequence in order, ctx = [200, 512, 300, 100], bf16."""
    print("case reference parity shape D=64", flush=True)
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    B, Hq, Hkv, D, bs, NB = 4, 8, 2, 64, 256, 32
    rng = np.random.Generator(np.random.PCG64(42))
    q = draw_bf16_bits(rng, (B, Hq, D))
    kc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    vc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    bt = np.arange(16, dtype=np.int32).reshape(4, 4)
    ctx = np.array([200, 512, 300, 100], np.int32)
    scale = 1.0 / np.sqrt(D)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    for chunk in (0, 64, 256):
        got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
        assert_close_bf16(got, want, what=f"D=64 chunk={chunk}")


def test_reference_per_sequence_blocks_shape_d64_page64():
    """Shape of the reference's TEST 4 (test_mosaic_kernels.py:234-260): B=4, Hq=8,
    Hkv=2, D=64, 16 pages of 64, tables [[0..3],[4..7],[8..11],[12..15]],
    ctx = [100, 150, 200, 250]."""
    print("case reference per-sequence blocks shape D=64 page 64", flush=True)
    from nanovllm_jax_amd.workloads import draw_bf16_bits
    B, Hq, Hkv, D, bs, NB = 4, 8, 2, 64, 64, 16
    rng = np.random.Generator(np.random.PCG64(43))
    q = draw_bf16_bits(rng, (B, Hq, D))
    kc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    vc = draw_bf16_bits(rng, (NB, bs, Hkv, D))
    bt = np.arange(16, dtype=np.int32).reshape(4, 4)
    ctx = np.array([100, 150, 200, 250], np.int32)
    scale = 1.0 / np.sqrt(D)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, 0)
    assert_close_bf16(got, want, what="D=64 page 64")


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (16, 4), (8, 1)])
def test_d64_random_groups_and_tails(Hq, Hkv):
    print(f"case D=64 random Hq={Hq} Hkv={Hkv}", flush=True)
    B, D, bs, NB = 5, 64, 32, 60
    q, kc, vc, bt, ctx = make_problem(200 + Hq, B, Hq, Hkv, D, bs, NB, [1, 31, 33, 0, 700])
    scale = 1.0 / np.sqrt(D)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    for chunk in (0, 96):
        got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
        assert_close_bf16(got, want, what=f"D=64 Hq={Hq} Hkv={Hkv} chunk={chunk}")
    assert np.array_equal(got[0], np.repeat(vc[bt[0, 0], 0], Hq // Hkv, axis=0))


# ---- whole-sequence mode (chunk = -1): every sequence finished inside one workgroup ----
@pytest.mark.parametrize("B,Hq,Hkv,D", [(3, 32, 8, 128),     # 1 head per workgroup, 8 parts
                                        (64, 16, 8, 128),    # 2 heads x 4 parts
                                        (128, 16, 8, 128),   # 4 heads x 2 parts
                                        (260, 8, 8, 128),    # 8 heads, no split inside
                                        (90, 12, 6, 128),    # 6 KV heads: 2 per workgroup
                                        (70, 8, 4, 64),      # head_dim 64, 1 head x 8 parts
                                        (140, 8, 4, 64),     # head_dim 64, 2 heads x 4 parts
                                        (5, 4, 1, 128)])
def test_whole_sequence_mode(B, Hq, Hkv, D):
    """Lengths around the number of parts (fewer steps than parts, empty parts),
    empty sequences, tails, several pages; compared with the oracle and with the
    balanced split."""
    print(f"case whole-sequence B={B} Hq={Hq} Hkv={Hkv} D={D}", flush=True)
    rng = np.random.Generator(np.random.PCG64(900 + B + Hkv))
    bs = 64
    ctx = rng.integers(1, 400, size=B)
    ctx[:min(B, 12)] = [0, 1, 31, 32, 33, 64, 65, 255, 256, 257, 300, 96][:min(B, 12)]
    NB = int((-(-ctx // bs)).sum()) + 2
    q, kc, vc, bt, ctx = make_problem(900 + B, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, -1)
    assert_close_bf16(got, want, what=f"whole-sequence B={B}")
    assert not got[ctx == 0].any(), "ctx=0 must give zeros"
    one = np.flatnonzero(ctx == 1)[0]
    assert np.array_equal(got[one], np.repeat(vc[bt[one, 0], 0], Hq // Hkv, axis=0))
    balanced = run_hip(q, kc, vc, bt, ctx, scale, bs, 0)
    assert_close_bf16(got, balanced, what="whole-sequence vs balanced")


def test_whole_sequence_mode_needs_no_workspace_and_ignores_garbage():
    """workspace_bytes is 0, a NULL workspace is accepted, and nothing beyond
    ctx or in padding table entries is read."""
    print("case whole-sequence no workspace / garbage", flush=True)
    import torch
    from nanovllm_jax_amd import _lib
    from nanovllm_jax_amd.layers.paged_attention import WHOLE_SEQUENCE, paged_decode_workspace_bytes
    B, Hq, Hkv, D, bs, NB = 40, 32, 8, 128, 256, 200
    assert paged_decode_workspace_bytes(B, Hq, D, 4, bs, Hkv, WHOLE_SEQUENCE) == 0
    rng = np.random.Generator(np.random.PCG64(77))
    ctx = rng.integers(200, 1000, size=B)
    q, kc, vc, bt, ctx = make_problem(78, B, Hq, Hkv, D, bs, NB, ctx)
    want = oracle(q, kc, vc, bt, ctx, 0.09, bs)
    # poison: NaN patterns in every slot past ctx of the last live page, wild padding entries
    kc2, vc2, bt2 = kc.copy(), vc.copy(), bt.copy()
    for b in range(B):
        pages = -(-int(ctx[b]) // bs)
        tail = int(ctx[b]) - (pages - 1) * bs
        kc2[bt[b, pages - 1], tail:] = 0x7FC0
        vc2[bt[b, pages - 1], tail:] = 0x7FC0
        bt2[b, pages:] = 2 ** 30
    dev = "cuda:0"
    lib = _lib.load()
    qt, kt, vt = bits_to_torch(q, dev), bits_to_torch(kc2, dev), bits_to_torch(vc2, dev)
    btt, ct = torch.from_numpy(bt2).to(dev), torch.from_numpy(ctx).to(dev)
    out = torch.empty_like(qt)
    code = lib.nvj_paged_decode_launch(
        torch.cuda.current_stream().cuda_stream, qt.data_ptr(), kt.data_ptr(), vt.data_ptr(),
        btt.data_ptr(), ct.data_ptr(), out.data_ptr(), None, 0, B, Hq, Hkv, D, bs, bt.shape[1],
        NB, 0.09, WHOLE_SEQUENCE, _lib.NVJ_DTYPE_BF16)
    assert code == 0
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(out), want, what="whole-sequence, NULL workspace, poison")


@pytest.mark.parametrize("chunk", [0, -1])
def test_decode_call_replays_in_a_hip_graph(chunk):
    """The decode launch(es) captured once and replayed with the lengths and the
    query updated in place between replays give what eager calls give, every
    time (balanced split behind its counter-clearing launch, and the whole-sequence
    split)."""
    print(f"case decode graph replays chunk={chunk}", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.paged_attention import paged_decode_workspace_bytes
    B, Hq, Hkv, D, bs, NB = 48, 32, 8, 128, 64, 400
    rng = np.random.Generator(np.random.PCG64(4242))
    ctx0 = rng.integers(100, 500, size=B)
    q, kc, vc, bt, ctx0 = make_problem(4243, B, Hq, Hkv, D, bs, NB, ctx0)
    dev = "cuda:0"
    qt, kt, vt = bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev)
    btt, ct = torch.from_numpy(bt).to(dev), torch.from_numpy(ctx0).to(dev)
    out = torch.empty_like(qt)
    ws = torch.empty(max(16, paged_decode_workspace_bytes(B, Hq, D, bt.shape[1], bs, Hkv, chunk)),
                     dtype=torch.uint8, device=dev)
    call = lambda: paged_attention(qt, kt, vt, btt, ct, 0.088, bs, chunk=chunk, out=out,
                                   workspace=ws)
    s = torch.cuda.Stream(dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        call()
    torch.cuda.current_stream(dev).wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for step in range(4):
        # shorter lengths every replay (always inside the pages each sequence owns)
        new_ctx = np.maximum(1, ctx0 - 37 * step).astype(np.int32)
        ct.copy_(torch.from_numpy(new_ctx).to(dev))
        qt.copy_(bits_to_torch(np.roll(q, step, axis=0), dev))
        graph.replay()
        torch.cuda.synchronize()
        replayed = torch_to_bits(out).copy()
        out.zero_()
        call()                                   # eager, same inputs
        torch.cuda.synchronize()
        assert np.array_equal(replayed, torch_to_bits(out)), f"replay {step} differs from eager"
        want = oracle(np.roll(q, step, axis=0), kc, vc, bt, new_ctx, 0.088, bs)
        assert_close_bf16(replayed, want, what=f"graph replay {step}")


@pytest.mark.parametrize("chunk", [0, 64, -1])
def test_scale_zero_gives_the_mean_of_v_over_the_live_positions(chunk):
    """softmax of all-zero scores is uniform over the positions below ctx, and
    positions past the end of a partly filled 32-position step must weigh
    exactly 0 there too (the exponential of a masked score times scale 0 is 1)."""
    print(f"case scale 0 chunk={chunk}", flush=True)
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    B, Hq, Hkv, D, bs, NB = 6, 16, 8, 128, 64, 30
    ctx = [1, 5, 33, 70, 100, 191]
    q, kc, vc, bt, ctx = make_problem(55, B, Hq, Hkv, D, bs, NB, ctx)
    got = bf16_bits_to_f32(run_hip(q, kc, vc, bt, ctx, 0.0, bs, chunk))
    v = bf16_bits_to_f32(vc).astype(np.float64)
    for b in range(B):
        rows = np.concatenate([v[bt[b, p]] for p in range(-(-int(ctx[b]) // bs))])[:ctx[b]]
        mean = np.repeat(rows.mean(axis=0), Hq // Hkv, axis=0)          # [Hq, D]
        assert np.all(np.abs(got[b] - mean) <= 1e-2 + 1e-2 * np.abs(mean)), f"sequence {b}"


@pytest.mark.parametrize("Hq,Hkv,D", [(32, 1, 128), (48, 2, 128), (17, 1, 128), (64, 2, 64),
                                      (40, 1, 64)])
@pytest.mark.parametrize("chunk", [0, 64, -1])
def test_more_than_16_query_heads_per_kv_head(Hq, Hkv, D, chunk):
    """Groups above the 16 MFMA columns of a wave are served in parts (32 = 2 x 16,
    24 = 2 x 12, 17 = 17 x 1, 40 = 4 x 10), every part reading its KV head's rows."""
    print(f"case large group Hq={Hq} Hkv={Hkv} D={D} chunk={chunk}", flush=True)
    B, bs, NB = 9, 64, 60
    ctx = [0, 1, 33, 64, 100, 257, 300, 31, 129]
    q, kc, vc, bt, ctx = make_problem(600 + Hq + Hkv, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    got = run_hip(q, kc, vc, bt, ctx, scale, bs, chunk)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    assert_close_bf16(got, want, what=f"large group Hq={Hq} Hkv={Hkv} chunk={chunk}")


# ---- the vector-ALU measurement variant (phases | NVJ_PHASE_VALU_PRODUCTS) ----
def run_hip_valu(q, kc, vc, bt, ctx, scale, bs, chunk):
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    dev = "cuda:0"
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
                          scale, bs, chunk=chunk,
                          phases=_lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE |
                          _lib.NVJ_PHASE_VALU_PRODUCTS)
    torch.cuda.synchronize()
    return torch_to_bits(out)


@pytest.mark.parametrize("chunk", [0, -1])
@pytest.mark.parametrize("B,Hq,Hkv", [(7, 32, 8), (7, 64, 8), (70, 64, 16), (300, 32, 8)])
def test_vector_alu_variant_matches_the_oracle(B, Hq, Hkv, chunk):
    print(f"case vector-ALU variant B={B} Hq={Hq} Hkv={Hkv} chunk={chunk}", flush=True)
    rng = np.random.Generator(np.random.PCG64(950 + B + Hq))
    bs = 64
    ctx = rng.integers(1, 700, size=B)
    ctx[:7] = [0, 1, 31, 33, 64, 257, 1000]
    NB = int((-(-ctx // bs)).sum()) + 2
    q, kc, vc, bt, ctx = make_problem(950 + B, B, Hq, Hkv, 128, bs, NB, ctx, q_gain=2.0)
    scale = 1.0 / np.sqrt(128)
    want = oracle(q, kc, vc, bt, ctx, scale, bs)
    got = run_hip_valu(q, kc, vc, bt, ctx, scale, bs, chunk)
    assert_close_bf16(got, want, what=f"vector-ALU variant chunk={chunk}")
    assert not got[0].any(), "ctx=0 must give zeros"
    assert np.array_equal(got[1], np.repeat(vc[bt[1, 0], 0], Hq // Hkv, axis=0))
    assert_close_bf16(got, run_hip(q, kc, vc, bt, ctx, scale, bs, chunk), what="vs MFMA")


def test_vector_alu_variant_refuses_other_shapes():
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    dev = "cuda:0"
    flags = _lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE | _lib.NVJ_PHASE_VALU_PRODUCTS
    bt = torch.zeros((1, 1), dtype=torch.int32, device=dev)
    ctx = torch.ones(1, dtype=torch.int32, device=dev)
    for Hq, Hkv, D, dt, chunk in [(16, 8, 128, torch.bfloat16, 0),     # group 2
                                  (32, 8, 64, torch.bfloat16, 0),      # head_dim 64
                                  (32, 8, 128, torch.float16, 0),      # float16
                                  (16, 4, 128, torch.bfloat16, 0),     # 4 KV heads
                                  (32, 8, 128, torch.bfloat16, 64)]:   # fixed chunks
        q = torch.zeros((1, Hq, D), dtype=dt, device=dev)
        kc = torch.zeros((2, 64, Hkv, D), dtype=dt, device=dev)
        with pytest.raises(_lib.NativeLibraryError, match="unsupported"):
            paged_attention(q, kc, kc, bt, ctx, 0.1, 64, chunk=chunk, phases=flags)


def test_loads_only_variant_runs_and_leaves_finite_values():
    """NVJ_PHASE_LOADS_ONLY (the K/V stream with no arithmetic behind it, a timing aid) runs
    in both modes it exists for and leaves finite values in `out`."""
    print("case loads-only variant", flush=True)
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    B, Hq, Hkv, D, bs, NB = 7, 32, 8, 128, 64, 120
    q, kc, vc, bt, ctx = make_problem(808, B, Hq, Hkv, D, bs, NB, [900, 33, 0, 640, 1, 1000, 257])
    dev = "cuda:0"
    for chunk in (0, -1):
        out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                              torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), 0.09, bs,
                              chunk=chunk,
                              phases=_lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_LOADS_ONLY)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("B,Hq,Hkv,bs,MB", [(64, 2, 1, 64, 8192),     # 1 KV head x 8 parts
                                            (300, 8, 8, 32, 8192)])   # 8 KV heads x 1 part
def test_balanced_split_with_a_very_wide_block_table(B, Hq, Hkv, bs, MB):
    """The cut of the balanced split is computed in 32-bit arithmetic; when the block
    table could describe so many positions that (steps x sub-runs) would not fit, the
    kernel cuts in coarser units.  Only the table's width decides that, so short
    sequences behind a table 8192 pages wide exercise it."""
    print(f"case very wide block table B={B} Hkv={Hkv} MB={MB}", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    rng = np.random.Generator(np.random.PCG64(B + MB))
    D = 128
    ctx = rng.integers(0, 900, size=B)
    ctx[0] = 3000
    q, kc, vc, bt, ctx = make_problem(5150 + B, B, Hq, Hkv, D, bs,
                                      int((-(-ctx // bs)).sum()) + 1, ctx)
    wide = np.full((B, MB), -1, np.int32)
    wide[:, :bt.shape[1]] = bt
    dev = "cuda:0"
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(wide).to(dev), torch.from_numpy(ctx).to(dev), 0.088, bs,
                          chunk=0)
    torch.cuda.synchronize()
    assert_close_bf16(torch_to_bits(out), oracle(q, kc, vc, bt, ctx, 0.088, bs),
                      what=f"wide table B={B}")
