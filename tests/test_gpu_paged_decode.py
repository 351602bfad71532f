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


def _steps(ctx, cap):
    return -(-np.clip(np.asarray(ctx, np.int64), 0, cap) // 32)


def deals_whole_rows(ctx, num_kv_heads, table_positions, cus=256, tolerance=64, tight=8):
    """The balanced kernel's own layout rule, restated: are whole (sequence, head
    group) rows dealt to the workgroups (nothing shared, workspace untouched)?
    Returns (whole_rows, sorted): `sorted` when it took the order by decreasing
    length to get there."""
    B = len(ctx)
    max_steps = -(-table_positions // 32)
    hpw = 2
    if B * num_kv_heads <= 16 and max_steps >= 192:
        hpw = 1
    elif B >= 32 or (B >= 16 and max_steps >= 128):
        hpw = 4
    while hpw > 1 and num_kv_heads % hpw:
        hpw //= 2
    axis = (num_kv_heads // hpw) * B * max_steps
    wgs = min(cus, max(1, -(-axis // (8 // hpw))))

    def usable(h):      # rows per sequence a power of two, a row for every workgroup
        rps = num_kv_heads // h if h > 0 and num_kv_heads % h == 0 else 0
        return rps > 0 and rps & (rps - 1) == 0 and B * rps >= wgs

    candidates = []
    h = hpw
    while B <= 256 and wgs <= 256 and h >= 2:
        if num_kv_heads % h == 0 and B * (num_kv_heads // h) >= wgs:
            if usable(h):
                candidates = [h] + ([h // 2] if usable(h // 2) else [])
            break
        h //= 2
    steps = _steps(ctx, table_positions)
    if steps.sum() == 0:
        return False, False
    by_length = np.argsort(-steps, kind="stable")
    for h in candidates:
        rps = num_kv_heads // h
        rows = B * rps
        rounds = -(-rows // wgs)
        share = rps * int(steps.sum())

        def largest(order):
            load = np.zeros(wgs, np.int64)
            for p in range(rows):
                t, w = divmod(p, wgs)
                load[wgs - 1 - w if t % 2 else w] += steps[order[p // rps]]
            return int(load.max())

        if int(steps.max()) * wgs * 256 > share * (256 + tolerance):   # one row alone is too much
            continue
        if rounds == 1:
            return True, False
        # the order of the batch: only when the lengths are close and the deal all but even
        if (steps.max() - steps.min()) * 8 <= steps.max() and \
                largest(np.arange(B)) * wgs * 256 <= share * (256 + min(tolerance, tight)):
            return True, False
        if largest(by_length) * wgs * 256 <= share * (256 + tolerance):
            return True, True
    return False, False


def _run_over_marked_workspace(q, kc, vc, bt, ctx, scale, bs, extra_phases=0):
    """A chunk = 0 call over a workspace full of ones: returns the output and whether
    the partials are still all ones afterwards (then no row was shared)."""
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    from nanovllm_jax_amd.layers.paged_attention import paged_decode_workspace_bytes
    dev = "cuda:0"
    B, Hq, D = q.shape
    Hkv = kc.shape[2]
    ws = torch.full((paged_decode_workspace_bytes(B, Hq, D, bt.shape[1], bs, Hkv, 0),), 0xFF,
                    dtype=torch.uint8, device=dev)
    out = paged_attention(bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
                          torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), scale, bs,
                          chunk=0, workspace=ws,
                          phases=_lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE | extra_phases)
    torch.cuda.synchronize()
    counters = int(_lib.load().nvj_paged_decode_counter_bytes(B, Hq, Hkv))
    assert not ws[:counters].any(), "the counter region is zero after the call"
    return torch_to_bits(out), bool((ws[counters:] == 0xFF).all())


@pytest.mark.parametrize("name", ["equal", "within_tolerance", "one_short", "one_long",
                                  "a_sixth_apart", "a_half_apart",
                                  "pairs_by_length", "pairs_four_rounds", "log_uniform",
                                  "equal_forced_shared"])
def test_balanced_split_deals_whole_rows_when_that_is_balanced(name):
    """The kernel looks at the lengths and, when whole rows can be dealt to the
    workgroups within a quarter of an equal share, shares no row (the workspace stays
    untouched): equal lengths; lengths a few percent or a sixth apart; one short
    sequence among equal ones; lengths that only balance when long rows are paired with short ones
    (the order by decreasing length, two and four rounds of rows).  Lengths a half apart only balance with half as many KV heads per
    workgroup (twice the rows, paired by length): the kernel's second choice.  It must
    not deal whole rows when one long sequence or a log-uniform spread would leave
    workgroups idle for long, and
    not when the caller forbids it.  Every case against the oracle, and the layout
    against the rule restated in deals_whole_rows."""
    print(f"case whole rows {name}", flush=True)
    from nanovllm_jax_amd import _lib
    rng = np.random.Generator(np.random.PCG64(len(name) * 131 + 5))
    bs, extra = 64, 0
    if name in ("equal", "equal_forced_shared", "within_tolerance", "one_short", "one_long",
                "a_sixth_apart", "a_half_apart"):
        B, Hq, Hkv, D = 128, 8, 4, 128                 # 128 rows of 4 heads, 256 rows of 2
        ctx = {"equal": lambda: rng.integers(930, 961, size=B),            # 30 steps each
               "equal_forced_shared": lambda: rng.integers(930, 961, size=B),
               "within_tolerance": lambda: rng.integers(870, 961, size=B),  # 28..30 steps
               "a_sixth_apart": lambda: rng.integers(700, 961, size=B),     # 22..30 steps
               "a_half_apart": lambda: rng.integers(300, 961, size=B),      # 10..30 steps
               "one_short": lambda: np.where(np.arange(B) == 77, 100, 960),
               "one_long": lambda: np.where(np.arange(B) == 77, 2900, 960)}[name]()
        if name == "equal_forced_shared":
            extra = _lib.NVJ_PHASE_SHARED_ROWS
    elif name == "pairs_by_length":
        B, Hq, Hkv, D = 256, 8, 8, 64                  # 512 rows of 4 heads: two rounds
        ctx = rng.integers(64, 1400, size=B)
    elif name == "pairs_four_rounds":
        B, Hq, Hkv, D = 256, 16, 16, 64                # 1024 rows of 4 heads: four rounds
        ctx = rng.integers(64, 1000, size=B)
    else:
        B, Hq, Hkv, D = 256, 8, 8, 64
        ctx = np.rint(np.exp(rng.uniform(np.log(16.0), np.log(4096.0), size=B))).astype(np.int64)
    NB = int((-(-ctx // bs)).sum()) + 2
    q, kc, vc, bt, ctx = make_problem(4242 + B, B, Hq, Hkv, D, bs, NB, ctx)
    scale = 1.0 / np.sqrt(D)
    got, untouched = _run_over_marked_workspace(q, kc, vc, bt, ctx, scale, bs, extra)
    assert_close_bf16(got, oracle(q, kc, vc, bt, ctx, scale, bs), what=f"whole rows {name}")
    whole, by_length = deals_whole_rows(ctx, Hkv, bt.shape[1] * bs)
    expect = {"equal": (True, False), "within_tolerance": (True, False),
              "one_short": (True, False), "one_long": (False, False),
              "a_sixth_apart": (True, False), "a_half_apart": (True, True),
              "pairs_by_length": (True, True), "pairs_four_rounds": (True, True),
              "log_uniform": (False, False), "equal_forced_shared": (True, False)}[name]
    assert (whole, by_length) == expect, "the case does not exercise what its name says"
    assert untouched == (whole and not extra), \
        f"{name}: partials {'untouched' if untouched else 'written'}"


def test_balanced_split_whole_rows_equal_the_shared_rows_split():
    """The two layouts of chunk = 0 on one batch each: same result to fp32 round-off of
    the merge order (far inside the bar), for bf16 and float16, head_dim 128 and 64,
    groups of 16 and of 32 query heads (a cache head walked as two), and a batch with empty
    sequences in it."""
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    dev = "cuda:0"
    for seed, B, Hq, Hkv, D, lo, hi, dt in [(1, 64, 32, 8, 128, 1000, 1024, torch.bfloat16),
                                            (2, 128, 16, 8, 64, 400, 420, torch.float16),
                                            (3, 256, 32, 2, 128, 200, 224, torch.bfloat16),
                                            (4, 128, 16, 16, 64, 0, 1200, torch.bfloat16),
                                            (5, 128, 128, 4, 128, 300, 320, torch.float16)]:
        print(f"case both layouts seed={seed} B={B} Hq={Hq} Hkv={Hkv} D={D} {dt}", flush=True)
        rng = np.random.Generator(np.random.PCG64(seed))
        bs = 32
        ctx = rng.integers(lo, hi + 1, size=B)
        if lo == 0:
            # short and empty sequences, each with a partner that makes up the difference
            half = rng.integers(0, hi // 32 + 1, size=B // 2) * 32
            half[rng.integers(0, B // 2, size=20)] = 0
            ctx = rng.permutation(np.concatenate([half, 2 * hi - half]))
        q, kc, vc, bt, ctx = make_problem(50 + seed, B, Hq, Hkv, D, bs,
                                          int((-(-ctx // bs)).sum()) + 1, ctx)
        assert deals_whole_rows(ctx, Hkv * max(1, Hq // Hkv // 16), bt.shape[1] * bs)[0]
        args = (bits_to_torch(q, dev).view(torch.int16).view(dt),
                bits_to_torch(kc, dev).view(torch.int16).view(dt),
                bits_to_torch(vc, dev).view(torch.int16).view(dt),
                torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), 0.09, bs)
        base = _lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE
        a = paged_attention(*args, chunk=0, phases=base)
        b = paged_attention(*args, chunk=0, phases=base | _lib.NVJ_PHASE_SHARED_ROWS)
        torch.cuda.synchronize()
        fa, fb = a.float().cpu().numpy(), b.float().cpu().numpy()
        assert np.isfinite(fa).all()
        assert np.abs(fa - fb).max() <= 2e-3 + 8e-3 * np.abs(fb).max(), np.abs(fa - fb).max()
        assert not fa[ctx == 0].any()
        if dt == torch.bfloat16:
            assert_close_bf16(torch_to_bits(a), oracle(q, kc, vc, bt, ctx, 0.09, bs),
                              what=f"whole rows seed={seed}")


@pytest.mark.parametrize("B,ctx_len", [(1, 8200), (2, 6100)])
@pytest.mark.parametrize("f16", [False, True])
def test_balanced_split_head_dim_64_merge_in_several_passes(B, ctx_len, f16):
    """head_dim 64: the merging wave's tile holds the (max, sum) pairs of 32 slots, so a
    row shared by more sub-runs than that is merged in several passes (one or two long
    sequences over all workgroups)."""
    print(f"case D=64 several merge passes B={B} f16={f16}", flush=True)
    import torch
    from nanovllm_jax_amd import paged_attention
    Hq, Hkv, D, bs = 8, 8, 64, 64
    ctx = [ctx_len] + [ctx_len - 900] * (B - 1)
    q, kc, vc, bt, ctx = make_problem(640 + B, B, Hq, Hkv, D, bs, sum(-(-c // bs) for c in ctx) + 1,
                                      ctx)
    scale = 1.0 / np.sqrt(D)
    if not f16:
        got = run_hip(q, kc, vc, bt, ctx, scale, bs, 0)
        assert_close_bf16(got, oracle(q, kc, vc, bt, ctx, scale, bs), what=f"D=64 passes B={B}")
        return
    from oracle.paged_attention_oracle import paged_decode_attention_per_seq_ref
    dev = "cuda:0"
    to_f16 = lambda bits: bits_to_torch(bits, dev).float().to(torch.float16)
    tq, tk, tv = to_f16(q), to_f16(kc), to_f16(vc)
    out = paged_attention(tq, tk, tv, torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev),
                          scale, bs, chunk=0)
    torch.cuda.synchronize()
    as_bits = lambda t: t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    want = paged_decode_attention_per_seq_ref(as_bits(tq), as_bits(tk), as_bits(tv), bt, ctx,
                                              scale, bs, dtype="f16")
    w = torch.from_numpy(want.view(np.int16)).view(torch.float16).float().numpy()
    g = out.float().cpu().numpy()
    assert (np.abs(g - w) <= ATOL + RTOL * np.abs(w)).all(), np.abs(g - w).max()


def test_stale_counter_is_flagged_and_the_workspace_recovers():
    """A counter that is not zero when a launch starts (an earlier launch cut short, two
    launches overlapping on one workspace) loses rows; the wave that sees more arrivals
    than the row has pieces raises the stale flag, which DecodeWorkspace.check() reads
    back; the call after that clears the region and is right again.  Every kernel ends
    normally."""
    print("case stale counter flag", flush=True)
    import torch
    from nanovllm_jax_amd import _lib, paged_attention
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace
    B, Hq, Hkv, D, bs = 3, 32, 8, 128, 64
    ctx = [3000, 2500, 2800]                            # every row shared by many sub-runs
    q, kc, vc, bt, ctx = make_problem(99, B, Hq, Hkv, D, bs, sum(-(-c // bs) for c in ctx) + 1, ctx)
    assert not deals_whole_rows(ctx, Hkv, bt.shape[1] * bs)[0]
    dev = "cuda:0"
    args = (bits_to_torch(q, dev), bits_to_torch(kc, dev), bits_to_torch(vc, dev),
            torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev), 0.088, bs)
    want = oracle(q, kc, vc, bt, ctx, 0.088, bs)
    ws = DecodeWorkspace.for_shape(B, Hq, D, bt.shape[1], bs, Hkv, dev)
    one = _lib.NVJ_PHASE_SPLITK
    good = paged_attention(*args, chunk=0, workspace=ws, phases=one)
    assert ws.check()
    assert_close_bf16(torch_to_bits(good), want, what="clean workspace")
    ws.counters[1 + 1 * Hkv + 5] = 1000                  # (sequence 1, KV head 5)
    bad = paged_attention(*args, chunk=0, workspace=ws, phases=one)
    assert not ws.check(), "the stale counter went unnoticed"
    rows = slice(5 * (Hq // Hkv), 6 * (Hq // Hkv))
    bad_bits, good_bits = torch_to_bits(bad), torch_to_bits(good)
    keep = np.ones(bad_bits.shape, bool)
    keep[1, rows] = False
    assert np.array_equal(bad_bits[keep], good_bits[keep]), "only the spoilt row may differ"
    again = paged_attention(*args, chunk=0, workspace=ws, phases=one)   # clears first
    assert ws.check()
    assert np.array_equal(torch_to_bits(again), good_bits)
    assert not ws.counters.any()


def _hip_runtime():
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    hip.hipMemcpy.restype = ctypes.c_int
    return hip


def test_library_owned_counters_one_launch_for_any_workspace():
    """nvj_paged_decode_launch_counters with counters = NULL: the partials in a buffer the
    caller owns and never initialises (what an XLA custom call is handed), the counters
    in the library's own region: bit-equal to nvj_paged_decode_launch on calls of
    different shapes in a row; a counter of that region set from outside is flagged and
    nvj_paged_decode_counters_reset(NULL) puts the region right again."""
    print("case library-owned counters", flush=True)
    import ctypes
    import torch
    from nanovllm_jax_amd import _lib
    lib = _lib.load()
    hip = _hip_runtime()
    dev = "cuda:0"
    stream = torch.cuda.current_stream().cuda_stream
    region = ctypes.c_void_p()
    size = ctypes.c_size_t()
    assert lib.nvj_paged_decode_library_counters(ctypes.byref(region), ctypes.byref(size)) == 0
    assert size.value == 64 << 10 and region.value

    def flag():
        torch.cuda.synchronize()
        word = ctypes.c_int32(-1)
        assert hip.hipMemcpy(ctypes.byref(word), region, 4, 2) == 0     # device to host
        return word.value

    def both(prob, scale, bs):
        q, kc, vc, bt, ctx = prob
        tq, tk, tv = (bits_to_torch(x, dev) for x in (q, kc, vc))
        tbt, tctx = torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev)
        B, Hq, D = q.shape
        NB, _, Hkv, _ = kc.shape
        MB = bt.shape[1]
        need = int(lib.nvj_paged_decode_workspace_bytes(B, Hq, D, MB, bs, Hkv, 0))
        part = need - int(lib.nvj_paged_decode_counter_bytes(B, Hq, Hkv))
        ws = torch.full((need,), 0xA5, dtype=torch.uint8, device=dev)
        pt = torch.full((part,), 0x5A, dtype=torch.uint8, device=dev)
        o1, o2 = torch.full_like(tq, 7.0), torch.full_like(tq, -7.0)
        assert lib.nvj_paged_decode_launch(stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                           tbt.data_ptr(), tctx.data_ptr(), o1.data_ptr(),
                                           ws.data_ptr(), need, B, Hq, Hkv, D, bs, MB, NB, scale,
                                           0, 0) == 0
        assert lib.nvj_paged_decode_launch_counters(
            stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), tbt.data_ptr(), tctx.data_ptr(),
            o2.data_ptr(), pt.data_ptr(), part, None, 0, B, Hq, Hkv, D, bs, MB, NB, scale, 0,
            _lib.NVJ_PHASE_SPLITK) == 0
        torch.cuda.synchronize()
        return torch_to_bits(o1), torch_to_bits(o2)

    assert lib.nvj_paged_decode_counters_reset(stream, None, 0) == 0
    bs, D = 64, 128
    cases = [(31, 12, 32, 8, [3000, 17, 0, 1024, 2049, 700, 1, 256, 1500, 333, 2900, 64]),
             (32, 3, 16, 8, [700, 90, 257]),
             (33, 40, 16, 8, [300 + 7 * i for i in range(40)])]
    for seed, B, Hq, Hkv, ctx in cases:
        prob = make_problem(seed, B, Hq, Hkv, D, bs, sum(-(-c // bs) for c in ctx) + 1, ctx)
        plain, shared = both(prob, 0.088, bs)
        assert np.array_equal(plain, shared), f"call {seed} differs"
        assert flag() == 0
        assert_close_bf16(shared, oracle(*prob, 0.088, bs), what=f"library counters {seed}")
    # set one counter of the region from outside: the next call notices
    seed, B, Hq, Hkv, ctx = cases[0]
    prob = make_problem(seed, B, Hq, Hkv, D, bs, sum(-(-c // bs) for c in ctx) + 1, ctx)
    bogus = ctypes.c_int32(12345)
    assert hip.hipMemcpy(ctypes.c_void_p(region.value + 4 * (1 + 0 * Hkv + 2)),
                         ctypes.byref(bogus), 4, 1) == 0                 # host to device
    plain, shared = both(prob, 0.088, bs)
    assert flag() == 1
    assert not np.array_equal(plain, shared)
    assert lib.nvj_paged_decode_counters_reset(stream, None, 0) == 0
    assert flag() == 0
    plain, shared = both(prob, 0.088, bs)
    assert np.array_equal(plain, shared) and flag() == 0


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
        assert not ws.counters.any(), f"replay {step} left a counter set"
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
