"""Whole-model decode step harness: the HIP store + attention inside a small
Qwen3-shaped model, against an fp32 torch-CPU restatement of the same model
whose attention and store are the CPU oracle; and HIP-graph replays against the
eager step."""
import numpy as np
import pytest
import torch

from helpers import bits_to_torch, torch_to_bits

pytestmark = pytest.mark.gpu


def _small_runner(fused=True):
    from nanovllm_jax_amd.engine.decode_step import DecodeModelConfig, DecodeStepRunner
    cfg = DecodeModelConfig(num_layers=2, hidden_size=256, num_heads=4, num_kv_heads=2,
                            head_dim=128, intermediate_size=512, vocab_size=1024,
                            max_position=2048, block_size=256, num_kvcache_blocks=12)
    return cfg, DecodeStepRunner(cfg, "cuda:0", seed=3, fused_qk_rope_store=fused)


def _batch(cfg):
    seq_lens = [5, 256, 257, 700]
    rng = np.random.Generator(np.random.PCG64(9))
    pages = rng.permutation(cfg.num_kvcache_blocks).tolist()
    tables, off = [], 0
    for n in seq_lens:
        k = -(-n // cfg.block_size)
        tables.append(pages[off:off + k]); off += k
    last_tokens = rng.integers(0, cfg.vocab_size, len(seq_lens)).tolist()
    return last_tokens, seq_lens, tables


def _cpu_reference(runner, cfg, ids, pos, ctx_lens, slots, bt):
    """Same model in fp32 on the CPU; store and attention by the oracle."""
    from oracle.paged_attention_oracle import (paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    f = lambda t: t.detach().float().cpu()
    kv = runner.kv_cache.detach().cpu()
    h = f(runner.embed)[torch.from_numpy(ids).long()]
    bf = lambda t: t.to(torch.bfloat16).float()

    def rms(x, w, res=None):
        if res is not None:
            x = x + res
            res = bf(x)
        else:
            res = x
        return bf(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps) * f(w)), res

    cs = f(runner.cos_sin)[torch.from_numpy(pos).long()][:, None, :]
    cos, sin = cs.chunk(2, -1)
    rope = lambda x: torch.cat([x[..., :64] * cos - x[..., 64:] * sin,
                                x[..., 64:] * cos + x[..., :64] * sin], -1)
    residual = None
    qs, ks = cfg.num_heads * cfg.head_dim, cfg.num_kv_heads * cfg.head_dim
    for li, lw in enumerate(runner.layers):
        h, residual = rms(h, lw["ln1"], residual)
        qkv = bf(h @ f(lw["qkv"]).T)
        q, k, v = qkv.split([qs, ks, ks], -1)
        q = rms(q.reshape(-1, cfg.num_heads, cfg.head_dim), lw["q_norm"])[0]
        k = rms(k.reshape(-1, cfg.num_kv_heads, cfg.head_dim), lw["k_norm"])[0]
        v = v.reshape(-1, cfg.num_kv_heads, cfg.head_dim)
        q, k = rope(q), rope(k)
        flat = (-1, cfg.num_kv_heads, cfg.head_dim)
        kc, vc = store_kv_to_cache_ref(k.numpy().astype(np.float32),
                                       torch_to_bits(v.to(torch.bfloat16)),
                                       torch_to_bits(kv[0, li]).reshape(flat),
                                       torch_to_bits(kv[1, li]).reshape(flat), slots,
                                       negative_slots="skip")
        shape = kv[0, li].shape
        o = paged_decode_attention_per_seq_ref(torch_to_bits(q.to(torch.bfloat16)), kc.reshape(shape),
                                               vc.reshape(shape), bt, ctx_lens,
                                               cfg.head_dim ** -0.5, cfg.block_size)
        o = bits_to_torch(o).float().reshape(-1, qs)
        h = bf(o @ f(lw["o"]).T)
        h, residual = rms(h, lw["ln2"], residual)
        gate, up = bf(h @ f(lw["gate_up"]).T).chunk(2, -1)
        h = bf(bf(torch.nn.functional.silu(gate) * up) @ f(lw["down"]).T)
    h, _ = rms(h, runner.final_norm, residual)
    return h @ f(runner.embed).T


@pytest.mark.parametrize("fused", [True, False])
def test_decode_step_matches_cpu_model_with_oracle_attention(fused):
    print(f"case decode step vs CPU model fused={fused}", flush=True)
    from nanovllm_jax_amd.engine.decode_step import prepare_decode
    cfg, runner = _small_runner(fused)
    last, lens, tables = _batch(cfg)
    ids, pos, ctx_lens, slots, bt = prepare_decode(last, lens, tables, cfg.block_size)
    want = _cpu_reference(runner, cfg, ids, pos, ctx_lens, slots, bt)   # before the step mutates the cache
    inp, p, ctx = runner.make_inputs(last, lens, tables)
    logits = runner.forward(inp, p, ctx).float().cpu()
    torch.cuda.synchronize()
    err = (logits - want).abs().max().item()
    scale = want.abs().max().item()
    print(f"  logits max abs err {err:.3e} (max |logit| {scale:.3f})", flush=True)
    assert err <= 0.02 * scale + 0.02
    # slot formula put the new K/V rows where the filler says
    assert slots[0] == tables[0][-1] * cfg.block_size + 4


def test_graph_replays_match_eager_step():
    """Every replay is checked against the eager step, with eager work and
    synchronisation between replays."""
    print("case decode step graph replays", flush=True)
    cfg, runner = _small_runner()
    last, lens, tables = _batch(cfg)
    inp, p, ctx = runner.make_inputs(last, lens, tables)
    eager_logits = runner.forward(inp, p, ctx).clone()
    eager_tokens = eager_logits.argmax(-1).clone()
    torch.cuda.synchronize()
    replay = runner.capture(inp, p, ctx)
    for i in range(4):
        toks = replay().clone()
        torch.cuda.synchronize()
        again = runner.step(inp, p, ctx)          # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(toks, eager_tokens), f"replay {i} differs from eager"
        assert torch.equal(again, eager_tokens)


def test_captured_graph_keeps_a_workspace_of_its_own():
    """A captured step must not share its split workspace with eager steps or with
    other captures: an eager step of another batch size, and a second capture, between
    two replays leave the first graph's replays equal to the eager step of its batch.
    Ragged lengths, so rows are shared between workgroups and the counters are in use."""
    print("case captured graph owns its workspace", flush=True)
    from nanovllm_jax_amd.engine.decode_step import DecodeModelConfig, DecodeStepRunner
    cfg = DecodeModelConfig(num_layers=2, hidden_size=256, num_heads=4, num_kv_heads=2,
                            head_dim=128, intermediate_size=512, vocab_size=1024,
                            max_position=4096, block_size=256, num_kvcache_blocks=160)
    runner = DecodeStepRunner(cfg, "cuda:0", seed=5)
    rng = np.random.Generator(np.random.PCG64(21))
    lens = rng.integers(40, 1500, size=24).tolist()
    lens[3], lens[17] = 3000, 2600
    pages = rng.permutation(cfg.num_kvcache_blocks).tolist()
    tables, off = [], 0
    for n in lens:
        k = -(-n // cfg.block_size)
        tables.append(pages[off:off + k]); off += k
    last = rng.integers(0, cfg.vocab_size, len(lens)).tolist()
    big = runner.make_inputs(last, lens, tables)
    small = runner.make_inputs(last[:10], lens[:10], tables[:10])
    want_big = runner.step(*big).clone()
    want_small = runner.step(*small).clone()
    torch.cuda.synchronize()
    replay_big = runner.capture(*big)
    assert torch.equal(replay_big(), want_big)
    assert torch.equal(runner.step(*small), want_small)      # eager, another batch size
    assert torch.equal(replay_big(), want_big)
    replay_small = runner.capture(*small)                    # a second capture
    assert torch.equal(replay_small(), want_small)
    assert torch.equal(replay_big(), want_big)
    assert torch.equal(runner.step(*big), want_big)
    assert torch.equal(replay_small(), want_small)
    torch.cuda.synchronize()
    assert replay_big.workspace is not replay_small.workspace
    assert replay_big.workspace.check() and replay_small.workspace.check()
    assert runner._eager_ws.check()


def test_advance_decode_matches_oracle_over_many_steps():
    """Device-resident metadata advance, bit-exact against the oracle, with the
    host only maintaining the block tables."""
    print("case advance_decode many steps", flush=True)
    from nanovllm_jax_amd import create_decode_context
    from nanovllm_jax_amd.engine.decode_step import advance_decode
    from oracle.paged_attention_oracle import advance_decode_ref, prepare_decode_ref
    bs = 32
    rng = np.random.Generator(np.random.PCG64(4))
    B = 300
    lens = rng.integers(1, 200, B).tolist()
    lens[5] = 64; lens[6] = 65; lens[7] = 63
    free = list(range(5000))
    tables = [[free.pop() for _ in range(-(-n // bs))] for n in lens]
    ids, pos, ctx, slots, bt = prepare_decode_ref(rng.integers(0, 50000, B).tolist(), lens, tables, bs)
    ctx[11] = 0                                       # an inactive row
    width = bt.shape[1] + 2
    bt_host = np.full((B, width), -1, np.int32); bt_host[:, :bt.shape[1]] = bt
    dev = "cuda:0"
    t = lambda a: torch.from_numpy(a.copy()).to(dev)
    d_ids, d_pos = t(ids), t(pos)
    d_ctx = create_decode_context(t(ctx), t(slots), t(bt_host))
    for step in range(40):
        for i in range(B):                            # host keeps the tables current
            if ctx[i] > 0 and (ctx[i] + 1) % bs == 1 and len(tables[i]) < width - 1:
                tables[i].append(free.pop()); bt_host[i, len(tables[i]) - 1] = tables[i][-1]
        d_ctx.block_tables.copy_(torch.from_numpy(bt_host))
        dtype = np.int64 if step % 2 else np.int32
        nxt = rng.integers(0, 50000, B).astype(dtype)
        ids, pos, ctx, slots = advance_decode_ref(nxt, ids, pos, ctx, slots, bt_host, bs)
        advance_decode(t(nxt), d_ids, d_pos, d_ctx, bs)
        torch.cuda.synchronize()
        assert np.array_equal(d_ids.cpu().numpy(), ids), step
        assert np.array_equal(d_pos.cpu().numpy(), pos), step
        assert np.array_equal(d_ctx.context_lens.cpu().numpy(), ctx), step
        assert np.array_equal(d_ctx.slot_mapping.cpu().numpy(), slots), step
    assert (slots == -1).sum() >= 1 and ctx[11] == 0


def test_generation_graph_matches_host_driven_loop():
    """step + advance captured in one graph and replayed N times == N eager steps
    whose metadata the host rebuilds each time (the reference's way)."""
    print("case generation graph vs host loop", flush=True)
    cfg, dev_runner = _small_runner()
    _, host_runner = _small_runner()
    last, lens, tables = _batch(cfg)
    lens = [5, 250, 100, 700]                          # room inside the last page for 5 steps
    rng = np.random.Generator(np.random.PCG64(9))
    pages = rng.permutation(cfg.num_kvcache_blocks).tolist()
    tables, off = [], 0
    for n in lens:
        k = -(-(n + 6) // cfg.block_size)
        tables.append(pages[off:off + k]); off += k
    ids, pos, ctx = dev_runner.make_inputs(last, lens, tables)
    replay = dev_runner.capture_generation(ids, pos, ctx)
    cur_last, cur_lens = list(last), list(lens)
    for step in range(5):
        used = [t[:-(-n // cfg.block_size)] for t, n in zip(tables, cur_lens)]
        h_ids, h_pos, h_ctx = host_runner.make_inputs(cur_last, cur_lens, used)
        want = host_runner.step(h_ids, h_pos, h_ctx).cpu()
        got = replay().cpu()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"step {step}: {got.tolist()} vs {want.tolist()}"
        cur_last = want.tolist()
        cur_lens = [n + 1 for n in cur_lens]
    assert ctx.context_lens.cpu().tolist() == cur_lens


@pytest.mark.parametrize("fused", [True, False])
def test_prefill_then_decode_equals_one_longer_prefill(fused):
    """End to end over every kernel of the path: prefill the prompts (store +
    prefill attention), decode a few tokens (store + paged decode + metadata),
    and compare each decode step's logits with a fresh prefill of prompt +
    generated tokens (its last row sees exactly the same keys)."""
    print(f"case prefill then decode vs longer prefill fused={fused}", flush=True)
    cfg, runner = _small_runner(fused)
    _, check = _small_runner(fused)
    rng = np.random.Generator(np.random.PCG64(12))
    lens = [3, 250, 130]
    prompts = [rng.integers(0, cfg.vocab_size, n).tolist() for n in lens]
    pages = rng.permutation(cfg.num_kvcache_blocks).tolist()
    tables, off = [], 0
    for n in lens:
        k = -(-(n + 8) // cfg.block_size)
        tables.append(pages[off:off + k]); off += k
    ids, pos, ctx = runner.make_prefill_inputs(prompts, tables)
    logits = runner.forward(ids, pos, ctx).float()
    assert logits.shape == (len(lens), cfg.vocab_size)
    seqs = [list(p) for p in prompts]
    for step in range(4):
        nxt = logits.argmax(-1).tolist()
        for s_, t_ in zip(seqs, nxt):
            s_.append(int(t_))
        # reference: prefill everything again on a runner with a clean cache
        c_ids, c_pos, c_ctx = check.make_prefill_inputs(seqs, tables)
        want = check.forward(c_ids, c_pos, c_ctx).float()
        # path under test: one decode step on top of the cache built so far
        used = [t[:-(-len(s_) // cfg.block_size)] for t, s_ in zip(tables, seqs)]
        d_ids, d_pos, d_ctx = runner.make_inputs(nxt, [len(s_) for s_ in seqs], used)
        logits = runner.forward(d_ids, d_pos, d_ctx).float()
        torch.cuda.synchronize()
        err = (logits - want).abs().max().item()
        scale = want.abs().max().item()
        print(f"  step {step}: max |logit diff| {err:.3e} (max |logit| {scale:.2f})", flush=True)
        assert err <= 0.015 * scale + 0.01


@pytest.mark.parametrize("fused", [True, False])
def test_prefill_in_two_chunks_equals_one_prefill(fused):
    """Chunked prefill over the whole layer stack: the first part of every prompt
    is prefilled and cached, the rest is prefilled behind it (keys and values of
    both parts read from the paged cache, positions and slots of the second part
    only), and the logits of the last tokens match a one-shot prefill."""
    print(f"case prefill in two chunks fused={fused}", flush=True)
    cfg, runner = _small_runner(fused)
    _, check = _small_runner(fused)
    rng = np.random.Generator(np.random.PCG64(13))
    lens = [70, 300, 131, 9]
    first = [64, 129, 0, 8]               # cached before the second chunk (0: nothing)
    prompts = [rng.integers(0, cfg.vocab_size, n).tolist() for n in lens]
    pages = rng.permutation(cfg.num_kvcache_blocks).tolist()
    tables, off = [], 0
    for n in lens:
        k = -(-n // cfg.block_size)
        tables.append(pages[off:off + k]); off += k
    ids, pos, ctx = check.make_prefill_inputs(prompts, tables)
    want = check.forward(ids, pos, ctx).float()
    # chunk 1: the sequences that have a first part
    part = [i for i, c in enumerate(first) if c > 0]
    ids, pos, ctx = runner.make_prefill_inputs([prompts[i][:first[i]] for i in part],
                                               [tables[i] for i in part])
    runner.forward(ids, pos, ctx)
    # chunk 2: everything that is left, behind the cached part
    ids, pos, ctx = runner.make_prefill_inputs(prompts, tables, num_cached_tokens=first)
    assert ctx.block_tables is not None and int(ctx.cu_seqlens_q[-1]) == sum(lens) - sum(first)
    got = runner.forward(ids, pos, ctx).float()
    torch.cuda.synchronize()
    err = (got - want).abs().max().item()
    scale = want.abs().max().item()
    print(f"  max |logit diff| {err:.3e} (max |logit| {scale:.2f})", flush=True)
    assert err <= 0.015 * scale + 0.01
    assert torch.equal(got.argmax(-1), want.argmax(-1))
    # the caches of both runners hold the same rows
    assert torch.equal(runner.kv_cache, check.kv_cache)


def test_full_size_c5_step_graph_equals_eager_and_layer0_attention_matches_the_oracle():
    """Config C5 at full size: 28 layers, hidden 1024, Hq=16, Hkv=8, D=128, vocab 151936,
    B=128, every sequence at context 1024, page 256.  The step captured as one HIP graph
    picks the tokens the eager step picks, no cache row other than the slots the filler
    computed is written in any layer, and the attention output of layer 0 (its q, the cache
    with the new row in it) is within the bar of the C oracle."""
    print("case C5 full-size decode step", flush=True)
    import torch.nn.functional as F
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.engine.decode_step import DecodeModelConfig, DecodeStepRunner
    from nanovllm_jax_amd.layers.qk_rope_store import qk_norm_rope_store
    from oracle import c_oracle
    from oracle.paged_attention_oracle import bf16_bits_to_f32
    cfg = DecodeModelConfig()
    batch, ctx_len = 128, 1024
    runner = DecodeStepRunner(cfg, "cuda:0", seed=1005)
    rng = np.random.Generator(np.random.PCG64(1005))
    pages = rng.permutation(cfg.num_kvcache_blocks).reshape(batch, -1)[:, :ctx_len // cfg.block_size]
    last = rng.integers(0, cfg.vocab_size, batch).tolist()
    ids, pos, ctx = runner.make_inputs(last, [ctx_len] * batch, pages.tolist())
    before = runner.kv_cache[:, :, :, :, 0, 0].clone()       # one element per cache row
    eager = runner.step(ids, pos, ctx).clone()
    torch.cuda.synchronize()
    # exactly the rows named by slot_mapping changed, in every layer, K and V
    changed = (runner.kv_cache[:, :, :, :, 0, 0] != before).flatten(2)       # [2, L, slots]
    want_rows = torch.zeros(changed.shape[-1], dtype=torch.bool, device=changed.device)
    want_rows[ctx.slot_mapping.long()] = True
    assert not (changed & ~want_rows).any(), "a cache row that no slot names was written"
    # (a new value can coincide with the old one in the single element compared)
    assert changed.sum().item() >= 0.98 * 2 * cfg.num_layers * batch
    replay = runner.capture(ids, pos, ctx)
    for i in range(2):
        assert torch.equal(replay(), eager), f"replay {i} differs from the eager step"
    # layer 0, recomputed up to the attention call
    lw, attn = runner.layers[0], runner.attn[0]
    h, _ = runner._rms(F.embedding(ids.long(), runner.embed), lw["ln1"])
    q = qk_norm_rope_store(F.linear(h, lw["qkv"]), pos, runner.cos_sin, lw["q_norm"], lw["k_norm"],
                           cfg.rms_norm_eps, attn.k_cache, attn.v_cache, ctx.slot_mapping,
                           cfg.num_heads, cfg.num_kv_heads, cfg.head_dim)
    for chunk in (0, -1):
        out = paged_attention(q, attn.k_cache, attn.v_cache, ctx.block_tables, ctx.context_lens,
                              attn.scale, attn.block_size, chunk=chunk)
        torch.cuda.synchronize()
        want = c_oracle.paged_decode(torch_to_bits(q), torch_to_bits(attn.k_cache),
                                     torch_to_bits(attn.v_cache), ctx.block_tables.cpu().numpy(),
                                     ctx.context_lens.cpu().numpy(), attn.scale, attn.block_size,
                                     return_f32=True)
        got = bf16_bits_to_f32(torch_to_bits(out))
        err = np.abs(got - want)
        assert (err <= 1e-2 + 1e-2 * np.abs(want)).all(), f"chunk {chunk}: max err {err.max()}"
