#!/usr/bin/env python3
"""Benchmark of the paged-decode hot path on one MI355X.

A step is one paged decode attention call over one synthetic batch that is
already resident in HBM.  The default workload is C2 (Qwen3-8B shape: B=64,
Hq=32, Hkv=8, D=128, page 256, ctx 4096) in the balanced split (chunk 0, the
mode a caller that does not know the lengths on the host gets), which is one
kernel launch.  One JSON line is printed on stdout.

  value                GB/s = algorithmic bytes per call / mean time per call
  roofline.achieved    same bytes / mean duration of the attention kernel alone,
                       timed with events on the launch stream
  cpu_baseline         the CPU oracle on a bounded sample of the same batch: the
                       C restatement (OpenMP), and under "literal" the NumPy
                       restatement of the reference's own materialising algorithm
  others               the other workloads and neighbours of the path, each
                       timed in this same run (skipped with --no-others)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per decode launch as measured by rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs of this command on an earlier day, scaled by the same counters over a plain
# 1 GiB copy.  Not measured by the run that prints them: reported with the file
# they come from, and only for the exact configuration that was profiled.
PROFILED_TRAFFIC = {
    ("C2", 0, "bf16", "mfma"): (1_075_029_000, "profiles/paged_decode_balanced_kernel_C2.md"),
    ("RAGGED_SHORT", 0, "bf16", "mfma"): (1_182_717_000,
                                          "profiles/paged_decode_balanced_kernel_ragged_batches.md"),
    ("C2", -1, "bf16", "mfma"): (1_074_914_000, "profiles/paged_decode_whole_kernel_C2.md"),
}


def device_inputs(w, torch, dev, dt=None):
    """Seeded N(0,1) q / K / V of dtype `dt` (bf16 by default) drawn on the
    device, plus the metadata."""
    dt = dt or torch.bfloat16
    g = torch.Generator(device=dev)
    g.manual_seed(w.seed)
    shape = (w.num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
    kc = torch.empty(shape, dtype=dt, device=dev)
    vc = torch.empty(shape, dtype=dt, device=dev)
    # page by page keeps the fp32 temporaries small at the multi-GiB configs
    step = max(1, (1 << 26) // (w.block_size * w.num_kv_heads * w.head_dim))
    for t in (kc, vc):
        for p0 in range(0, w.num_blocks, step):
            n = min(step, w.num_blocks - p0)
            t[p0:p0 + n] = torch.randn((n,) + shape[1:], generator=g, device=dev,
                                       dtype=torch.float32).to(dt)
    q = (torch.randn((w.batch, w.num_heads, w.head_dim), generator=g, device=dev,
                     dtype=torch.float32) * w.q_gain).to(dt)
    k_new = torch.randn((w.batch, w.num_kv_heads, w.head_dim), generator=g, device=dev,
                        dtype=torch.float32)
    v_new = torch.randn((w.batch, w.num_kv_heads, w.head_dim), generator=g, device=dev,
                        dtype=torch.float32).to(dt)
    bt = torch.from_numpy(w.block_tables).to(dev)
    ctx = torch.from_numpy(w.context_lens).to(dev)
    slots = torch.from_numpy(w.slot_mapping).to(dev)
    return q, kc, vc, bt, ctx, slots, k_new, v_new


def to_bits(t):
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def timed(fn, steps, torch):
    """Mean ms per call over `steps` back-to-back calls, from events on the
    current stream, plus the wall-clock mean."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return start.elapsed_time(end) / steps, (t1 - t0) * 1e3 / steps


# one side stream for every warm-up before a capture (see others_block: streams are kept few)
_warmup_stream = None


def timed_in_graph(fn, torch, calls=20, replays=20, warm_seconds=0.2):
    """Mean ms per call when `calls` back-to-back calls are replayed from one HIP
    graph (launch cost of the host binding excluded)."""
    global _warmup_stream
    if _warmup_stream is None:
        _warmup_stream = torch.cuda.Stream()
    side = _warmup_stream
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    # replays behind host-side work find the GPU's clocks down: warm up by time
    until = time.perf_counter() + warm_seconds
    graph.replay()
    while time.perf_counter() < until:
        graph.replay()
        torch.cuda.synchronize()
    ms, _ = timed(graph.replay, replays, torch)
    return ms / calls


def cpu_baseline(w, q, kc, vc, budget_s=20.0, dtype="bf16"):
    """The CPU oracle on the host cores (C restatement, OpenMP over
    (sequence, kv head)), same inputs, on a bounded sample: whole calls over
    the first `n` sequences of the batch, 2 warm-up + up to 5 timed calls
    within the time budget; median.  Falls back to the single-threaded NumPy
    restatement when the C oracle has not been built."""
    from nanovllm_jax_amd.workloads import algorithmic_bytes
    from oracle import c_oracle
    qb, kb, vb = to_bits(q), to_bits(kc), to_bits(vc)
    if c_oracle.available():
        fn, cores, impl = c_oracle.paged_decode, c_oracle.num_threads(), "C oracle (OpenMP)"
    else:
        from oracle.paged_attention_oracle import paged_decode_attention_per_seq_ref
        fn, cores, impl = paged_decode_attention_per_seq_ref, 1, "NumPy oracle"

    def call(n):
        t0 = time.perf_counter()
        fn(qb[:n], kb, vb, w.block_tables[:n], w.context_lens[:n], w.scale, w.block_size,
           dtype=dtype)
        return time.perf_counter() - t0

    # size the sample so one call costs at most ~1/7 of the budget
    n = min(w.batch, max(1, cores))
    t = call(n)
    while n < w.batch and t * 2 < budget_s / 7:
        n = min(w.batch, n * 2)
        t = call(n)
    times = []
    spent = 0.0
    call(n)
    while len(times) < 5 and (spent + t < budget_s or not times):
        t = call(n)
        times.append(t)
        spent += t
    med = float(np.median(times))
    byts = algorithmic_bytes(w.context_lens[:n], n, w.num_heads, w.num_kv_heads, w.head_dim,
                             w.max_blocks)
    pos = int(w.context_lens[:n].sum())
    rec = {"value": round(byts / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
           "us_per_call_full_batch": round(med / max(pos, 1) * int(w.context_lens.sum()) * 1e6, 1),
           "sample": f"{impl}, {cores} threads, first {n} of {w.batch} sequences of {w.name} "
                     f"({pos} positions), median of {len(times)} calls of {med * 1e3:.1f} ms; "
                     "a streaming restatement written for speed, which flatters the CPU: the "
                     "reference's own algorithm is under 'literal'"}
    if dtype == "bf16":
        rec["literal"] = cpu_baseline_literal(w, qb, kb, vb, budget_s / 2)
    return rec


def cpu_baseline_literal(w, qb, kb, vb, budget_s):
    """The reference's algorithm as it stands (layers/pallas_attention.py:188-236:
    gather the pages of the whole table, repeat K/V for the query group, convert to
    fp32, masked softmax over every table position), restated in NumPy, on the
    first sequences of the batch: as many as keep one call within the budget and
    the fp32 copies within a few GiB."""
    from nanovllm_jax_amd.workloads import algorithmic_bytes
    from oracle.paged_attention_oracle import paged_decode_attention_vectorized_ref
    per_seq = 2 * w.max_blocks * w.block_size * w.num_heads * w.head_dim * 4   # K and V, fp32
    n_max = max(1, min(w.batch, (8 << 30) // per_seq))

    def call(n):
        t0 = time.perf_counter()
        paged_decode_attention_vectorized_ref(qb[:n], kb, vb, w.block_tables[:n],
                                              w.context_lens[:n], w.scale, w.block_size)
        return time.perf_counter() - t0

    n, t = 1, call(1)
    while n < n_max and t * 2 * 2 < budget_s:       # one more timed call must still fit
        n = min(n_max, n * 2)
        t = call(n)
    t = min(t, call(n)) if t * 2 < budget_s else t
    byts = algorithmic_bytes(w.context_lens[:n], n, w.num_heads, w.num_kv_heads, w.head_dim,
                             w.max_blocks)
    pos = int(w.context_lens[:n].sum())
    return {"value": round(byts / t / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "us_per_call_full_batch": round(t / max(pos, 1) * int(w.context_lens.sum()) * 1e6, 1),
            "sample": f"NumPy restatement of paged_decode_attention_vectorized, first {n} of "
                      f"{w.batch} sequences of {w.name} ({pos} positions), best of the calls "
                      f"made, {t * 1e3:.0f} ms"}


def decode_step_record(steps, warmup, torch):
    """Whole-model decode step at the Qwen3-0.6B shape: 28 layers, B=128, every
    sequence at context 1024, page 256, random bf16 weights, greedy pick; the
    step is one HIP graph.  Reports decode tokens/s."""
    from nanovllm_jax_amd.engine.decode_step import DecodeModelConfig, DecodeStepRunner
    cfg = DecodeModelConfig()
    batch, ctx_len = 128, 1024
    runner = DecodeStepRunner(cfg, "cuda:0", seed=1005)
    rng = np.random.Generator(np.random.PCG64(1005))
    pages = rng.permutation(cfg.num_kvcache_blocks).reshape(batch, -1)[:, :ctx_len // cfg.block_size]
    last = rng.integers(0, cfg.vocab_size, batch).tolist()
    ids, pos, ctx = runner.make_inputs(last, [ctx_len] * batch, pages.tolist())
    eager = runner.step(ids, pos, ctx).clone()
    replay = runner.capture(ids, pos, ctx)
    same = bool(torch.equal(replay(), eager))
    for _ in range(warmup):
        replay()
    ms, wall = timed(replay, steps, torch)
    ms_eager, _ = timed(lambda: runner.step(ids, pos, ctx), max(3, steps // 10), torch)
    kv_bytes = cfg.num_layers * batch * ctx_len * cfg.num_kv_heads * cfg.head_dim * 2 * 2
    rec = {"metric": "decode tokens/s, Qwen3-0.6B shape whole-model decode step", "value":
           round(batch / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": round(wall, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "C5: 28 layers, hidden 1024, Hq=16, Hkv=8, D=128, vocab 151936, "
                                  "B=128, ctx=1024, page=256, random-init weights, greedy",
                      "step": "one HIP graph: embedding .. LM head .. argmax",
                      "kv_bytes_per_step": kv_bytes},
           "ms_per_step_eager": round(ms_eager, 4), "graph_matches_eager": same}
    del runner, replay
    return rec


MFMA_BF16_PEAK_TFLOPS = 2500.0


def prefill_record(lens, prefix, steps, warmup, torch, zero_inputs=False):
    """Variable-length causal prefill attention at the Qwen3-8B head shape
    (Hq=32, Hkv=8, D=128): 8 prompts of 4096 tokens, packed.  Reports TFLOP/s
    (4 * Hq * D flop per visible (query, key) pair) against the dense bf16 MFMA
    peak.  `zero_inputs`: q, k and v all zero, a measuring aid: the kernel issues
    the same instructions in the same number of cycles, but operands that never
    toggle draw little power, so the chip holds its full clock and the figure shows
    what the kernel's cycle count alone would give."""
    from nanovllm_jax_amd import paged_prefill_attention, variable_length_attention_prefill
    dev = torch.device("cuda:0")
    hq, hkv, d = 32, 8, 128
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    total = int(cu[-1])
    q = torch.randn((total, hq, d), generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn((total, hkv, d), generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn((total, hkv, d), generator=g, device=dev).to(torch.bfloat16)
    if zero_inputs:
        q.zero_(), k.zero_(), v.zero_()
    cu_t = torch.from_numpy(cu).to(dev)
    out = torch.empty_like(q)
    fn = lambda: variable_length_attention_prefill(q, k, v, cu_t, cu_t, scale=d ** -0.5, out=out)
    if prefix > 0:
        # every prompt sits behind `prefix` cached positions: keys and values come
        # from a paged cache (page 256, pages in random order)
        bs = 256
        lens_k = [n + prefix for n in lens]
        nblk = [-(-n // bs) for n in lens_k]
        rng = np.random.Generator(np.random.PCG64(7))
        pages = rng.permutation(sum(nblk))
        bt = np.full((len(lens), max(nblk)), -1, np.int32)
        used = 0
        for i, n in enumerate(nblk):
            bt[i, :n] = pages[used:used + n]
            used += n
        kc = torch.randn((sum(nblk), bs, hkv, d), generator=g, device=dev).to(torch.bfloat16)
        vc = torch.randn((sum(nblk), bs, hkv, d), generator=g, device=dev).to(torch.bfloat16)
        if zero_inputs:
            kc.zero_(), vc.zero_()
        cu_k = torch.from_numpy(np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)).to(dev)
        bt_t = torch.from_numpy(bt).to(dev)
        fn = lambda: paged_prefill_attention(q, kc, vc, bt_t, cu_t, cu_k, d ** -0.5, out=out)
    for _ in range(warmup):
        fn()
    ms, wall = timed(fn, steps, torch)
    pairs = sum(n * (n + 1) // 2 + n * prefix for n in lens)
    flops = 4.0 * hq * d * pairs
    tflops = flops / (ms * 1e-3) / 1e12
    rec = {"metric": "prefill attention TFLOP/s (causal, varlen, Qwen3-8B head shape)",
           "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": round(wall, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
           "data": "all zeros (clock probe)" if zero_inputs else "synthetic",
           "config": {"workload": f"prefill: Hq={hq} Hkv={hkv} D={d}, prompt lengths {lens}" +
                                  (f" behind {prefix} cached positions each (paged cache)"
                                   if prefix > 0 else ""),
                      "flops_per_call": flops},
           "roofline": {"bound": "mfma", "achieved": round(tflops, 1),
                        "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                        "kernel": "prefill_attention_kernel", "kernel_us": round(ms * 1e3, 1)}}
    return rec


def decode_record(name, chunk, dtype, products, steps, warmup, torch, dev, in_graph=False,
                  keep_inputs=False, warm_seconds=0.0, shared_rows=False):
    """Time the decode call (and the KV store) on one workload.  Returns the
    measurements, plus the device inputs when `keep_inputs`.  `warm_seconds`:
    keep making untimed calls for that long after the `warmup` calls (a workload
    measured behind host-side work finds the GPU's clocks down)."""
    from nanovllm_jax_amd import _lib, paged_attention, store_kv_to_cache
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace
    from nanovllm_jax_amd.workloads import algorithmic_bytes, make_workload
    w = make_workload(name)
    dt = torch.float16 if dtype == "f16" else torch.bfloat16
    q, kc, vc, bt, ctx, slots, k_new, v_new = device_inputs(w, torch, dev, dt)
    # one workspace kept across the calls of this stream: its counters are zero
    # between calls, so a balanced call is a single launch
    ws = DecodeWorkspace.for_shape(w.batch, w.num_heads, w.head_dim, w.max_blocks, w.block_size,
                                   w.num_kv_heads, dev, chunk)
    out = torch.empty_like(q)
    kflat = kc.view(-1, w.num_kv_heads, w.head_dim)
    vflat = vc.view(-1, w.num_kv_heads, w.head_dim)
    variant = {"valu": _lib.NVJ_PHASE_VALU_PRODUCTS, "none": _lib.NVJ_PHASE_LOADS_ONLY}.get(
        products, 0)
    if shared_rows:      # the equal cut with rows shared between workgroups, whatever the lengths
        variant |= _lib.NVJ_PHASE_SHARED_ROWS

    def decode(phases=_lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE):
        paged_attention(q, kc, vc, bt, ctx, w.scale, w.block_size, chunk=chunk, out=out,
                        workspace=ws, phases=phases | variant)

    def store():
        store_kv_to_cache(k_new, v_new, kflat, vflat, slots)

    store()
    for _ in range(warmup):
        decode()
    if warm_seconds > 0:
        torch.cuda.synchronize()
        until = time.perf_counter() + warm_seconds
        while time.perf_counter() < until:
            for _ in range(10):
                decode()
            torch.cuda.synchronize()
    ms_call, ms_wall = timed(decode, steps, torch)
    # the attention kernel alone: all there is for chunk 0 and -1, the first of the
    # two launches for a fixed chunk
    ms_kernel = ms_call if chunk <= 0 else timed(lambda: decode(_lib.NVJ_PHASE_SPLITK), steps,
                                                 torch)[0]
    ms_store, _ = timed(store, steps, torch)
    m = {"workload": w, "ms_call": ms_call, "ms_wall": ms_wall, "ms_kernel": ms_kernel,
         "ms_store": ms_store,
         "bytes": algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads,
                                    w.head_dim, w.max_blocks)}
    if in_graph:
        m["ms_graph"] = timed_in_graph(decode, torch)
        m["ms_store_graph"] = timed_in_graph(store, torch)
    if keep_inputs:
        m["inputs"] = (q, kc, vc)
    return m


def brief(m):
    """One workload's line in the `others` block."""
    gbps = m["bytes"] / (m["ms_call"] * 1e-3) / 1e9
    r = {"us_per_call": round(m["ms_call"] * 1e3, 2), "GB/s": round(gbps, 1),
         "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2)}
    if "ms_graph" in m:
        r["us_per_call_in_graph"] = round(m["ms_graph"] * 1e3, 2)
        r["store_us_per_call_in_graph"] = round(m["ms_store_graph"] * 1e3, 2)
    return r


def others_block(args, torch, dev):
    """The numbers quoted beside the headline, measured in this same run: the
    other split of C2, the other workloads in the default split, C1 inside a HIP
    graph (it is launch-bound), the prefill kernel and the whole-model decode
    step.  Fewer timed steps than the headline; every figure says what it is.
    The decode step comes last, and every graph timing warms up on the same side
    stream: long kernels have measured ~3 % slower for the rest of a process after
    work on further streams or after device memory went back to the driver."""
    st, wu = max(10, args.steps // 2), max(5, args.warmup)
    o = {"split": "balanced (chunk 0, one launch) unless a key says otherwise", "steps": st}

    def run(key, fn):
        try:
            o[key] = fn()
        except Exception as e:          # one failing extra must not take the headline down
            o[key] = {"error": f"{type(e).__name__}: {e}"}

    # each workload is built on the host first, which leaves the GPU idle: warm up by time
    warm = dict(warm_seconds=0.2)
    run("C2_whole_sequence_split", lambda: brief(decode_record("C2", -1, "bf16", "mfma", st, wu,
                                                              torch, dev, **warm)))
    # the headline batch is the special case of equal lengths (whole rows dealt to the
    # workgroups, nothing shared): the same shape with lengths that differ, and with
    # the general layout (rows shared between workgroups) forced
    run("C2_jitter_ctx_3840_4096", lambda: brief(decode_record(
        "C2_JITTER", 0, "bf16", "mfma", st, wu, torch, dev, **warm)))
    run("C2_spread_ctx_2048_6144", lambda: brief(decode_record(
        "C2_SPREAD", 0, "bf16", "mfma", st, wu, torch, dev, **warm)))
    run("C2_rows_shared_between_workgroups", lambda: brief(decode_record(
        "C2", 0, "bf16", "mfma", st, wu, torch, dev, shared_rows=True, **warm)))
    run("ragged_short_B256_ctx_200_2048", lambda: brief(decode_record(
        "RAGGED_SHORT", 0, "bf16", "mfma", st, wu, torch, dev, **warm)))
    run("C1", lambda: brief(decode_record("C1", 0, "bf16", "mfma", st, wu, torch, dev,
                                          in_graph=True, **warm)))
    run("C5_layer", lambda: brief(decode_record("C5", 0, "bf16", "mfma", st, wu, torch, dev,
                                                **warm)))
    run("C4", lambda: brief(decode_record("C4", 0, "bf16", "mfma", st, wu, torch, dev, **warm)))
    run("C3", lambda: brief(decode_record("C3", 0, "bf16", "mfma", st, wu, torch, dev, **warm)))

    def prefill():
        r = prefill_record([4096] * 8, 0, max(5, st // 5), 2, torch)
        # the same launch on all-zero inputs: same cycles at the chip's full clock
        z = prefill_record([4096] * 8, 0, max(5, st // 5), 2, torch, zero_inputs=True)
        return {"TFLOP/s": r["value"], "pct_of_mfma_bf16_peak": round(100 * r["roofline"]["frac"], 2),
                "us_per_call": r["roofline"]["kernel_us"],
                "TFLOP/s_on_zero_inputs_clock_probe": z["value"],
                "workload": r["config"]["workload"]}
    run("prefill_8x4096", prefill)

    def step():
        r = decode_step_record(max(5, st // 5), 2, torch)
        return {"tokens/s": r["value"], "ms_per_step": round(128 / r["value"] * 1e3, 4),
                "ms_per_step_eager": r["ms_per_step_eager"],
                "graph_matches_eager": r["graph_matches_eager"],
                "workload": r["config"]["workload"]}
    run("C5_decode_step", step)
    return o


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2",
                    help="C1..C5, R1, C2_JITTER, C2_SPREAD, RAGGED_SHORT, or "
                         "UNIFORM:<batch>:<lo>:<hi>[:<kv heads>[:<query heads>]] "
                         "(lengths uniform in [lo, hi])")
    ap.add_argument("--shared-rows", action="store_true",
                    help="balanced split: keep the kernel from dealing whole rows to the "
                         "workgroups (the equal cut with shared rows, whatever the lengths)")
    ap.add_argument("--chunk", type=int, default=0,
                    help="split mode: 0 = balanced (one launch, the default), > 0 = positions "
                         "per workgroup plus a combine launch, -1 = whole sequence per workgroup")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16"],
                    help="cache / q / out dtype; f16 is what the reference's own timing "
                         "scripts use")
    ap.add_argument("--products", default="mfma", choices=["mfma", "valu", "none"],
                    help="valu: time the measurement variant of the kernel that does "
                         "Q.K and P.V with vector-ALU dot products (group 4 or 8, bf16, "
                         "balanced or whole-sequence split); none: the variant that only "
                         "streams K and V (no arithmetic: the memory stream by itself)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the `others` block (the other workloads, prefill, decode step)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy a few times, so a "
                         "counter run has a kernel of known traffic to scale against")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--prefill", action="store_true",
                    help="time the prefill attention kernel instead; prints its own JSON line")
    ap.add_argument("--prefill-lens", default=",".join(["4096"] * 8),
                    help="comma-separated prompt lengths for --prefill")
    ap.add_argument("--prefill-prefix", type=int, default=0,
                    help="with --prefill: cached positions in front of every prompt; keys and "
                         "values are then read from a paged cache")
    ap.add_argument("--prefill-zero-inputs", action="store_true",
                    help="with --prefill: q, k, v all zero (a clock probe: same instructions and "
                         "cycles, little power, so the chip holds its full clock)")
    ap.add_argument("--decode-step", action="store_true",
                    help="time the whole-model decode step (config C5) instead of the "
                         "attention call; prints its own JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (every (sequence, kv head) pair is "
              "independent, so more GPUs would just split the batch); --gpus must be 1",
              file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the paged-decode path has no CPU implementation",
              file=sys.stderr)
        return 1

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.decode_step:
        print(json.dumps(decode_step_record(args.steps, args.warmup, torch)), flush=True)
        return 0
    if args.prefill:
        lens = [int(x) for x in args.prefill_lens.split(",")]
        print(json.dumps(prefill_record(lens, int(args.prefill_prefix), args.steps, args.warmup,
                                        torch, zero_inputs=args.prefill_zero_inputs)), flush=True)
        return 0

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    chunk = args.chunk
    # the W warm-up calls are 3 ms of work; the clocks of an idle GPU take longer to
    # come up, so untimed calls go on for a fifth of a second before the K timed ones
    m = decode_record(args.workload, chunk, args.dtype, args.products, args.steps, args.warmup,
                      torch, dev, in_graph=True, keep_inputs=True, warm_seconds=0.2,
                      shared_rows=args.shared_rows)
    w = m["workload"]
    split_name = {0: "balanced", -1: "whole sequence per workgroup"}.get(chunk,
                                                                        f"fixed chunk {chunk}")
    kernel_name = {0: "paged_decode_balanced_kernel", -1: "paged_decode_whole_kernel"}.get(
        chunk, "paged_decode_splitk_kernel")
    byts = m["bytes"]
    gbps = byts / (m["ms_call"] * 1e-3) / 1e9
    gbps_kernel = byts / (m["ms_kernel"] * 1e-3) / 1e9
    traffic, traffic_source = PROFILED_TRAFFIC.get((w.name, chunk, args.dtype, args.products),
                                                   (None, None))
    rec = {
        "metric": "paged decode attn HBM GB/s (us/call alongside), Qwen3-8B shape B=64 ctx4k"
                  if w.name == "C2" else f"paged decode attn HBM GB/s, workload {w.name}",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(m["ms_wall"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "us_per_call": round(m["ms_call"] * 1e3, 2),
        "us_per_call_in_graph": round(m["ms_graph"] * 1e3, 2),
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "config": {"workload": f"{w.name}: B={w.batch} Hq={w.num_heads} Hkv={w.num_kv_heads} "
                               f"D={w.head_dim} page={w.block_size} "
                               f"ctx={int(w.context_lens.min())}..{int(w.context_lens.max())} "
                               f"pool={w.num_blocks} pages",
                   "split": split_name + (", rows shared between workgroups forced"
                                          if args.shared_rows else ""),
                   "products": args.products,
                   "algorithmic_bytes_per_call": byts,
                   "step": "split-K launch + combine launch" if chunk > 0 else "one launch"},
        "roofline": {"bound": "hbm", "achieved": round(gbps_kernel, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(gbps_kernel / HBM_PEAK_GBPS, 4),
                     # not measured by this run: the counter figure of an earlier
                     # profile of this configuration, with the file it is in
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": kernel_name,
                     "kernel_us": round(m["ms_kernel"] * 1e3, 2)},
        # eager launches of this short kernel are paced by the host binding (one
        # Python -> ctypes call each); inside a graph only the kernel remains
        "store_kvcache_us": {"host_paced": round(m["ms_store"] * 1e3, 2),
                             "in_graph": round(m["ms_store_graph"] * 1e3, 2)},
    }
    q, kc, vc = m.pop("inputs")
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(w, q, kc, vc, args.cpu_budget, args.dtype)
    # (freed blocks stay with torch's allocator on purpose: memory handed back to
    # the driver and mapped again has measured 3-6 % slower for these kernels)
    del q, kc, vc, m
    if not args.no_others:
        rec["others"] = others_block(args, torch, dev)
    print(json.dumps(rec), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
