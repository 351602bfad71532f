#!/usr/bin/env python3
"""Benchmark of the paged-decode hot path on one MI355X.

A step is one paged decode attention call (split-K launch + combine launch)
over one synthetic batch that is already resident in HBM.  The default
workload is C2 (Qwen3-8B shape: B=64, Hq=32, Hkv=8, D=128, page 256,
ctx 4096).  One JSON line is printed on stdout.

  value                GB/s = algorithmic bytes per call / mean time per call
  roofline.achieved    same bytes / mean duration of the split-K kernel alone,
                       timed with events on the launch stream
  cpu_baseline         the CPU oracle (a NumPy port of the reference's pure-JAX
                       paged attention) on a bounded sample of the same batch
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

# HBM bytes per decode launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this very command, scaled by the same counters over a plain 1 GiB copy
# (FETCH_SIZE x1.9999, WRITE_SIZE x1.0).  Keyed by (workload, chunk); other
# configurations report null.
MEASURED_TRAFFIC_BYTES = {("C2", 0): 1_080_210_000, ("C2", 1024): 1_080_188_000,
                          ("C2", -1): 1_074_909_000}


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


def timed_in_graph(fn, torch, calls=20, replays=20):
    """Mean ms per call when `calls` back-to-back calls are replayed from one HIP
    graph (launch cost of the host binding excluded)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
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
    return {"value": round(byts / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "us_per_call_full_batch": round(med / max(pos, 1) * int(w.context_lens.sum()) * 1e6, 1),
            "sample": f"{impl}, {cores} threads, first {n} of {w.batch} sequences of {w.name} "
                      f"({pos} positions), median of {len(times)} calls of {med * 1e3:.1f} ms"}


def bench_decode_step(args, torch):
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
    for _ in range(args.warmup):
        replay()
    ms, wall = timed(replay, args.steps, torch)
    ms_eager, _ = timed(lambda: runner.step(ids, pos, ctx), max(3, args.steps // 10), torch)
    kv_bytes = cfg.num_layers * batch * ctx_len * cfg.num_kv_heads * cfg.head_dim * 2 * 2
    rec = {"metric": "decode tokens/s, Qwen3-0.6B shape whole-model decode step", "value":
           round(batch / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": round(wall, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "C5: 28 layers, hidden 1024, Hq=16, Hkv=8, D=128, vocab 151936, "
                                  "B=128, ctx=1024, page=256, random-init weights, greedy",
                      "step": "one HIP graph: embedding .. LM head .. argmax",
                      "kv_bytes_per_step": kv_bytes},
           "ms_per_step_eager": round(ms_eager, 4), "graph_matches_eager": same}
    print(json.dumps(rec), flush=True)
    return 0


MFMA_BF16_PEAK_TFLOPS = 2500.0


def bench_prefill(args, torch):
    """Variable-length causal prefill attention at the Qwen3-8B head shape
    (Hq=32, Hkv=8, D=128): 8 prompts of 4096 tokens, packed.  Reports TFLOP/s
    (4 * Hq * D flop per visible (query, key) pair) against the dense bf16 MFMA
    peak."""
    from nanovllm_jax_amd import paged_prefill_attention, variable_length_attention_prefill
    dev = torch.device("cuda:0")
    hq, hkv, d = 32, 8, 128
    lens = [int(x) for x in args.prefill_lens.split(",")]
    prefix = int(args.prefill_prefix)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    g = torch.Generator(device=dev)
    g.manual_seed(7)
    total = int(cu[-1])
    q = torch.randn((total, hq, d), generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn((total, hkv, d), generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn((total, hkv, d), generator=g, device=dev).to(torch.bfloat16)
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
        cu_k = torch.from_numpy(np.concatenate([[0], np.cumsum(lens_k)]).astype(np.int32)).to(dev)
        bt_t = torch.from_numpy(bt).to(dev)
        fn = lambda: paged_prefill_attention(q, kc, vc, bt_t, cu_t, cu_k, d ** -0.5, out=out)
    for _ in range(args.warmup):
        fn()
    ms, wall = timed(fn, args.steps, torch)
    pairs = sum(n * (n + 1) // 2 + n * prefix for n in lens)
    flops = 4.0 * hq * d * pairs
    tflops = flops / (ms * 1e-3) / 1e12
    rec = {"metric": "prefill attention TFLOP/s (causal, varlen, Qwen3-8B head shape)",
           "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": round(wall, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": f"prefill: Hq={hq} Hkv={hkv} D={d}, prompt lengths {lens}" +
                                  (f" behind {prefix} cached positions each (paged cache)"
                                   if prefix > 0 else ""),
                      "flops_per_call": flops},
           "roofline": {"bound": "mfma", "achieved": round(tflops, 1),
                        "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                        "kernel": "prefill_attention_kernel", "kernel_us": round(ms * 1e3, 1)}}
    print(json.dumps(rec), flush=True)
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2", choices=["C1", "C2", "C3", "C4", "C5", "R1"])
    ap.add_argument("--chunk", type=int, default=None,
                    help="split mode: 0 = balanced, > 0 = positions per workgroup, -1 = whole "
                         "sequence per workgroup; default: what the host filler would pick from "
                         "the workload's lengths (layers.paged_attention.choose_split)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16"],
                    help="cache / q / out dtype; f16 is what the reference's own timing "
                         "scripts use")
    ap.add_argument("--products", default="mfma", choices=["mfma", "valu"],
                    help="valu: time the measurement variant of the split-K kernel that does "
                         "Q.K and P.V with vector-ALU dot products (group 4 or 8, bf16, "
                         "balanced or whole-sequence split)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    from nanovllm_jax_amd import _lib, paged_attention, store_kv_to_cache
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace, choose_split
    from nanovllm_jax_amd.workloads import algorithmic_bytes, make_workload

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.decode_step:
        return bench_decode_step(args, torch)
    if args.prefill:
        return bench_prefill(args, torch)
    w = make_workload(args.workload)
    dt = torch.float16 if args.dtype == "f16" else torch.bfloat16
    q, kc, vc, bt, ctx, slots, k_new, v_new = device_inputs(w, torch, dev, dt)
    # like the reference's filler, the workload generator knows the lengths on the host
    chunk = (choose_split(w.context_lens, w.num_kv_heads, w.num_heads) if args.chunk is None
             else args.chunk)
    split_name = {0: "balanced", -1: "whole sequence per workgroup"}.get(chunk,
                                                                        f"fixed chunk {chunk}")
    kernel_name = {0: "paged_decode_balanced_kernel", -1: "paged_decode_whole_kernel"}.get(
        chunk, "paged_decode_splitk_kernel")
    ws = DecodeWorkspace.for_shape(w.batch, w.num_heads, w.head_dim, w.max_blocks, w.block_size,
                                   w.num_kv_heads, dev, chunk)
    out = torch.empty_like(q)
    kflat = kc.view(-1, w.num_kv_heads, w.head_dim)
    vflat = vc.view(-1, w.num_kv_heads, w.head_dim)

    variant = _lib.NVJ_PHASE_VALU_PRODUCTS if args.products == "valu" else 0

    def decode(phases=3):
        paged_attention(q, kc, vc, bt, ctx, w.scale, w.block_size, chunk=chunk, out=out,
                        workspace=ws, phases=phases | variant)

    def store():
        store_kv_to_cache(k_new, v_new, kflat, vflat, slots)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    store()
    for _ in range(args.warmup):
        decode()
    ms_call, ms_wall = timed(decode, args.steps, torch)
    ms_splitk, _ = timed(lambda: decode(_lib.NVJ_PHASE_SPLITK), args.steps, torch)
    ms_combine, _ = timed(lambda: decode(_lib.NVJ_PHASE_COMBINE), args.steps, torch)
    ms_store, _ = timed(store, args.steps, torch)
    ms_graph = timed_in_graph(decode, torch)

    byts = algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads, w.head_dim,
                             w.max_blocks)
    gbps = byts / (ms_call * 1e-3) / 1e9
    gbps_kernel = byts / (ms_splitk * 1e-3) / 1e9
    rec = {
        "metric": "paged decode attn HBM GB/s (us/call alongside), Qwen3-8B shape B=64 ctx4k"
                  if w.name == "C2" else f"paged decode attn HBM GB/s, workload {w.name}",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_wall, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "us_per_call": round(ms_call * 1e3, 2),
        "us_per_call_in_graph": round(ms_graph * 1e3, 2),
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "config": {"workload": f"{w.name}: B={w.batch} Hq={w.num_heads} Hkv={w.num_kv_heads} "
                               f"D={w.head_dim} page={w.block_size} "
                               f"ctx={int(w.context_lens.min())}..{int(w.context_lens.max())} "
                               f"pool={w.num_blocks} pages",
                   "split": split_name, "products": args.products,
                   "algorithmic_bytes_per_call": byts,
                   "step": "one launch" if chunk == -1 else "split-K launch + combine launch"},
        "roofline": {"bound": "hbm", "achieved": round(gbps_kernel, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(gbps_kernel / HBM_PEAK_GBPS, 4),
                     "traffic": (MEASURED_TRAFFIC_BYTES.get((w.name, chunk))
                                 if args.products == "mfma" else None),
                     "kernel": kernel_name,
                     "kernel_us": round(ms_splitk * 1e3, 2)},
        # back-to-back launches of these two short kernels are paced by the host
        # (one Python -> ctypes call each), not by the kernels themselves
        "host_paced_launch_us": {"paged_decode_combine_kernel":
                                 None if chunk == -1 else round(ms_combine * 1e3, 2),
                                 "store_kvcache_kernel": round(ms_store * 1e3, 2)},
    }
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline(w, q, kc, vc, args.cpu_budget, args.dtype)
    print(json.dumps(rec), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
