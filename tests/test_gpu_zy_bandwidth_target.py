"""The stated target, as a test: paged decode attention at the Qwen3-8B shape
(C2: B=64, ctx 4096) sustains at least 70 % of the 8 TB/s HBM peak, whole call,
in both the whole-sequence split and the length-agnostic balanced split (here with
a plain workspace, i.e. behind its counter-clearing launch, as a caller that cannot
keep a workspace would run it).  Measured values are ~86 % and ~85 %; the floor is
the target itself, so only a real regression (or a fallback path) trips it.
Collected late on purpose: a timing assertion should not hide other failures."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("chunk", [-1, 0])
def test_c2_whole_call_meets_the_bandwidth_target(chunk):
    print(f"case C2 bandwidth target chunk={chunk}", flush=True)
    import torch
    import bench
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.paged_attention import paged_decode_workspace_bytes
    from nanovllm_jax_amd.workloads import algorithmic_bytes, make_workload
    dev = torch.device("cuda:0")
    w = make_workload("C2")
    q, kc, vc, bt, ctx, *_ = bench.device_inputs(w, torch, dev)
    ws = torch.empty(max(16, paged_decode_workspace_bytes(w.batch, w.num_heads, w.head_dim,
                                                          w.max_blocks, w.block_size,
                                                          w.num_kv_heads, chunk)),
                     dtype=torch.uint8, device=dev)
    out = torch.empty_like(q)
    call = lambda: paged_attention(q, kc, vc, bt, ctx, w.scale, w.block_size, chunk=chunk,
                                   out=out, workspace=ws)
    for _ in range(20):
        call()
    best = min(bench.timed(call, 50, torch)[0] for _ in range(3))      # ms per call
    byts = algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads, w.head_dim,
                             w.max_blocks)
    frac = byts / (best * 1e-3) / 1e9 / bench.HBM_PEAK_GBPS
    print(f"C2 chunk={chunk}: {best * 1e3:.1f} us/call = {100 * frac:.1f} % of peak", flush=True)
    assert frac >= 0.70, f"{100 * frac:.1f} % of the HBM peak, target 70 %"


@pytest.mark.parametrize("name", ["C2_JITTER", "C2_SPREAD", "RAGGED_SHORT"])
def test_batches_of_unequal_lengths_meet_the_bandwidth_target(name):
    """The same floor for batches as a serving loop sees them (lengths a few percent
    apart, from half to one and a half times 4096, 256 short ragged sequences), through
    the balanced split with a kept workspace.  Measured: 85 %, 81 %, 82 %."""
    print(f"case bandwidth target {name}", flush=True)
    import torch
    import bench
    from nanovllm_jax_amd import paged_attention
    from nanovllm_jax_amd.layers.paged_attention import DecodeWorkspace
    from nanovllm_jax_amd.workloads import algorithmic_bytes, make_workload
    dev = torch.device("cuda:0")
    w = make_workload(name)
    q, kc, vc, bt, ctx, *_ = bench.device_inputs(w, torch, dev)
    ws = DecodeWorkspace.for_shape(w.batch, w.num_heads, w.head_dim, w.max_blocks, w.block_size,
                                   w.num_kv_heads, dev)
    out = torch.empty_like(q)
    call = lambda: paged_attention(q, kc, vc, bt, ctx, w.scale, w.block_size, chunk=0, out=out,
                                   workspace=ws)
    for _ in range(20):
        call()
    best = min(bench.timed(call, 50, torch)[0] for _ in range(3))      # ms per call
    assert ws.check(), "the workspace's counters were found stale"
    byts = algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads, w.head_dim,
                             w.max_blocks)
    frac = byts / (best * 1e-3) / 1e9 / bench.HBM_PEAK_GBPS
    print(f"{name}: {best * 1e3:.1f} us/call = {100 * frac:.1f} % of peak", flush=True)
    assert frac >= 0.70, f"{100 * frac:.1f} % of the HBM peak, target 70 %"
