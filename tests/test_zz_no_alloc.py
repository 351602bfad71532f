"""The allocation-free decode entry point (nvj_paged_decode_static_launch, its
workspace in a device array inside the library) against
nvj_paged_decode_launch(chunk = 0) with a caller-owned workspace: bit-equal
outputs on calls in a row, the second with a smaller input, and within the
attention parity bar of the CPU oracle.  Both are called through the C ABI."""
import numpy as np
import pytest

from helpers import assert_close_bf16, bits_to_torch, make_problem, torch_to_bits

pytestmark = pytest.mark.gpu


def _call_pair(lib, prob, scale, bs):
    import torch
    q, kc, vc, bt, ctx = prob
    dev = "cuda:0"
    tq, tk, tv = (bits_to_torch(x, dev) for x in (q, kc, vc))
    tbt, tctx = torch.from_numpy(bt).to(dev), torch.from_numpy(ctx).to(dev)
    B, Hq, D = q.shape
    NB, _, Hkv, _ = kc.shape
    MB = bt.shape[1]
    need = int(lib.nvj_paged_decode_workspace_bytes(B, Hq, D, MB, bs, Hkv, 0))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    out_ws = torch.full_like(tq, 7.0)
    out_st = torch.full_like(tq, -7.0)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.nvj_paged_decode_launch(stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                     tbt.data_ptr(), tctx.data_ptr(), out_ws.data_ptr(),
                                     ws.data_ptr(), ws.numel(), B, Hq, Hkv, D, bs, MB, NB,
                                     scale, 0, 0)
    assert rc == 0, rc
    static = lambda: lib.nvj_paged_decode_static_launch(
        stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), tbt.data_ptr(), tctx.data_ptr(),
        out_st.data_ptr(), B, Hq, Hkv, D, bs, MB, NB, scale, 0)
    assert static() == 0          # (the first call on a device looks the array's address up)
    torch.cuda.synchronize()
    # free device memory as the driver counts it (torch's own counter would not see a
    # hipMalloc made inside the library) and torch's allocator, before and after
    free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    out_st.fill_(-7.0)
    assert static() == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_reserved() == held_before
    return torch_to_bits(out_ws), torch_to_bits(out_st)


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from nanovllm_jax_amd import _lib
    from oracle.paged_attention_oracle import paged_decode_attention_per_seq_ref
    lib = _lib.load()
    bs, D = 256, 128
    scale = float(1.0 / np.sqrt(D))
    # first call: ragged, several partials per sequence; second call: smaller in
    # every dimension, so most of what the first left in the array is stale
    # third call: more sequences again, so its counters are words the smaller call did
    # not use
    cases = [(21, 12, 32, 8, 64, [3000, 17, 0, 1024, 2049, 700, 1, 256, 1500, 333, 2900, 64]),
             (22, 3, 16, 8, 8, [700, 90, 257]),
             (23, 40, 16, 8, 128, [300 + 7 * i for i in range(40)])]
    for seed, B, Hq, Hkv, NB, ctx in cases:
        print(f"case static seed={seed} B={B} Hq={Hq} Hkv={Hkv}", flush=True)
        prob = make_problem(seed, B, Hq, Hkv, D, bs, NB, ctx)
        got_ws, got_st = _call_pair(lib, prob, scale, bs)
        assert np.array_equal(got_ws, got_st), "static-scratch call differs from workspace call"
        q, kc, vc, bt, c = prob
        want = paged_decode_attention_per_seq_ref(q, kc, vc, bt, c, scale, bs)
        assert_close_bf16(got_st, want, what=f"static seed={seed}")


def test_static_scratch_entry_point_replayed_from_a_graph():
    """What the entry point is for: the launch recorded into a HIP graph and replayed
    with the lengths changing between replays, each replay bit-equal to an eager call of
    the workspace entry point and leaving the library's counter region zero."""
    import ctypes
    import torch
    from nanovllm_jax_amd import _lib
    lib = _lib.load()
    print("case static launch in a graph", flush=True)
    dev, bs, D = "cuda:0", 256, 128
    B, Hq, Hkv, NB = 12, 32, 8, 64
    cap = np.array([3000, 17, 300, 1024, 2049, 700, 1, 256, 1500, 333, 2900, 64])
    q, kc, vc, bt, cap = make_problem(41, B, Hq, Hkv, D, bs, NB, cap)
    tq, tk, tv = (bits_to_torch(x, dev) for x in (q, kc, vc))
    tbt, tctx = torch.from_numpy(bt).to(dev), torch.from_numpy(cap).to(dev)
    MB = bt.shape[1]
    scale = float(1.0 / np.sqrt(D))
    out = torch.empty_like(tq)
    ref = torch.empty_like(tq)
    need = int(lib.nvj_paged_decode_workspace_bytes(B, Hq, D, MB, bs, Hkv, 0))
    ws = torch.empty(need, dtype=torch.uint8, device=dev)

    def static():
        rc = lib.nvj_paged_decode_static_launch(
            torch.cuda.current_stream().cuda_stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
            tbt.data_ptr(), tctx.data_ptr(), out.data_ptr(), B, Hq, Hkv, D, bs, MB, NB, scale, 0)
        assert rc == 0, rc

    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        static()
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static()
    region, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert lib.nvj_paged_decode_library_counters(ctypes.byref(region), ctypes.byref(size)) == 0
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    host = np.empty(size.value // 4, np.int32)
    rng = np.random.Generator(np.random.PCG64(8))
    for step in range(6):
        new_ctx = (cap * rng.random(B)).astype(np.int32) if step else cap.copy()
        new_ctx[rng.integers(0, B)] = 0
        tctx.copy_(torch.from_numpy(new_ctx).to(dev))
        out.fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert hip.hipMemcpy(host.ctypes.data, region, size.value, 2) == 0
        assert not host.any(), f"replay {step} left the counter region non-zero"
        rc = lib.nvj_paged_decode_launch(torch.cuda.current_stream().cuda_stream, tq.data_ptr(),
                                         tk.data_ptr(), tv.data_ptr(), tbt.data_ptr(),
                                         tctx.data_ptr(), ref.data_ptr(), ws.data_ptr(), need, B,
                                         Hq, Hkv, D, bs, MB, NB, scale, 0, 0)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert np.array_equal(torch_to_bits(out), torch_to_bits(ref)), f"replay {step} differs"


def test_static_scratch_limit_is_reported():
    """A problem whose partials exceed the array is refused before any launch."""
    from nanovllm_jax_amd import _lib
    lib = _lib.load()
    x = 0x1000
    need = lib.nvj_paged_decode_workspace_bytes(2048, 64, 128, 4, 256, 8, 0)
    assert need > _lib.NVJ_STATIC_SCRATCH_BYTES
    rc = lib.nvj_paged_decode_static_launch(None, x, x, x, x, x, x, 2048, 64, 8, 128, 256, 4, 64,
                                            0.1, 0)
    assert rc == _lib.NVJ_ERR_SCRATCH_LIMIT
    assert b"scratch" in lib.nvj_error_string(rc)
