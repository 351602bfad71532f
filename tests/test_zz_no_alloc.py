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
    before = torch.cuda.memory_allocated()
    rc = lib.nvj_paged_decode_static_launch(stream, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                            tbt.data_ptr(), tctx.data_ptr(), out_st.data_ptr(),
                                            B, Hq, Hkv, D, bs, MB, NB, scale, 0)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
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
