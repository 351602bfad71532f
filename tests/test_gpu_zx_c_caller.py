"""The C ABI driven from a plain-C program (no C++, torch or Python in that
process): KV store + paged decode of one problem, results compared with the
CPU oracle (store bit-exact, attention atol/rtol 1e-2)."""
import os
import subprocess

import numpy as np
import pytest

from helpers import assert_close_bf16, make_problem

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CALLER = os.path.join(ROOT, "nanovllm_jax_amd", "_native", "nvj_c_caller")


@pytest.mark.parametrize("chunk,k_f32", [(0, True), (-1, False), (64, True)])
def test_plain_c_program_stores_and_decodes(tmp_path, chunk, k_f32):
    print(f"case plain-C caller chunk={chunk} k_f32={k_f32}", flush=True)
    from oracle.paged_attention_oracle import (paged_decode_attention_per_seq_ref,
                                               store_kv_to_cache_ref)
    if not os.path.exists(CALLER):
        pytest.skip("nvj_c_caller is not built here (build() compiles csrc/c_caller/nvj_c_caller.c)")
    B, Hq, Hkv, D, bs, NB = 6, 16, 4, 128, 64, 40
    ctx = np.array([1, 64, 65, 130, 300, 33])
    q, kc, vc, bt, ctx = make_problem(990 + chunk, B, Hq, Hkv, D, bs, NB, ctx)
    rng = np.random.Generator(np.random.PCG64(991))
    # the new token of every sequence goes to its last position
    slots = np.array([bt[b, (n - 1) // bs] * bs + (n - 1) % bs for b, n in enumerate(ctx)],
                     np.int32)
    k_new = rng.standard_normal((B, Hkv, D), dtype=np.float32)
    v_new = (rng.standard_normal((B, Hkv, D), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
    if not k_f32:
        k_new = (k_new.view(np.uint32) >> 16).astype(np.uint16)
    scale = np.float32(D ** -0.5)
    problem, result = tmp_path / "problem.bin", tmp_path / "result.bin"
    with open(problem, "wb") as f:
        f.write(np.array([B, Hq, Hkv, D, bs, bt.shape[1], NB, chunk, 0, int(k_f32), 0, 0],
                         np.int32).tobytes())
        f.write(scale.tobytes())
        for a in (q, kc, vc, bt.astype(np.int32), ctx.astype(np.int32), slots, k_new, v_new):
            f.write(np.ascontiguousarray(a).tobytes())
    run = subprocess.run([CALLER, str(problem), str(result)], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    raw = np.fromfile(result, dtype=np.uint16)
    n_out, n_cache = B * Hq * D, NB * bs * Hkv * D
    assert raw.size == n_out + 2 * n_cache
    out = raw[:n_out].reshape(B, Hq, D)
    kc_after = raw[n_out:n_out + n_cache].reshape(NB * bs, Hkv, D)
    vc_after = raw[n_out + n_cache:].reshape(NB * bs, Hkv, D)
    flat = (NB * bs, Hkv, D)
    wk, wv = store_kv_to_cache_ref(k_new, v_new, kc.reshape(flat), vc.reshape(flat), slots,
                                   negative_slots="skip")
    assert np.array_equal(kc_after, wk) and np.array_equal(vc_after, wv), "store not bit-exact"
    want = paged_decode_attention_per_seq_ref(q, wk.reshape(kc.shape), wv.reshape(vc.shape), bt,
                                              ctx, float(scale), bs)
    assert_close_bf16(out, want, what=f"plain-C caller chunk={chunk}")
