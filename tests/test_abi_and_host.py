"""CPU-side checks: the C-ABI library loads and exports every symbol the header
declares; the host mirror validates its arguments and never computes on the
CPU; workload metadata follows the reference's filler formulas."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "nvj_paged_attn.h")).read()
    return re.findall(r"NVJ_API\s+[\w\s\*]+?\b(nvj_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    from nanovllm_jax_amd import _lib
    names = header_symbols()
    assert len(names) >= 7 and len(set(names)) == len(names)
    raw = ctypes.CDLL(_lib.lib_path())
    for n in names:
        assert hasattr(raw, n), f"{n} declared in the header but not exported"
    assert set(names) == set(_lib.SYMBOLS), "ctypes table and header disagree"
    lib = _lib.load()
    assert lib.nvj_abi_version() == _lib.NVJ_ABI_VERSION
    assert lib.nvj_error_string(0) == b"ok"
    for code in range(-8, 0):
        assert lib.nvj_error_string(code) not in (b"ok", b"unknown error code")


def test_argument_validation_without_a_gpu():
    """Entry points reject bad arguments before touching the device."""
    from nanovllm_jax_amd import _lib
    lib = _lib.load()
    L = lib.nvj_paged_decode_launch
    ok = dict(batch=2, Hq=32, Hkv=8, D=128, bs=256, MB=4, NB=16)

    def call(**kw):
        a = dict(ok); a.update(kw)
        p = kw.get("ptr", 0x1000)
        return L(None, p, p, p, p, p, p, p, 1 << 30, a["batch"], a["Hq"], a["Hkv"], a["D"],
                 a["bs"], a["MB"], a["NB"], 0.1, kw.get("chunk", 0), kw.get("dtype", 0))

    assert call(D=96) == -3                # head_dim not built (128 and 64 are)
    assert call(Hq=30) == -2               # Hq % Hkv
    assert call(bs=48) == -3
    assert call(chunk=100) == -3
    assert call(chunk=-2) == -2                   # only -1 (whole sequence) is a mode below 0
    assert call(batch=-1) == -2
    assert call(dtype=1) == -6                    # the cache is bf16 (0) or float16 (2), not f32
    assert call(dtype=3) == -6
    assert call(batch=0) == 0              # empty batch: nothing to do
    assert call(ptr=0) == -1
    assert call(ptr=0x1004) == -8          # misaligned
    assert L(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 16, 2, 32, 8, 128, 256,
             4, 16, 0.1, 0, 0) == -4       # workspace too small
    # the vector-ALU measurement variant exists for group 4 or 8, head_dim 128, bf16 only
    P = lib.nvj_paged_decode_launch_phases
    valu = _lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE | _lib.NVJ_PHASE_VALU_PRODUCTS
    x = 0x1000
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 16, 8, 128, 256, 4, 16, 0.1, 0, 0, valu) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 32, 8, 128, 256, 4, 16, 0.1, 0, 2, valu) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 32, 8, 128, 256, 4, 16, 0.1, 256, 0, valu) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 0, 32, 8, 128, 256, 4, 16, 0.1, 0, 0, valu) == 0
    # the loads-only measurement variant: head_dim 128, bf16, not with a fixed chunk or with valu
    lo = _lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_LOADS_ONLY
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 32, 8, 128, 256, 4, 16, 0.1, 256, 0, lo) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 32, 8, 128, 256, 4, 16, 0.1, 0, 2, lo) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 8, 2, 64, 256, 4, 16, 0.1, 0, 0, lo) == -3
    assert P(None, x, x, x, x, x, x, x, 1 << 30, 2, 32, 8, 128, 256, 4, 16, 0.1, 0, 0,
             lo | _lib.NVJ_PHASE_VALU_PRODUCTS) == -3
    # counter region of the balanced split: the stale flag, then one int32 per (sequence,
    # KV head as the kernels walk them: a group above 16 query heads counts as several),
    # padded to 256 bytes
    C = lib.nvj_paged_decode_counter_bytes
    assert C(64, 32, 8) == 2304 and C(1, 8, 8) == 256 and C(3, 32, 1) == 256
    assert C(100, 64, 2) == 1792          # (1 + 100 x 2 cache heads x 2 virtual heads of 16) x 4 B, padded
    assert C(0, 32, 8) == 0 and C(4, 30, 8) == 0
    # the balanced split with its counters apart from its partials
    LC = lib.nvj_paged_decode_launch_counters
    one = _lib.NVJ_PHASE_SPLITK
    assert LC(None, x, x, x, x, x, x, x, 1 << 30, x, 1 << 16, 2, 32, 8, 96, 256, 4, 16, 0.1, 0, one) == -3
    assert LC(None, x, x, x, x, x, x, x, 1 << 30, x, 16, 2, 32, 8, 128, 256, 4, 16, 0.1, 0, one) == -4
    assert LC(None, x, x, x, x, x, x, x, 16, x, 1 << 16, 2, 32, 8, 128, 256, 4, 16, 0.1, 0, one) == -4
    assert LC(None, x, x, x, x, x, x, x, 1 << 30, x + 2, 1 << 16, 2, 32, 8, 128, 256, 4, 16, 0.1, 0,
              one) == -8
    assert LC(None, x, x, x, x, x, x, x, 1 << 30, x, 1 << 16, 0, 32, 8, 128, 256, 4, 16, 0.1, 0, one) == 0
    # the library's own counter region holds 16383 counters
    assert LC(None, x, x, x, x, x, x, x, 1 << 30, None, 0, 2048, 8, 8, 128, 256, 4, 16, 0.1, 0,
              one) == -7
    R = lib.nvj_paged_decode_counters_reset
    assert R(None, x + 1, 64) == -8 and R(None, x, 0) == 0
    PP = lib.nvj_paged_prefill_attention_launch
    assert PP(None, x, x, x, x, x, x, x, 10, 2, 32, 8, 128, 48, 4, 16, 0.1, 0) == -3   # page % 32
    assert PP(None, x, x, x, x, x, x, x, 10, 2, 32, 8, 64, 64, 4, 16, 0.1, 0) == -3    # head_dim
    assert PP(None, x, x, x, x, x, x, x, 10, 2, 32, 8, 128, 64, 4, 16, 0.1, 1) == -6   # f32
    assert PP(None, x, x, x, 0, x, x, x, 10, 2, 32, 8, 128, 64, 4, 16, 0.1, 0) == -1   # no tables
    assert PP(None, x, x, x, x, x, x, x, 0, 2, 32, 8, 128, 64, 4, 16, 0.1, 0) == 0     # no rows
    S = lib.nvj_store_kvcache_launch
    assert S(None, 0, 0, 0, 0, 0, 0, 8, 128, 1024, 0, 0, 0) == 0       # no tokens
    assert S(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 4, 8, 128, 1024, 7, 0, 0) == -6
    assert S(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 4, 8, 128, 1024, 2, 0, 0) == -6  # f16 rows, bf16 cache
    assert S(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 4, 8, 128, 1024, 0, 0, 1) == -6  # f32 cache
    assert S(None, 0, 0x1000, 0x1000, 0x1000, 0x1000, 4, 8, 128, 1024, 0, 0, 0) == -1
    assert S(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 4, 3, 3, 1024, 0, 0, 0) == -3
    assert S(None, 0x1000, 0x1000, 0x1000, 0x1000, 0x1000, -4, 8, 128, 1024, 0, 0, 0) == -2


def test_workspace_and_chunk_queries():
    from nanovllm_jax_amd.layers.paged_attention import default_chunk, paged_decode_workspace_bytes
    c = default_chunk(64, 8, 16, 256)
    assert c % 32 == 0 and 32 <= c <= 4096
    need = paged_decode_workspace_bytes(64, 32, 128, 16, 256, 8, 256)
    assert need == 64 * 16 * 32 * (128 + 2) * 4
    assert paged_decode_workspace_bytes(64, 32, 128, 16, 256, 8, 100) == 0   # bad chunk
    # balanced split (no GPU here: 256 compute units assumed): counters, one int32 per
    # (sequence, KV head) padded to 256 bytes, then one partial slot per wave part of a
    # workgroup (<= 256 workgroups) plus one per (sequence, head group) row; at batch 64
    # a workgroup is 4 KV heads x 2 parts, at batch 2 it is 2 KV heads x 4 parts, and 1 KV
    # head x 8 parts for a single long sequence
    assert paged_decode_workspace_bytes(64, 32, 128, 16, 256, 8, 0) == \
        2304 + (256 * 2 + 64 * 2) * 4 * 4 * (128 + 2) * 4
    assert paged_decode_workspace_bytes(2, 8, 128, 1, 32, 8, 0) == 256 + (2 * 4 + 2 * 4) * 2 * 130 * 4
    assert paged_decode_workspace_bytes(1, 8, 128, 32, 256, 8, 0) == 256 + (256 * 8 + 8) * 130 * 4


def test_host_mirror_refuses_cpu_tensors():
    """No CPU fallback: host tensors are an error, not a slow path."""
    from nanovllm_jax_amd import Attention, create_decode_context, paged_attention, store_kv_to_cache
    q = torch.zeros(2, 32, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 256, 8, 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    ctx = torch.ones(2, dtype=torch.int32)
    with pytest.raises(ValueError, match="GPU"):
        paged_attention(q, kc, kc.clone(), bt, ctx, 0.1, 256)
    with pytest.raises(ValueError, match="GPU"):
        store_kv_to_cache(torch.zeros(2, 8, 128), torch.zeros(2, 8, 128), kc.view(-1, 8, 128),
                          kc.view(-1, 8, 128).clone(), torch.zeros(2, dtype=torch.int32))
    attn = Attention(32, 128, 0.1, 8, 256)
    c = create_decode_context(ctx, torch.zeros(2, dtype=torch.int32), bt)
    assert c.is_prefill is False and c.last_token_indices is None
    with pytest.raises(RuntimeError, match="set_kv_cache"):
        attn(q, q, q, c)
    attn.set_kv_cache(kc, kc.clone())
    with pytest.raises(ValueError, match="GPU"):
        attn(q, q[:, :8].contiguous(), q[:, :8].contiguous(), c)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from nanovllm_jax_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "_LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.NativeLibraryError, match="no fallback"):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "nanovllm_jax_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cc")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), f
                assert "paged_oracle" not in text, f


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_workload_metadata(name):
    from nanovllm_jax_amd.workloads import algorithmic_bytes, make_workload
    w = make_workload(name)
    bs = w.block_size
    assert w.block_tables.shape == (w.batch, w.max_blocks) and w.block_tables.dtype == np.int32
    nblk = -(-w.context_lens // bs)
    live = np.arange(w.max_blocks)[None, :] < nblk[:, None]
    assert (w.block_tables[~live] == -1).all()                       # -1 padding
    pages = w.block_tables[live]
    assert pages.min() >= 0 and pages.max() < w.num_blocks and len(set(pages.tolist())) == len(pages)
    # slot = block_table[-1] * block_size + last_block_num_tokens - 1
    for b in range(0, w.batch, max(1, w.batch // 8)):
        n = int(w.context_lens[b])
        last_tokens = n - (nblk[b] - 1) * bs
        assert w.slot_mapping[b] == w.block_tables[b, nblk[b] - 1] * bs + last_tokens - 1
    same = make_workload(name)
    assert np.array_equal(same.block_tables, w.block_tables)          # seeded
    if name == "C2":
        assert algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads,
                                 w.head_dim, w.max_blocks) == 1_074_794_752
    if name == "C4":
        assert algorithmic_bytes(w.context_lens, w.batch, w.num_heads, w.num_kv_heads,
                                 w.head_dim, w.max_blocks) == 2_148_016_192
    if name == "C3":
        assert w.context_lens.min() >= 16 and w.context_lens.max() <= 32768
        assert w.num_blocks == int(np.ceil(1.1 * nblk.sum()))


def test_choose_split_policy():
    from nanovllm_jax_amd.layers.paged_attention import WHOLE_SEQUENCE, choose_split
    assert choose_split([4096] * 64, 8) == WHOLE_SEQUENCE          # C2
    assert choose_split([1024] * 128, 8) == WHOLE_SEQUENCE         # C5
    assert choose_split([32768] * 16, 8) == 0                      # C4: too few workgroups
    assert choose_split([16, 32768] * 128, 8) == 0                 # ragged
    assert choose_split([], 8) == 0
    assert choose_split([2048] * 40, 8) == 0       # 320 workgroups: a second round at 25 %
    assert choose_split([2048] * 96, 8) == 0       # 384 workgroups
    assert choose_split([2048] * 250, 8) == WHOLE_SEQUENCE         # 250 of 256
    assert choose_split([2048] * 4096, 8) == WHOLE_SEQUENCE        # 16 full rounds


def test_reference_profile_shape_workload():
    """R1 restates the inputs of the reference's own timing script
    (profile_attention.py:19-34): MHA cache, identity tables, lengths in [200, 2048)."""
    from nanovllm_jax_amd.workloads import make_workload
    w = make_workload("R1")
    assert (w.batch, w.num_heads, w.num_kv_heads, w.head_dim, w.block_size) == (64, 32, 32, 128, 256)
    assert np.array_equal(w.block_tables, np.arange(512, dtype=np.int32).reshape(64, 8))
    assert w.context_lens.min() >= 200 and w.context_lens.max() < 2048


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it exits with a message that says so."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)


@pytest.mark.parametrize("name", ["C2_JITTER", "C2_SPREAD", "RAGGED_SHORT", "UNIFORM:12:100:900",
                                  "LOGUNIFORM:7:16:5000:4:8"])
def test_ragged_workload_metadata(name):
    """The ragged bench workloads: lengths inside their stated range, every live page of
    a block table distinct and inside the pool, slots pointing at the last position."""
    from nanovllm_jax_amd.workloads import make_workload
    w = make_workload(name)
    again = make_workload(name)
    assert np.array_equal(w.context_lens, again.context_lens)
    assert np.array_equal(w.block_tables, again.block_tables)
    lo, hi = {"C2_JITTER": (3840, 4096), "C2_SPREAD": (2048, 6144), "RAGGED_SHORT": (200, 2048),
              "UNIFORM:12:100:900": (100, 900), "LOGUNIFORM:7:16:5000:4:8": (16, 5000)}[name]
    assert w.context_lens.min() >= lo and w.context_lens.max() <= hi
    nblk = -(-w.context_lens.astype(np.int64) // w.block_size)
    live = np.concatenate([w.block_tables[b, :n] for b, n in enumerate(nblk)])
    assert live.min() >= 0 and live.max() < w.num_blocks
    assert len(np.unique(live)) == len(live)
    for b, n in enumerate(nblk):
        assert (w.block_tables[b, n:] == -1).all()
        last = int(w.context_lens[b]) - 1
        assert w.slot_mapping[b] == w.block_tables[b, last // w.block_size] * w.block_size + \
            last % w.block_size
    if name.startswith("LOGUNIFORM"):
        assert (w.num_kv_heads, w.num_heads) == (4, 8)
