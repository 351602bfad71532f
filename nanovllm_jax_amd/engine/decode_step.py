"""Whole-model decode step harness around the HIP attention path.

The measured path of this package is the KV-cache store and the paged decode
attention, with the element-wise stages next to it (QK-RMSNorm + RoPE + store,
RMSNorm + residual, SiLU-and-multiply) as single HIP launches; the rest of a
decode step (embedding, the QKV / output / MLP projections, the LM head,
greedy pick) is plain ``torch`` here (hipBLASLt GEMMs), written from the
architecture the reference
describes: ``models/qwen3.py:130-172`` (attention block: fused QKV, per-head
QK-RMSNorm when there is no QKV bias, RoPE, attention, output projection),
``:285-318`` (pre-norm decoder layer with fused residual), ``:366-393`` (stack
+ final norm), ``:472-491`` (tied LM head), ``layers/layernorm.py:31-79``,
``layers/rotary_embedding.py:13-37,50-106``, ``layers/activation.py:22-33``.
Cache allocation, wiring and the per-step metadata follow
``engine/model_runner.py:140-204, 225-246, 334-376``.

Weights are random (N(0, 0.02), bf16); greedy = argmax of the logits, the
temperature -> 0 limit of the reference's Gumbel-max sampler
(``layers/sampler.py:39-48``).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as F

from .. import _lib
from ..layers.activation import silu_and_mul
from ..layers.attention import Attention
from ..layers.layernorm import rms_norm
from ..layers.paged_attention import (DecodeWorkspace, choose_split, paged_attention,
                                      paged_decode_workspace_bytes)
from ..layers.prefill_attention import (paged_prefill_attention,
                                        variable_length_attention_prefill)
from ..layers.qk_rope_store import qk_norm_rope_store
from ..utils.context import AttentionContext, create_decode_context, create_prefill_context

__all__ = ["DecodeModelConfig", "DecodeStepRunner", "prepare_block_tables", "prepare_decode",
           "prepare_prefill", "advance_decode"]


@dataclass
class DecodeModelConfig:
    """Qwen3-0.6B shape by default."""
    num_layers: int = 28
    hidden_size: int = 1024
    num_heads: int = 16
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 3072
    vocab_size: int = 151936
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    max_position: int = 4096
    block_size: int = 256
    num_kvcache_blocks: int = 512


def prepare_block_tables(block_tables: list[list[int]]) -> np.ndarray:
    """Rows padded with -1 to the longest table (``engine/model_runner.py:225-246``)."""
    width = max(len(t) for t in block_tables)
    out = np.full((len(block_tables), width), -1, dtype=np.int32)
    for i, t in enumerate(block_tables):
        out[i, :len(t)] = t
    return out


def prepare_decode(last_tokens, seq_lens, block_tables, block_size):
    """Host filler of one decode step (``engine/model_runner.py:334-376``):
    ``positions = len - 1``, ``context_lens = len``,
    ``slot = block_table[-1] * block_size + last_block_num_tokens - 1``."""
    n = len(seq_lens)
    input_ids = np.asarray(last_tokens, dtype=np.int32)
    positions = np.empty(n, np.int32)
    context_lens = np.empty(n, np.int32)
    slot_mapping = np.empty(n, np.int32)
    for i, (length, table) in enumerate(zip(seq_lens, block_tables)):
        positions[i] = length - 1
        context_lens[i] = length
        last_block_tokens = length - (len(table) - 1) * block_size
        slot_mapping[i] = table[-1] * block_size + last_block_tokens - 1
    return input_ids, positions, context_lens, slot_mapping, prepare_block_tables(block_tables)


def prepare_prefill(token_lists, block_tables, block_size, num_cached_tokens=None):
    """Host filler of one prefill step (``engine/model_runner.py:248-332``): packed
    ``input_ids`` and ``positions`` of the tokens that are not cached yet,
    ``cu_seqlens_q`` over those, ``cu_seqlens_k`` over whole sequences, and per
    sequence the slots of the new tokens, page by page (:300-309).
    ``num_cached_tokens[i]`` leading tokens of sequence i already sit in the cache
    (0 everywhere by default); unlike the reference's block-granular prefix cache
    it may be any count.  Returns ``(input_ids, positions, cu_seqlens_q,
    cu_seqlens_k, slot_mapping, max_seqlen_q, max_seqlen_k)``."""
    lens = [len(t) for t in token_lists]
    cached = list(num_cached_tokens) if num_cached_tokens is not None else [0] * len(lens)
    new = [n - c for n, c in zip(lens, cached)]
    cu_q = np.zeros(len(lens) + 1, np.int32)
    cu_q[1:] = np.cumsum(new)
    cu_k = np.zeros(len(lens) + 1, np.int32)
    cu_k[1:] = np.cumsum(lens)
    input_ids = (np.concatenate([np.asarray(t[c:], np.int32) for t, c in zip(token_lists, cached)])
                 if lens else np.zeros(0, np.int32))
    positions = (np.concatenate([np.arange(c, n, dtype=np.int32) for n, c in zip(lens, cached)])
                 if lens else np.zeros(0, np.int32))
    slots = []
    for n, c, table in zip(lens, cached, block_tables):
        pos = np.arange(c, n)
        slots.append((np.asarray(table, np.int64)[pos // block_size] * block_size +
                      pos % block_size).astype(np.int32))
    slot_mapping = np.concatenate(slots) if slots else np.zeros(0, np.int32)
    return (input_ids, positions, cu_q, cu_k, slot_mapping, max(new) if new else 0,
            max(lens) if lens else 0)


def advance_decode(next_tokens, input_ids, positions, context: AttentionContext, block_size):
    """Advance the device-resident metadata of a decode batch by one step, in
    place: every active sequence grows by its ``next_tokens`` entry and
    ``input_ids / positions / context.context_lens / context.slot_mapping`` get
    the values ``prepare_decode`` would compute for the grown sequences
    (``engine/model_runner.py:334-376``), without a host round trip.
    ``context.block_tables`` must already hold the page a sequence is about to
    enter."""
    lib = _lib.load()
    bt = context.block_tables
    for name, t in (("next_tokens", next_tokens), ("input_ids", input_ids),
                    ("positions", positions), ("context_lens", context.context_lens),
                    ("slot_mapping", context.slot_mapping), ("block_tables", bt)):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous GPU tensor")
        if name != "next_tokens" and t.dtype != torch.int32:
            raise ValueError(f"{name} must be int32, got {t.dtype}")
    if next_tokens.dtype not in (torch.int32, torch.int64):
        raise ValueError("next_tokens must be int32 or int64")
    batch = input_ids.shape[0]
    for name, t in (("next_tokens", next_tokens), ("positions", positions),
                    ("context_lens", context.context_lens),
                    ("slot_mapping", context.slot_mapping)):
        if t.shape != (batch,):
            raise ValueError(f"{name} must have shape [{batch}]")
    if bt.dim() != 2 or bt.shape[0] != batch:
        raise ValueError("block_tables must be [batch, max_blocks]")
    with torch.cuda.device(input_ids.device):
        stream = torch.cuda.current_stream(input_ids.device).cuda_stream
        code = lib.nvj_advance_decode_launch(
            stream, next_tokens.data_ptr(), next_tokens.element_size(), input_ids.data_ptr(),
            positions.data_ptr(), context.context_lens.data_ptr(),
            context.slot_mapping.data_ptr(), bt.data_ptr(), batch, bt.shape[1], int(block_size))
    _lib.check(code, "nvj_advance_decode_launch")


class DecodeStepRunner:
    """Owns random weights, the KV cache ``[2, L, NB, bs, Hkv, D]`` bf16 and one
    ``Attention`` per layer; ``step`` runs one decode step for a batch."""

    def __init__(self, cfg: DecodeModelConfig, device="cuda:0", seed: int = 0,
                 fill_cache: bool = True, fused_qk_rope_store: bool = True,
                 fused_layer_glue: bool = True):
        self.cfg = cfg
        # True: RMSNorm (+ residual add) and SiLU-and-multiply as one HIP launch
        # each; False: the same stages as chains of torch kernels
        self.fused_layer_glue = fused_layer_glue
        # True: one HIP launch for QK-RMSNorm + RoPE + KV store; False: the
        # reference's op-by-op chain in torch followed by the plain store
        self.fused_qk_rope_store = fused_qk_rope_store
        self.device = torch.device(device)
        g = torch.Generator(device=self.device)
        g.manual_seed(seed)
        c = cfg

        def w(*shape):
            return (torch.randn(shape, generator=g, device=self.device, dtype=torch.float32)
                    * 0.02).to(torch.bfloat16)

        qkv_out = (c.num_heads + 2 * c.num_kv_heads) * c.head_dim
        self.embed = w(c.vocab_size, c.hidden_size)            # tied with the LM head
        self.layers = []
        for _ in range(c.num_layers):
            self.layers.append(dict(
                ln1=torch.ones(c.hidden_size, device=self.device),    # fp32, layernorm.py:29
                ln2=torch.ones(c.hidden_size, device=self.device),
                qkv=w(qkv_out, c.hidden_size),
                o=w(c.hidden_size, c.num_heads * c.head_dim),
                q_norm=torch.ones(c.head_dim, device=self.device),
                k_norm=torch.ones(c.head_dim, device=self.device),
                gate_up=w(2 * c.intermediate_size, c.hidden_size),
                down=w(c.hidden_size, c.intermediate_size)))
        self.final_norm = torch.ones(c.hidden_size, device=self.device)
        inv_freq = 1.0 / (c.rope_theta ** (torch.arange(0, c.head_dim, 2, dtype=torch.float32,
                                                        device=self.device) / c.head_dim))
        freqs = torch.outer(torch.arange(c.max_position, dtype=torch.float32,
                                         device=self.device), inv_freq)
        self.cos_sin = torch.cat([freqs.cos(), freqs.sin()], dim=-1)     # [max_pos, D] f32
        # KV cache, engine/model_runner.py:176,190
        shape = (2, c.num_layers, c.num_kvcache_blocks, c.block_size, c.num_kv_heads, c.head_dim)
        self.kv_cache = torch.zeros(shape, dtype=torch.bfloat16, device=self.device)
        if fill_cache:
            for layer in range(c.num_layers):
                for kv in range(2):
                    self.kv_cache[kv, layer] = torch.randn(
                        shape[2:], generator=g, device=self.device,
                        dtype=torch.float32).to(torch.bfloat16)
        self.attn = []
        for layer in range(c.num_layers):                        # _wire_kv_cache, :195-204
            a = Attention(c.num_heads, c.head_dim, c.head_dim ** -0.5, c.num_kv_heads,
                          c.block_size)
            a.set_kv_cache(self.kv_cache[0, layer], self.kv_cache[1, layer])
            self.attn.append(a)
        self._graph = None
        self._eager_ws = None
        self._eager_ws_shapes = set()

    # -- small torch pieces -------------------------------------------------
    def _rms(self, x, weight, residual=None):
        """RMSNorm, optionally fused with the residual add (layernorm.py:31-79).
        The HIP launch norms the unrounded fp32 sum as the reference does and
        updates the residual in place; the torch chain rounds the sum to the
        model dtype first (one bf16 rounding apart)."""
        if self.fused_layer_glue and x.dim() == 2:
            if residual is None:
                return rms_norm(x, weight, self.cfg.rms_norm_eps), x
            return rms_norm(x, weight, self.cfg.rms_norm_eps, residual, residual_out=residual)
        if residual is not None:
            x = (x.float() + residual.float()).to(x.dtype)
        return F.rms_norm(x, (x.shape[-1],), weight.to(x.dtype), self.cfg.rms_norm_eps), x

    def _silu_mul(self, gate_up):
        """SiLU(gate) * up of the fused projection (activation.py:22-33)."""
        if self.fused_layer_glue:
            return silu_and_mul(gate_up)
        gate, up = gate_up.chunk(2, dim=-1)
        return F.silu(gate) * up

    def _rope(self, x, cos, sin):
        """x bf16 [T, H, D]; result float32 like the reference's promotion
        (rotary_embedding.py:31-37)."""
        x1, x2 = x.chunk(2, dim=-1)
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)

    def forward(self, input_ids, positions, context: AttentionContext):
        c = self.cfg
        h = F.embedding(input_ids.long(), self.embed)
        residual = None
        cs = self.cos_sin[positions.long()][:, None, :]
        cos, sin = cs.chunk(2, dim=-1)
        qs, ks = c.num_heads * c.head_dim, c.num_kv_heads * c.head_dim
        for lw, attn in zip(self.layers, self.attn):
            if residual is None:
                h, residual = self._rms(h, lw["ln1"])
            else:
                h, residual = self._rms(h, lw["ln1"], residual)
            qkv = F.linear(h, lw["qkv"])
            if self.fused_qk_rope_store:
                q = qk_norm_rope_store(qkv, positions, self.cos_sin, lw["q_norm"], lw["k_norm"],
                                       c.rms_norm_eps, attn.k_cache, attn.v_cache,
                                       context.slot_mapping, c.num_heads, c.num_kv_heads,
                                       c.head_dim)
                if context.is_prefill and context.block_tables is not None:
                    # prompt rows behind a cached prefix: keys and values, the rows the
                    # fused launch just stored included, come from the paged cache
                    o = paged_prefill_attention(q, attn.k_cache, attn.v_cache,
                                                context.block_tables, context.cu_seqlens_q,
                                                context.cu_seqlens_k, attn.scale)
                elif context.is_prefill:
                    # K/V of the prompt rows were normalised, rotated and stored by
                    # the fused launch; the prefill kernel wants them packed, so
                    # they are gathered back from the cache rows just written
                    flat = (-1, c.num_kv_heads, c.head_dim)
                    sl = context.slot_mapping.long()
                    if bool((sl < 0).any()):    # a skipped row was never stored
                        raise ValueError("packed prefill through the fused store needs every "
                                         "prompt row stored: slot_mapping has negative entries")
                    o = variable_length_attention_prefill(
                        q, attn.k_cache.view(flat)[sl], attn.v_cache.view(flat)[sl],
                        context.cu_seqlens_q, context.cu_seqlens_k, scale=attn.scale)
                else:
                    o = paged_attention(q, attn.k_cache, attn.v_cache, context.block_tables,
                                        context.context_lens, attn.scale, attn.block_size,
                                        chunk=context.decode_split,
                                        workspace=attn.workspace or self._eager_workspace(context))
                h = F.linear(o.reshape(-1, qs), lw["o"])
                h, residual = self._rms(h, lw["ln2"], residual)
                h = F.linear(self._silu_mul(F.linear(h, lw["gate_up"])), lw["down"])
                continue
            q, k, v = qkv.split([qs, ks, ks], dim=-1)
            q = q.reshape(-1, c.num_heads, c.head_dim)
            k = k.reshape(-1, c.num_kv_heads, c.head_dim)
            v = v.reshape(-1, c.num_kv_heads, c.head_dim).contiguous()
            q, _ = self._rms(q, lw["q_norm"])
            k, _ = self._rms(k, lw["k_norm"])
            q = self._rope(q, cos, sin)                 # f32
            k = self._rope(k, cos, sin).contiguous()    # f32, the store rounds it to bf16
            o = attn(q.to(torch.bfloat16).contiguous(), k, v, context)
            h = F.linear(o.reshape(-1, qs), lw["o"])
            h, residual = self._rms(h, lw["ln2"], residual)
            h = F.linear(self._silu_mul(F.linear(h, lw["gate_up"])), lw["down"])
        h, _ = self._rms(h, self.final_norm, residual)
        if context.is_prefill:                           # only the last token of each prompt
            h = h[context.last_token_indices.long()]     # (models/qwen3.py:472-491)
        return F.linear(h, self.embed)                   # logits [T or batch, vocab]

    # -- one decode step ------------------------------------------------------
    def make_inputs(self, last_tokens, seq_lens, block_tables):
        ids, pos, ctx, slots, bt = prepare_decode(last_tokens, seq_lens, block_tables,
                                                  self.cfg.block_size)
        d = self.device
        t = lambda a: torch.from_numpy(a).to(d)
        # the lengths are host integers here, as in the reference's filler: pick the split
        split = choose_split(ctx, self.cfg.num_kv_heads, self.cfg.num_heads)
        return t(ids), t(pos), create_decode_context(t(ctx), t(slots), t(bt), split)

    def make_prefill_inputs(self, token_lists, block_tables, num_cached_tokens=None):
        """Prefill inputs; with ``num_cached_tokens`` the context carries the block
        tables (as the reference's does when a prefix is cached,
        ``engine/model_runner.py:309-312``) and attention reads keys and values
        from the paged cache."""
        ids, pos, cu_q, cu_k, slots, max_q, max_k = prepare_prefill(
            token_lists, block_tables, self.cfg.block_size, num_cached_tokens)
        d = self.device
        t = lambda a: torch.from_numpy(a).to(d)
        bt = t(prepare_block_tables(block_tables)) if num_cached_tokens is not None else None
        return t(ids), t(pos), create_prefill_context(t(cu_q), t(cu_k), max_q, max_k, t(slots),
                                                      block_tables=bt)

    def step(self, input_ids, positions, context):
        """Eager decode step: logits -> greedy token ids [batch] int64."""
        return self.forward(input_ids, positions, context).argmax(dim=-1)

    def _eager_workspace(self, context):
        """The split workspace of the eager steps (one stream), grown on demand."""
        batch, max_blocks = context.block_tables.shape
        key = (batch, max_blocks, int(context.decode_split))
        if key not in self._eager_ws_shapes:
            ws = self._new_workspace(*key)
            if self._eager_ws is None or ws.buffer.numel() > self._eager_ws.buffer.numel():
                self._eager_ws = ws
            self._eager_ws_shapes.add(key)
        return self._eager_ws

    def _new_workspace(self, batch, max_blocks, decode_split):
        """A split workspace for all layers of one step (they run one after the
        other on one stream), large enough for the balanced split and for the
        split the context asks for; its counters are zero from the start."""
        c = self.cfg
        with torch.cuda.device(self.device):
            need = max(paged_decode_workspace_bytes(batch, c.num_heads, c.head_dim, max_blocks,
                                                    c.block_size, c.num_kv_heads, chunk)
                       for chunk in {0, int(decode_split)})
        return DecodeWorkspace(need, self.device)

    def _capture(self, input_ids, positions, context, body, warmups):
        """Record ``body()`` into a HIP graph.  The graph gets a split workspace of
        its own, which stays alive with the returned closure and is never handed
        to an eager call: a replay can then rely on counters that nothing but
        its own launches has touched, whatever eager steps (of any batch size)
        or further captures run in between."""
        batch, max_blocks = context.block_tables.shape
        graph_ws = self._new_workspace(batch, max_blocks, context.decode_split)
        eager_ws = [a.workspace for a in self.attn]
        for a in self.attn:
            a.workspace = graph_ws
        try:
            # warm every library handle on a side stream; a warm-up step writes the
            # K/V rows of the current step, which the captured step rewrites with
            # the same values, and does not touch the metadata
            s = torch.cuda.Stream(self.device)
            s.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(s):
                for _ in range(warmups):
                    self.step(input_ids, positions, context)
            torch.cuda.current_stream(self.device).wait_stream(s)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = body()
        finally:
            for a, ws in zip(self.attn, eager_ws):
                a.workspace = ws
        self._graph = graph

        def replay():
            graph.replay()
            return out
        replay.workspace = graph_ws      # keeps it alive; also lets a caller check() it
        return replay

    def capture(self, input_ids, positions, context):
        """Capture the whole step in one HIP graph over static input buffers;
        returns ``replay() -> token ids`` (the inputs may be updated in place
        between replays)."""
        return self._capture(input_ids, positions, context,
                             lambda: self.step(input_ids, positions, context), 2)

    def capture_generation(self, input_ids, positions, context):
        """Capture step + metadata advance in one HIP graph: every replay decodes
        one token per sequence and leaves ``input_ids / positions / context``
        ready for the next replay, with nothing but block-table maintenance left
        to the host.  Returns ``replay() -> token ids of that step``."""
        def body():
            out = self.step(input_ids, positions, context)
            advance_decode(out, input_ids, positions, context, self.cfg.block_size)
            return out
        return self._capture(input_ids, positions, context, body, 1)
