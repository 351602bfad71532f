"""Paged decode attention entry point.

Host-side mirror of ``paged_attention`` (``layers/pallas_attention.py:465-507``
of the reference): same positional contract
``(q, k_cache, v_cache, block_tables, context_lens, scale, block_size)`` and the
same result shape/dtype, with one dispatch target only: the HIP split-K kernel
behind ``nvj_paged_decode_launch``.  Tensors are device memory handles
(``torch`` on ROCm); all arithmetic happens in the HIP library.
"""
from __future__ import annotations

import torch

from .. import _lib

__all__ = ["paged_attention", "paged_decode_workspace_bytes", "default_chunk", "WHOLE_SEQUENCE",
           "choose_split", "DecodeWorkspace"]

WHOLE_SEQUENCE = _lib.NVJ_CHUNK_WHOLE_SEQUENCE


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


_CACHE_DTYPE_CODE = {torch.bfloat16: _lib.NVJ_DTYPE_BF16, torch.float16: _lib.NVJ_DTYPE_F16}


def _check_device_tensor(t: torch.Tensor, name: str, dtype, ndim: int) -> None:
    """``dtype`` None: bf16 or float16 (the cache dtypes)."""
    _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
    _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                        "the paged-decode path has no CPU implementation")
    if dtype is None:
        _require(t.dtype in _CACHE_DTYPE_CODE, f"{name} must be bfloat16 or float16, got {t.dtype}")
    else:
        _require(t.dtype == dtype, f"{name} must be {dtype}, got {t.dtype}")
    _require(t.dim() == ndim, f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")
    _require(t.is_contiguous(), f"{name} must be contiguous")


def default_chunk(batch: int, num_kv_heads: int, max_blocks: int, block_size: int) -> int:
    """Fixed chunk (positions per workgroup) the library recommends when a
    fixed split is wanted; ``chunk=0`` itself selects the balanced split."""
    return int(_lib.load().nvj_paged_decode_default_chunk(batch, num_kv_heads,
                                                          max_blocks, block_size))


def paged_decode_workspace_bytes(batch: int, num_heads: int, head_dim: int,
                                 max_blocks: int, block_size: int, num_kv_heads: int,
                                 chunk: int = 0) -> int:
    """Bytes of split-K workspace one call needs."""
    return int(_lib.load().nvj_paged_decode_workspace_bytes(
        batch, num_heads, head_dim, max_blocks, block_size, num_kv_heads, chunk))


class DecodeWorkspace:
    """Split workspace kept across the decode calls of ONE stream.

    The balanced split (``chunk=0``) merges the partials of a shared row inside
    its one launch, by way of counters that must be zero when a launch starts
    and are zero again when it ends.  Here the counters live in a buffer of
    their own, zeroed when it is created and apart from the partials, so calls
    of any shapes can share one ``DecodeWorkspace`` and each is a single kernel
    launch (``nvj_paged_decode_launch_counters``); a plain tensor (contents
    unknown) costs a small clearing launch in front of every call.  Calls that
    may overlap in time (different streams, a captured graph and eager calls)
    need a workspace each."""

    COUNTER_BYTES = 64 << 10

    def __init__(self, nbytes: int, device, counter_bytes: int = COUNTER_BYTES):
        self.buffer = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)
        self.counters = torch.zeros(max(int(counter_bytes), 256) // 4, dtype=torch.int32,
                                    device=device)
        self._clear_next = False

    @classmethod
    def for_shape(cls, batch: int, num_heads: int, head_dim: int, max_blocks: int,
                  block_size: int, num_kv_heads: int, device, chunk: int = 0):
        with torch.cuda.device(device):   # the size follows the device's CU count
            need = paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks,
                                                block_size, num_kv_heads, chunk)
            counters = int(_lib.load().nvj_paged_decode_counter_bytes(batch, num_heads,
                                                                      num_kv_heads))
        return cls(need, device, max(counters, cls.COUNTER_BYTES))

    def _counters_for(self, nbytes: int) -> torch.Tensor:
        if nbytes > self.counters.numel() * 4:
            self.counters = torch.zeros(-(-nbytes // 256) * 64, dtype=torch.int32,
                                        device=self.counters.device)
        return self.counters

    def check(self) -> bool:
        """Synchronises, then reads the stale flag of the counters: False when a
        launch since the last check found a counter that did not start at zero
        (an earlier launch cut short, two launches overlapping on this
        workspace) and so lost rows of its output.  The counters are then
        cleared in front of the next call."""
        ok = int(self.counters[0].item()) == 0
        if not ok:
            self._clear_next = True
        return ok


def _compute_units(device=None) -> int:
    """Compute units of a GPU (256 on an MI355X), asked once per device; 256 where
    no GPU is visible (planning on a host without one)."""
    if not torch.cuda.is_available():
        return 256
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    n = _CU_COUNT.get(index)
    if n is None:
        n = _CU_COUNT[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return n


_CU_COUNT: dict = {}


def choose_split(context_lens_host, num_kv_heads: int, num_heads: int | None = None,
                 device=None) -> int:
    """``chunk`` for a batch whose lengths the host knows (the reference's filler
    builds ``context_lens`` from Python ints, ``engine/model_runner.py:334-376``):
    ``WHOLE_SEQUENCE`` when the longest sequence is within 10 % of the mean and
    the workgroups of that mode fill whole rounds of the GPU's compute units to at
    least 95 % (one 8-wave workgroup is resident per CU), else 0 (balanced split,
    which is never more than a few percent behind and right for any batch)."""
    lens = [int(n) for n in context_lens_host]
    if not lens:
        return 0
    mean = sum(lens) / len(lens)
    if mean <= 0 or max(lens) > 1.1 * mean:
        return 0
    cus = _compute_units(device)
    count = lambda: int(_lib.load().nvj_paged_decode_whole_sequence_workgroups(
        len(lens), num_kv_heads if num_heads is None else num_heads, num_kv_heads))
    if device is None:
        wgs = count()
    else:
        with torch.cuda.device(device):     # the count follows the device's compute units
            wgs = count()
    rounds = -(-wgs // cus)
    return WHOLE_SEQUENCE if wgs > 0 and wgs >= 0.95 * rounds * cus else 0


def _raw_stream(device_index: int) -> int:
    """The current HIP stream of a device as an integer handle."""
    try:
        return torch._C._cuda_getCurrentRawStream(device_index)
    except AttributeError:      # a torch without the raw accessor
        return torch.cuda.current_stream(device_index).cuda_stream


# What a call signature (shapes, dtypes, devices, page size, split) was validated to:
# the integer arguments of the launch and the workspace it needs.  Validation costs
# several times the launch itself, so it runs once per signature.
_decode_plans: dict = {}


def _plan_decode(lib, q, k_cache, v_cache, block_tables, context_lens, block_size, chunk):
    _check_device_tensor(q, "q", None, 3)
    _check_device_tensor(k_cache, "k_cache", q.dtype, 4)
    _check_device_tensor(v_cache, "v_cache", q.dtype, 4)
    _check_device_tensor(block_tables, "block_tables", torch.int32, 2)
    _check_device_tensor(context_lens, "context_lens", torch.int32, 1)
    batch, num_heads, head_dim = q.shape
    num_blocks, bs, num_kv_heads, d2 = k_cache.shape
    _require(v_cache.shape == k_cache.shape, "k_cache and v_cache shapes differ")
    _require(d2 == head_dim, f"head_dim mismatch: q {head_dim}, cache {d2}")
    _require(int(block_size) == bs, f"block_size {block_size} != k_cache.shape[1] {bs}")
    _require(block_tables.shape[0] == batch, "block_tables batch mismatch")
    _require(context_lens.shape[0] == batch, "context_lens batch mismatch")
    _require(num_heads % num_kv_heads == 0, "num_heads must be a multiple of num_kv_heads")
    max_blocks = block_tables.shape[1]
    dev = q.device
    for name, t in (("k_cache", k_cache), ("v_cache", v_cache),
                    ("block_tables", block_tables), ("context_lens", context_lens)):
        _require(t.device == dev, f"{name} is on {t.device}, q on {dev}")
    need = counters = 0
    if batch and max_blocks:
        with torch.cuda.device(dev):      # the balanced sizes follow the device's CU count
            need = int(lib.nvj_paged_decode_workspace_bytes(batch, num_heads, head_dim,
                                                            max_blocks, bs, num_kv_heads, chunk))
            if chunk == 0:
                counters = int(lib.nvj_paged_decode_counter_bytes(batch, num_heads, num_kv_heads))
    return (dev.index, batch, num_heads, num_kv_heads, head_dim, bs, max_blocks, num_blocks, need,
            counters, _CACHE_DTYPE_CODE[q.dtype])


def paged_attention(q, k_cache, v_cache, block_tables, context_lens, scale, block_size,
                    *, chunk: int = 0, out: torch.Tensor | None = None,
                    workspace: "torch.Tensor | DecodeWorkspace | None" = None,
                    phases: int = _lib.NVJ_PHASE_SPLITK | _lib.NVJ_PHASE_COMBINE) -> torch.Tensor:
    """Decode attention over a block-paged KV cache.

    q            [batch, num_heads, head_dim]                          bf16 or float16
    k_cache      [num_blocks, block_size, num_kv_heads, head_dim]      same dtype
    v_cache      same shape
    block_tables [batch, max_blocks] int32 (padding entries are never read)
    context_lens [batch] int32
    scale        softmax scale (Python float)
    block_size   positions per page; must equal ``k_cache.shape[1]``

    Returns [batch, num_heads, head_dim] in q's dtype.  ``chunk`` (0 = balanced split
    derived from ``context_lens`` on the device, one launch; > 0 = that many
    positions per workgroup, multiple of 32, plus a combine launch;
    ``WHOLE_SEQUENCE`` = each sequence finished inside one workgroup, no workspace,
    for batches of similar lengths), ``out`` and ``workspace`` (a
    ``DecodeWorkspace``, or a uint8 tensor of at least
    ``paged_decode_workspace_bytes`` bytes whose counters are then cleared by an
    extra small launch) are optional tuning/reuse knobs the reference does not
    have; ``phases`` selects the launches (timing aid).
    """
    lib = _lib.load()
    try:
        sig = (q.shape, q.dtype, q.device, k_cache.shape, k_cache.dtype, k_cache.device,
               v_cache.shape, v_cache.dtype, v_cache.device, block_tables.shape,
               block_tables.dtype, block_tables.device, context_lens.shape, context_lens.dtype,
               context_lens.device, int(block_size), int(chunk))
    except AttributeError as e:
        raise ValueError("paged_attention takes torch tensors") from e
    plan = _decode_plans.get(sig)
    if plan is None:
        plan = _plan_decode(lib, q, k_cache, v_cache, block_tables, context_lens, block_size,
                            chunk)
        if len(_decode_plans) < 256:
            _decode_plans[sig] = plan
    # layout is a property of the tensor, not of the signature
    _require(q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()
             and block_tables.is_contiguous() and context_lens.is_contiguous(),
             "q, k_cache, v_cache, block_tables and context_lens must be contiguous")
    (dev_index, batch, num_heads, num_kv_heads, head_dim, bs, max_blocks, num_blocks, need,
     counter_bytes, dtype_code) = plan
    dev = q.device

    if out is None:
        out = torch.empty_like(q)
    else:
        _require(isinstance(out, torch.Tensor) and out.dtype == q.dtype and out.shape == q.shape
                 and out.device == dev and out.is_contiguous(),
                 "out must be a contiguous tensor matching q")
    phases = int(phases)
    counters = None
    if isinstance(workspace, DecodeWorkspace):
        if chunk == 0 and need:
            counters = workspace._counters_for(counter_bytes)
            if workspace._clear_next:
                phases |= _lib.NVJ_PHASE_CLEAR_COUNTERS
                workspace._clear_next = False
            need -= counter_bytes           # the buffer holds the partials only
        workspace = workspace.buffer
    else:
        phases |= _lib.NVJ_PHASE_CLEAR_COUNTERS
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    else:
        _require(workspace.is_cuda and workspace.device == dev and workspace.is_contiguous(),
                 "workspace must be a contiguous tensor on q's device")
    ws_bytes = workspace.numel() * workspace.element_size()
    _require(ws_bytes >= need, f"workspace too small: need {need} bytes")

    def launch():
        if counters is not None:
            _require(counters.device == dev, "the workspace's counters are on another device")
            return lib.nvj_paged_decode_launch_counters(
                _raw_stream(dev_index), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                block_tables.data_ptr(), context_lens.data_ptr(), out.data_ptr(),
                workspace.data_ptr(), ws_bytes, counters.data_ptr(), counters.numel() * 4,
                batch, num_heads, num_kv_heads, head_dim, bs, max_blocks, num_blocks,
                float(scale), dtype_code, phases)
        return lib.nvj_paged_decode_launch_phases(
            _raw_stream(dev_index), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            block_tables.data_ptr(), context_lens.data_ptr(), out.data_ptr(),
            workspace.data_ptr(), ws_bytes, batch, num_heads, num_kv_heads, head_dim, bs,
            max_blocks, num_blocks, float(scale), int(chunk), dtype_code, phases)

    if torch.cuda.current_device() == dev_index:
        code = launch()
    else:
        with torch.cuda.device(dev_index):
            code = launch()
    if code != 0:
        _lib.check(code, "nvj_paged_decode_launch_counters" if counters is not None
                   else "nvj_paged_decode_launch_phases")
    return out
