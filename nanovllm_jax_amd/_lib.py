"""ctypes binding of the C ABI declared in ``include/nvj_paged_attn.h``.

The library is loaded from ``nanovllm_jax_amd/_native/``; it is never built
here.  A missing library is an error: there is no CPU or PyTorch fallback for
this path.
"""
from __future__ import annotations

import ctypes
import os
import threading

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_native",
                         "libnvj_paged_attn.so")

NVJ_ABI_VERSION = 3
NVJ_DTYPE_BF16 = 0
NVJ_DTYPE_F32 = 1
NVJ_DTYPE_F16 = 2

# every symbol include/nvj_paged_attn.h declares: name -> (restype, argtypes)
_c = ctypes
SYMBOLS = {
    "nvj_error_string": (_c.c_char_p, [_c.c_int]),
    "nvj_abi_version": (_c.c_int, []),
    "nvj_store_kvcache_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_int32, _c.c_int32, _c.c_int32]),
    "nvj_paged_decode_default_chunk": (_c.c_int32, [_c.c_int32] * 4),
    "nvj_paged_decode_whole_sequence_workgroups": (_c.c_int32, [_c.c_int32] * 3),
    "nvj_paged_decode_workspace_bytes": (_c.c_size_t, [_c.c_int32] * 7),
    "nvj_paged_decode_counter_bytes": (_c.c_size_t, [_c.c_int32] * 3),
    "nvj_paged_decode_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_void_p, _c.c_void_p, _c.c_size_t,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32,
        _c.c_int32, _c.c_float, _c.c_int32, _c.c_int32]),
    "nvj_paged_decode_launch_phases": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_void_p, _c.c_void_p, _c.c_size_t,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32,
        _c.c_int32, _c.c_float, _c.c_int32, _c.c_int32, _c.c_uint32]),
    "nvj_paged_decode_launch_counters": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_void_p, _c.c_void_p, _c.c_size_t, _c.c_void_p, _c.c_size_t,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32,
        _c.c_int32, _c.c_float, _c.c_int32, _c.c_uint32]),
    "nvj_paged_decode_counters_reset": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "nvj_paged_decode_library_counters": (_c.c_int, [_c.POINTER(_c.c_void_p),
                                                     _c.POINTER(_c.c_size_t)]),
    "nvj_paged_decode_static_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_void_p,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32,
        _c.c_int32, _c.c_float, _c.c_int32]),
    "nvj_qk_norm_rope_store_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_void_p,
        _c.c_void_p, _c.c_float, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64]),
    "nvj_advance_decode_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_void_p, _c.c_int32, _c.c_int32, _c.c_int32]),
    "nvj_prefill_attention_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
        _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int32, _c.c_float, _c.c_int32]),
    "nvj_paged_prefill_attention_launch": (_c.c_int, [
        _c.c_void_p] * 8 + [_c.c_int32] * 8 + [_c.c_float, _c.c_int32]),
    "nvj_add_rms_norm_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_float, _c.c_void_p, _c.c_void_p,
        _c.c_int32, _c.c_int32]),
    "nvj_silu_and_mul_launch": (_c.c_int, [
        _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int32, _c.c_int32]),
}
NVJ_CHUNK_WHOLE_SEQUENCE = -1
NVJ_STATIC_SCRATCH_BYTES = 16 << 20
NVJ_ERR_SCRATCH_LIMIT = -7
NVJ_ERR_ALIGNMENT = -8
NVJ_PHASE_SPLITK = 1
NVJ_PHASE_COMBINE = 2
NVJ_PHASE_VALU_PRODUCTS = 4
NVJ_PHASE_CLEAR_COUNTERS = 8
NVJ_PHASE_LOADS_ONLY = 16
NVJ_PHASE_SHARED_ROWS = 32

_lock = threading.Lock()
_lib = None


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, stale or returned an error code."""


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load the shared library once and type every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise NativeLibraryError(
                f"{_LIB_PATH} not found: build it with "
                "`python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no fallback for the paged-decode path)")
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as e:
                raise NativeLibraryError(f"{_LIB_PATH} does not export {name}") from e
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.nvj_abi_version()
        if got != NVJ_ABI_VERSION:
            raise NativeLibraryError(
                f"{_LIB_PATH} has ABI version {got}, expected {NVJ_ABI_VERSION}: rebuild")
        _lib = lib
        return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().nvj_error_string(code).decode()
        raise NativeLibraryError(f"{what} failed: {msg} (code {code})")
