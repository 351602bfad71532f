"""ctypes binding of oracle/paged_oracle.c (TEST INFRASTRUCTURE ONLY).

Used by tests and by the cpu_baseline leg of bench.py; never by the product
package.  The shared object is built by ``make -C oracle`` (``build()`` of
``__graft_entry__`` does it)."""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libpaged_oracle.so")
_lib = None


def available() -> bool:
    return os.path.exists(_SO)


def _load():
    global _lib
    if _lib is None:
        if not available():
            raise RuntimeError(f"{_SO} missing: run `make -C oracle`")
        lib = ctypes.CDLL(_SO)
        lib.oracle_num_threads.restype = ctypes.c_int
        lib.oracle_paged_decode.restype = ctypes.c_int
        lib.oracle_paged_decode.argtypes = ([ctypes.c_void_p] * 7 + [ctypes.c_int] * 7 +
                                            [ctypes.c_float, ctypes.c_int])
        lib.oracle_store_kvcache.restype = None
        lib.oracle_store_kvcache.argtypes = ([ctypes.c_void_p] * 5 + [ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int])
        _lib = lib
    return _lib


def num_threads() -> int:
    return int(_load().oracle_num_threads())


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def paged_decode(q, k_cache, v_cache, block_tables, context_lens, scale, block_size,
                 return_f32=False, dtype="bf16"):
    """Same contract as ``paged_decode_attention_per_seq_ref``."""
    assert dtype in ("bf16", "f16")
    lib = _load()
    q = np.ascontiguousarray(q, np.uint16)
    kc = np.ascontiguousarray(k_cache, np.uint16)
    vc = np.ascontiguousarray(v_cache, np.uint16)
    bt = np.ascontiguousarray(block_tables, np.int32)
    ctx = np.ascontiguousarray(context_lens, np.int32)
    B, Hq, D = q.shape
    NB, bs, Hkv, _ = kc.shape
    assert bs == block_size
    MB = bt.shape[1]
    of = np.empty((B, Hq, D), np.float32)
    ob = np.empty((B, Hq, D), np.uint16)
    rc = lib.oracle_paged_decode(_ptr(q), _ptr(kc), _ptr(vc), _ptr(bt), _ptr(ctx), _ptr(of),
                                 _ptr(ob), B, Hq, Hkv, D, bs, MB, NB, float(scale),
                                 int(dtype == "f16"))
    if rc != 0:
        raise RuntimeError("oracle_paged_decode: unsupported sizes")
    return of if return_f32 else ob


def store_kvcache(key, value, k_cache, v_cache, slot_mapping, negative_slots="reference",
                  dtype="bf16"):
    """Same contract as ``store_kv_to_cache_ref`` (returns new caches)."""
    lib = _load()
    key = np.ascontiguousarray(key)
    value = np.ascontiguousarray(value)
    kc = np.array(k_cache, np.uint16, copy=True)
    vc = np.array(v_cache, np.uint16, copy=True)
    slots = np.ascontiguousarray(slot_mapping, np.int32)
    T = key.shape[0]
    row = int(np.prod(key.shape[1:]))
    lib.oracle_store_kvcache(_ptr(key), _ptr(value), _ptr(kc), _ptr(vc), _ptr(slots), T, row,
                             kc.shape[0], int(key.dtype == np.float32),
                             int(value.dtype == np.float32),
                             1 if negative_slots == "skip" else 0, int(dtype == "f16"))
    return kc, vc
