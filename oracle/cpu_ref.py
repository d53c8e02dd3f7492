"""ctypes binding of ``cpu_ref.c`` (TEST INFRASTRUCTURE ONLY).

The C file restates the reference's exact-scan CPU path
(diffcache_cpu/src/nsw.rs:592-630, lib.rs:373-404); this module loads the
shared object built by ``oracle/Makefile`` and exposes it on numpy arrays.
Used by tests, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libdc_cpu_ref.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.dcref_dot_bf16.restype = C.c_float
        _lib.dcref_distance_qk.restype = C.c_float
        _lib.dcref_pack.restype = C.c_uint64
        _lib.dcref_pack.argtypes = [C.c_float, C.c_uint32]
        _lib.dcref_dualheap_new.restype = C.c_void_p
        _lib.dcref_dualheap_new.argtypes = [C.c_size_t, C.c_size_t]
        _lib.dcref_dualheap_free.argtypes = [C.c_void_p]
        _lib.dcref_dualheap_push.argtypes = [C.c_void_p, C.c_int64]
        _lib.dcref_dualheap_len.restype = C.c_size_t
        _lib.dcref_dualheap_len.argtypes = [C.c_void_p]
        _lib.dcref_dualheap_dth_min.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
        _lib.dcref_dualheap_kept_max.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
        _lib.dcref_dualheap_sorted.restype = C.c_size_t
        _lib.dcref_dualheap_sorted.argtypes = [C.c_void_p, C.c_void_p]
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def dot_bf16(a_u16, b_u16) -> float:
    a, b = _c(a_u16, np.uint16), _c(b_u16, np.uint16)
    return float(lib().dcref_dot_bf16(_p(a), _p(b), C.c_int(a.size)))


def pack(dist: float, node: int) -> int:
    return int(lib().dcref_pack(C.c_float(dist), C.c_uint32(node)))


def search_bruteforce(keys_u16, vals_u16, query_u16, ef: int, pre_scores=None):
    """One unit.  Returns (out_keys, out_vals, ids, scores)."""
    keys, vals, q = _c(keys_u16, np.uint16), _c(vals_u16, np.uint16), _c(query_u16, np.uint16)
    n, dim = keys.shape
    efc = max(min(ef, n), 0)
    ok = np.zeros((efc, dim), np.uint16)
    ov = np.zeros((efc, dim), np.uint16)
    ids = np.zeros((efc,), np.uint32)
    sc = np.zeros((n,), np.float32)
    pre = None if pre_scores is None else _c(pre_scores, np.float32)
    got = lib().dcref_search_bruteforce(_p(keys), _p(vals), C.c_int(n), C.c_int(dim), _p(q),
                                        C.c_int(ef), _p(ok), _p(ov), _p(ids), _p(sc), _p(pre))
    assert got == efc
    return ok, ov, ids, sc


def query(keys_u16, vals_u16, queries_u16, ef: int, ctx_len: Optional[int] = None,
          n_threads: int = 1):
    """keys/vals (b, Hkv, n_max, hd), queries (b, Hkv, hd).
    Returns (out_keys, out_vals (b,Hkv,ef',hd), ids (b,Hkv,ef'))."""
    keys, vals, q = _c(keys_u16, np.uint16), _c(vals_u16, np.uint16), _c(queries_u16, np.uint16)
    b, h, n_max, dim = keys.shape
    ctx = n_max if ctx_len is None else ctx_len
    efc = min(ef, ctx)
    ok = np.zeros((b, h, efc, dim), np.uint16)
    ov = np.zeros((b, h, efc, dim), np.uint16)
    ids = np.zeros((b, h, efc), np.uint32)
    got = lib().dcref_query(_p(keys), _p(vals), _p(q), _p(ok), _p(ov), _p(ids), C.c_int(b * h),
                            C.c_int(ctx), C.c_int(n_max), C.c_int(dim), C.c_int(ef),
                            C.c_int(n_threads))
    assert got == efc
    return ok, ov, ids


def group_mean(q_u16, group: int):
    q = _c(q_u16, np.uint16)
    dim = q.shape[-1]
    n_units = q.size // (group * dim)
    out = np.zeros((n_units, dim), np.uint16)
    lib().dcref_group_mean(_p(q), _p(out), C.c_int(n_units), C.c_int(group), C.c_int(dim))
    return out


def sparse_attention(q_u16, k_rows_u16, v_rows_u16, scale: float):
    q, k, v = _c(q_u16, np.uint16), _c(k_rows_u16, np.uint16), _c(v_rows_u16, np.uint16)
    g, dim = q.shape
    out = np.zeros((g, dim), np.uint16)
    lib().dcref_sparse_attention(_p(q), _p(k), _p(v), C.c_int(k.shape[0]), C.c_int(g),
                                 C.c_int(dim), C.c_float(scale), _p(out))
    return out


def decode_layer(q_u16, k_u16, v_u16, budget: int, prefix: int, suffix: int,
                 n_ctx: Optional[int] = None, new_k_u16=None, new_v_u16=None,
                 n_threads: int = 1, want_ids: bool = True):
    """q (n_units, G, hd); k, v (n_units, n_max, hd); new_k/new_v (n_units, hd).
    Returns (out (n_units, G, hd) u16, ids (n_units, budget) u32 or None)."""
    q, k, v = _c(q_u16, np.uint16), _c(k_u16, np.uint16), _c(v_u16, np.uint16)
    n_units, g, dim = q.shape
    n_max = k.shape[1]
    ctx = n_max if n_ctx is None else n_ctx
    nk = None if new_k_u16 is None else _c(new_k_u16, np.uint16)
    nv = None if new_v_u16 is None else _c(new_v_u16, np.uint16)
    out = np.zeros((n_units, g, dim), np.uint16)
    ids = np.zeros((n_units, budget), np.uint32) if want_ids else None
    lib().dcref_decode_layer(_p(q), _p(k), _p(v), _p(nk), _p(nv), _p(out), _p(ids),
                             C.c_int(n_units), C.c_int(g), C.c_int(dim), C.c_int(ctx),
                             C.c_int(n_max), C.c_int(budget), C.c_int(prefix), C.c_int(suffix),
                             C.c_int(n_threads))
    return out, ids


class DualHeap:
    def __init__(self, d: int, cap: int) -> None:
        self._h = lib().dcref_dualheap_new(d, cap)
        if not self._h:
            raise AssertionError("cap must be >= d >= 1")
        self.d, self.cap = d, cap

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dcref_dualheap_free(self._h)
            self._h = None

    def push(self, x: int) -> None:
        lib().dcref_dualheap_push(self._h, int(x))

    def __len__(self) -> int:
        return int(lib().dcref_dualheap_len(self._h))

    def dth_min(self):
        v = C.c_int64()
        return v.value if lib().dcref_dualheap_dth_min(self._h, C.byref(v)) else None

    def kept_max(self):
        v = C.c_int64()
        return v.value if lib().dcref_dualheap_kept_max(self._h, C.byref(v)) else None

    def into_sorted_vec(self):
        out = np.zeros((max(len(self), 1),), np.int64)
        n = lib().dcref_dualheap_sorted(self._h, _p(out))
        return out[:n].tolist()
