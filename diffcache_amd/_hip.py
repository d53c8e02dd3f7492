"""ctypes binding of ``libdiffcache_hip.so`` and tensor-level wrappers.

The library is the product; there is no CPU or PyTorch fallback.  Importing
this module without the built library raises, and every wrapper raises if a
tensor is not on a GPU.  PyTorch is used only for device memory and streams.
"""
from __future__ import annotations

import ctypes as C
import math
import os
from typing import Optional, Tuple

import torch

MODE_IP = 0
MODE_REF_DIST = 1
ONE_KERNEL_AUTO, ONE_KERNEL_EXCLUSIVE, ONE_KERNEL_NEVER = 0, 1, -1
ORDER_ANY = 0
ORDER_BEST = 1
ORDER_INDEX = 2
HIST_BINS = 1024

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdiffcache_hip.so")

# every symbol include/diffcache_hip.h declares
SYMBOLS = (
    "dc_version", "dc_last_error", "dc_group_mean_bf16", "dc_score_bf16",
    "dc_topk_workspace_bytes", "dc_topk_select", "dc_gather_rows_bf16",
    "dc_attn_workspace_bytes", "dc_gather_attn_bf16", "dc_gather_attn_static_bf16", "dc_append_kv_bf16",
    "dc_step_advance", "dc_step_state_advance", "dc_step_state_rollover", "dc_ingest_kv_bf16", "dc_layer_workspace_bytes", "dc_decode_layer",
    "dc_decode_layer_status", "dc_set_wait_limit", "dc_decode_layer_route", "dc_last_route",
    "dc_decode_layer_errors", "dc_one_kernel_guard",
    "dc_pq_build_lut", "dc_pq_adc_scan", "dc_score_gathered_bf16", "dc_compose_idx",
    "dc_score_select_workspace_bytes", "dc_select_state_init", "dc_score_prune_bf16",
    "dc_sparse_select", "dc_score_select_bf16",
    "dc_sketch_build_bf16", "dc_sketch_select_workspace_bytes", "dc_sketch_select_state_init",
    "dc_score_select_sketch_bf16", "dc_kcheck_f32",
    "dc_pq_search_workspace_bytes", "dc_pq_search_bf16",
    "dc_data_layer_create", "dc_data_layer_destroy", "dc_data_layer_ctx_len", "dc_data_layer_sizes",
    "dc_data_layer_bind", "dc_data_layer_prefill", "dc_data_layer_insert", "dc_data_layer_query",
)


class LayerArgs(C.Structure):
    """struct dc_layer_args of include/diffcache_hip.h"""
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("new_k", C.c_void_p), ("new_v", C.c_void_p), ("out", C.c_void_p),
        ("lse", C.c_void_p), ("scores", C.c_void_p), ("idx_out", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("kv_batch_stride", C.c_int64), ("kv_head_stride", C.c_int64), ("kv_row_stride", C.c_int64),
        ("scores_unit_stride", C.c_int64), ("idx_unit_stride", C.c_int64),
        ("recent_lo", C.c_int64),
        ("n_b", C.c_int), ("n_h", C.c_int), ("group", C.c_int), ("hd", C.c_int),
        ("n_sink", C.c_int), ("n_recent", C.c_int), ("budget", C.c_int),
        ("mode", C.c_int), ("order", C.c_int), ("scale", C.c_float),
        ("select_state_ready", C.c_int),
        ("ev_scan_begin", C.c_void_p), ("ev_scan_end", C.c_void_p),
        ("sketch_codes", C.c_void_p), ("sketch_scale", C.c_void_p), ("sketch_resid", C.c_void_p),
        ("sketch_batch_stride", C.c_int64), ("sketch_head_stride", C.c_int64),
        ("sketch_row_stride", C.c_int64),
        ("n_recent_dev", C.c_void_p),
        ("one_kernel", C.c_int),
        ("region_hi_dev", C.c_void_p),
    ]


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python diffcache_amd/build.py` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path.")
    lib = C.CDLL(LIB_PATH)
    i, i64, p, sz, f = C.c_int, C.c_int64, C.c_void_p, C.c_size_t, C.c_float
    sigs = {
        "dc_version": (i, []),
        "dc_last_error": (C.c_char_p, []),
        "dc_group_mean_bf16": (i, [p, p, i, i, i, p]),
        "dc_score_bf16": (i, [p, p, p, p, i, i, i, i, i64, i64, i64, i64, i, i, p]),
        "dc_topk_workspace_bytes": (sz, [i, i, i]),
        "dc_topk_select": (i, [p, i64, p, i64, i, i, i, i, i, p, p, sz, p]),
        "dc_gather_rows_bf16": (i, [p, p, p, p, p, i, i, i, i64, i, i64, i64, i64, i64, i64, i64, i64, p]),
        "dc_attn_workspace_bytes": (sz, [i, i, i, i]),
        "dc_gather_attn_bf16": (i, [p, p, p, p, p, p, p, p, i, i, i, i, i, i64, p, i64, i, i64, i, p,
                                    i64, i64, i64, i64, i64, i64, f, p, sz, p]),
        "dc_gather_attn_static_bf16": (i, [p, p, p, p, p, p, p, p, i, i, i, i, i, i64, p, i64, i, i64, i, p,
                                           i64, i64, i64, i64, i64, i64, f, p]),
        "dc_append_kv_bf16": (i, [p, p, p, p, i, i, i, i64, p, i64, i64, i64, i64, p]),
        "dc_step_advance": (i, [p, i, i, p]),
        "dc_step_state_advance": (i, [p, i, i, p]),
        "dc_step_state_rollover": (i, [p, i, i, p]),
        "dc_ingest_kv_bf16": (i, [p, p, i, i, i, i, i64, i64, i64, i64, p]),
        "dc_layer_workspace_bytes": (sz, [i, i, i, i, i, i]),
        "dc_decode_layer": (i, [C.POINTER(LayerArgs), p]),
        "dc_decode_layer_status": (i, [C.POINTER(LayerArgs), p]),
        "dc_set_wait_limit": (None, [i]),
        "dc_decode_layer_route": (i, [C.POINTER(LayerArgs)]),
        "dc_last_route": (i, []),
        "dc_decode_layer_errors": (C.c_uint, []),
        "dc_one_kernel_guard": (i, [i, i, i, i, i]),
        "dc_pq_build_lut": (i, [p, p, p, i, i, i, i, p]),
        "dc_pq_adc_scan": (i, [p, p, p, p, i, i, i, i64, p]),
        "dc_score_gathered_bf16": (i, [p, p, p, p, i, i, i, i64, i, i64, i64, i64, i64, i64, p]),
        "dc_compose_idx": (i, [p, i64, p, i64, p, i64, i, i, p]),
        "dc_pq_search_workspace_bytes": (sz, [i, i, i]),
        "dc_data_layer_create": (i, [C.POINTER(p), i, i, i, i64, i, i]),
        "dc_data_layer_destroy": (None, [p]),
        "dc_data_layer_ctx_len": (i64, [p]),
        "dc_data_layer_sizes": (i, [p, i] + [C.POINTER(sz)] * 5),
        "dc_data_layer_bind": (i, [p, p, p, p, p, p, p, p, sz, i]),
        "dc_data_layer_prefill": (i, [p, p, p, i64, p]),
        "dc_data_layer_insert": (i, [p, p, p, p]),
        "dc_data_layer_query": (i, [p, p, p, i64, p, i, C.POINTER(i), p]),
        "dc_pq_search_bf16": (i, [p, p, p, p, p, i64, i, i, i, i, i, i64, i64, i64, i, i, i, p, sz, p, p, p]),
        "dc_score_select_workspace_bytes": (sz, [i, i, i]),
        "dc_select_state_init": (i, [i, i, i, p, sz, p]),
        "dc_score_prune_bf16": (i, [p, p, i, i, i, i, i64, i64, i64, i, i, i, p, sz, p]),
        "dc_sparse_select": (i, [p, i64, i, i, i, i, i, i, p, sz, p]),
        "dc_score_select_bf16": (i, [p, p, p, i64, i, i, i, i, i64, i64, i64, i, i, i, i, p, sz, p]),
        "dc_sketch_build_bf16": (i, [p, p, p, p, i, i, i, i, i64, i64, i64, i64, i64, i64, i, p]),
        "dc_kcheck_f32": (i, [p, i64, i, i, i, i, C.POINTER(C.c_int), i, f, p, p, p, p]),
        "dc_sketch_select_workspace_bytes": (sz, [i, i, i]),
        "dc_sketch_select_state_init": (i, [i, i, i, p, sz, p]),
        "dc_score_select_sketch_bf16": (i, [p, p, p, p, p, p, i64, i, i, i, i, i64, i64, i64, i64, i64, i64,
                                            i, i, i, i, i, p, sz, p, p, p]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


class DiffCacheError(RuntimeError):
    pass


def _check(rc: int) -> None:
    if rc != 0:
        raise DiffCacheError(f"[{rc}] {lib.dc_last_error().decode()}")


def _dev(t: torch.Tensor, name: str) -> int:
    if not t.is_cuda:
        raise DiffCacheError(f"{name} must live in GPU memory (got {t.device}); there is no CPU path")
    return t.data_ptr()


def _opt(t: Optional[torch.Tensor], name: str):
    return None if t is None else _dev(t, name)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _counter(t: Optional[torch.Tensor]):
    """Device pointer of a one-element int32 step counter, or None."""
    if t is None:
        return None
    if not t.is_cuda or t.dtype != torch.int32 or t.numel() < 1:
        raise DiffCacheError("a step counter must be an int32 tensor in GPU memory")
    return t.data_ptr()


def _store_strides(store: torch.Tensor) -> Tuple[int, int, int]:
    """(batch, head, row) element strides of a (b, h, n, hd) bf16 store."""
    if store.dim() != 4 or store.dtype != torch.bfloat16 or store.stride(3) != 1:
        raise DiffCacheError("a K/V store must be a (b, h, n, hd) bfloat16 tensor with contiguous rows")
    return store.stride(0), store.stride(1), store.stride(2)


def require(cond: bool, msg: str = "") -> None:
    """The reference asserts its invariants (Rust ``assert!`` -> a panic, Python ``assert``).
    Here they guard device memory, so they must survive ``python -O``: same exception type,
    not an ``assert`` statement."""
    if not cond:
        raise AssertionError(msg)


def alloc_workspace(nbytes: int, device) -> torch.Tensor:
    """Zero-filled, 256-byte aligned scratch (the attention counters must start at zero)."""
    return torch.zeros((max(int(nbytes), 256) + 255) // 256 * 256, dtype=torch.uint8, device=device)


# ---------------------------------------------------------------------------
# wrappers
# ---------------------------------------------------------------------------

def group_mean(q: torch.Tensor, group: int, out: Optional[torch.Tensor] = None,
               hd: Optional[int] = None) -> torch.Tensor:
    """q bf16 holding (n_units, group, hd) values in that order -> (n_units, hd) bf16.
    ``hd`` defaults to the last dimension of q."""
    hd = q.shape[-1] if hd is None else hd
    q = q.contiguous()
    n_units = q.numel() // (group * hd)
    if out is None:
        out = torch.empty((n_units, hd), dtype=torch.bfloat16, device=q.device)
    _check(lib.dc_group_mean_bf16(_dev(q, "q"), _dev(out, "out"), n_units, group, hd, _stream()))
    return out


def score(store_k: torch.Tensor, q: torch.Tensor, lo: int, n_rows: int, mode: int = MODE_REF_DIST,
          q_group: int = 1, scores: Optional[torch.Tensor] = None,
          hist: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Scores of rows [lo, lo + n_rows) of every unit.  q: (b*h*q_group*hd) bf16 in
    (b, h, q_group, hd) order.  Returns fp32 (b*h, n_rows)."""
    sb, sh, sr = _store_strides(store_k)
    b, h, n_max, hd = store_k.shape
    if lo < 0 or lo + n_rows > n_max:
        raise DiffCacheError(f"rows [{lo}, {lo + n_rows}) outside the store of {n_max} rows")
    q = q.contiguous()
    if q.dtype != torch.bfloat16 or q.numel() != b * h * q_group * hd:
        raise DiffCacheError("q must be bf16 with b*h*q_group*hd elements")
    if scores is None:
        scores = torch.empty((b * h, n_rows), dtype=torch.float32, device=store_k.device)
    kptr = _dev(store_k, "store_k") + lo * sr * 2
    _check(lib.dc_score_bf16(kptr, _dev(q, "q"), _dev(scores, "scores"), _opt(hist, "hist"), b, h,
                             n_rows, hd, sb, sh, sr, scores.stride(0), q_group, mode, _stream()))
    return scores


def new_hist(n_units: int, device) -> torch.Tensor:
    return torch.zeros((n_units, HIST_BINS), dtype=torch.int32, device=device)


def topk_select(scores: torch.Tensor, k: int, mode: int = MODE_REF_DIST, order: int = ORDER_ANY,
                hist: Optional[torch.Tensor] = None, idx_out: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None, n_rows: Optional[int] = None) -> torch.Tensor:
    """scores (n_units, >= n_rows) fp32 -> int32 ids (n_units, min(k, n_rows))."""
    if scores.dim() != 2 or scores.dtype != torch.float32 or scores.stride(1) != 1:
        raise DiffCacheError("scores must be a (n_units, n_rows) fp32 tensor with contiguous rows")
    n_units = scores.shape[0]
    n_rows = scores.shape[1] if n_rows is None else n_rows
    k_eff = min(k, n_rows)
    if idx_out is None:
        idx_out = torch.empty((n_units, max(k_eff, 1)), dtype=torch.int32, device=scores.device)
    need = lib.dc_topk_workspace_bytes(n_units, n_rows, k)
    if workspace is None:
        workspace = alloc_workspace(need, scores.device)
    _check(lib.dc_topk_select(_dev(scores, "scores"), scores.stride(0), _dev(idx_out, "idx_out"),
                              idx_out.stride(0), n_units, n_rows, k, mode, order, _opt(hist, "hist"),
                              _dev(workspace, "workspace"), workspace.numel(), _stream()))
    return idx_out[:, :k_eff]


def score_select_workspace_bytes(n_units: int, n_rows: int, budget: int) -> int:
    return int(lib.dc_score_select_workspace_bytes(n_units, n_rows, budget))


def _score_select_args(store_k, q, lo, n_rows, q_group):
    sb, sh, sr = _store_strides(store_k)
    b, h, n_max, hd = store_k.shape
    if lo < 0 or lo + n_rows > n_max:
        raise DiffCacheError(f"rows [{lo}, {lo + n_rows}) outside the store of {n_max} rows")
    if q.dtype != torch.bfloat16 or not q.is_contiguous() or q.numel() != b * h * q_group * hd:
        raise DiffCacheError("q must be contiguous bf16 with b*h*q_group*hd elements")
    return _dev(store_k, "store_k") + lo * sr * 2, b, h, hd, sb, sh, sr


def select_state_init(n_units: int, n_rows: int, budget: int, workspace: torch.Tensor) -> None:
    _check(lib.dc_select_state_init(n_units, n_rows, budget, _dev(workspace, "workspace"),
                                    workspace.numel(), _stream()))


def score_prune(store_k: torch.Tensor, q: torch.Tensor, lo: int, n_rows: int, budget: int,
                workspace: torch.Tensor, mode: int = MODE_REF_DIST, q_group: int = 1) -> None:
    kptr, b, h, hd, sb, sh, sr = _score_select_args(store_k, q, lo, n_rows, q_group)
    _check(lib.dc_score_prune_bf16(kptr, _dev(q, "q"), b, h, n_rows, hd, sb, sh, sr, q_group, budget,
                                   mode, _dev(workspace, "workspace"), workspace.numel(), _stream()))


def sparse_select(idx_out: torch.Tensor, n_units: int, n_rows: int, budget: int,
                  workspace: torch.Tensor, mode: int = MODE_REF_DIST, order: int = ORDER_ANY,
                  reinit: bool = False) -> torch.Tensor:
    _check(lib.dc_sparse_select(_dev(idx_out, "idx_out"), idx_out.stride(0), n_units, n_rows, budget,
                                mode, order, int(reinit), _dev(workspace, "workspace"),
                                workspace.numel(), _stream()))
    return idx_out[:, :min(budget, n_rows)]


def score_select(store_k: torch.Tensor, q: torch.Tensor, lo: int, n_rows: int, budget: int,
                 mode: int = MODE_REF_DIST, order: int = ORDER_ANY, q_group: int = 1,
                 idx_out: Optional[torch.Tensor] = None,
                 workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Streaming score + exact top-k (no dense scores).  Returns int32 ids
    (b*h, min(budget, n_rows)) relative to row `lo`."""
    kptr, b, h, hd, sb, sh, sr = _score_select_args(store_k, q, lo, n_rows, q_group)
    k_eff = min(budget, n_rows)
    if idx_out is None:
        idx_out = torch.empty((b * h, max(k_eff, 1)), dtype=torch.int32, device=store_k.device)
    if workspace is None:
        workspace = alloc_workspace(score_select_workspace_bytes(b * h, n_rows, budget), store_k.device)
    _check(lib.dc_score_select_bf16(kptr, _dev(q, "q"), _dev(idx_out, "idx_out"), idx_out.stride(0), b, h,
                                    n_rows, hd, sb, sh, sr, q_group, budget, mode, order,
                                    _dev(workspace, "workspace"), workspace.numel(), _stream()))
    return idx_out[:, :k_eff]


class Sketch:
    """8-bit sketch of a (b, h, n, hd) bf16 key store: ``codes`` (b, h, n, hd) uint8 with
    row r of the sketch describing row r of the store, ``scale`` and ``resid`` (b*h, hd)
    fp32 (see dc_sketch_build_bf16 in the header)."""

    def __init__(self, store_k: torch.Tensor, codes: Optional[torch.Tensor] = None):
        _store_strides(store_k)
        b, h, n, hd = store_k.shape
        self.codes = torch.empty((b, h, n, hd), dtype=torch.uint8, device=store_k.device) \
            if codes is None else codes
        if self.codes.shape != store_k.shape or self.codes.dtype != torch.uint8 or self.codes.stride(3) != 1:
            raise DiffCacheError("sketch codes must be a (b, h, n, hd) uint8 tensor with contiguous rows")
        self.scale = torch.zeros((b * h, hd), dtype=torch.float32, device=store_k.device)
        self.resid = torch.zeros((b * h, hd), dtype=torch.float32, device=store_k.device)

    def build(self, store_k: torch.Tensor, lo: int, n_rows: int, keep_scale: bool = False) -> "Sketch":
        """Sketch rows [lo, lo + n_rows).  keep_scale=False fits the scales to these rows
        (prefill); keep_scale=True keeps them and only raises the residual bounds (append)."""
        sb, sh, sr = _store_strides(store_k)
        b, h, n_max, hd = store_k.shape
        if lo < 0 or lo + n_rows > n_max:
            raise DiffCacheError(f"rows [{lo}, {lo + n_rows}) outside the store of {n_max} rows")
        c = self.codes
        _check(lib.dc_sketch_build_bf16(
            _dev(store_k, "store_k") + lo * sr * 2, _dev(c, "codes") + lo * c.stride(2),
            _dev(self.scale, "scale"), _dev(self.resid, "resid"), b, h, n_rows, hd, sb, sh, sr,
            c.stride(0), c.stride(1), c.stride(2), int(keep_scale), _stream()))
        return self


def sketch_select_workspace_bytes(n_units: int, n_rows: int, budget: int) -> int:
    return int(lib.dc_sketch_select_workspace_bytes(n_units, n_rows, budget))


def score_select_sketch(store_k: torch.Tensor, sketch: Sketch, q: torch.Tensor, lo: int, n_rows: int,
                        budget: int, mode: int = MODE_REF_DIST, order: int = ORDER_ANY, q_group: int = 1,
                        idx_out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                        state_ready: bool = False,
                        scan_events: Optional[Tuple[torch.cuda.Event, torch.cuda.Event]] = None
                        ) -> torch.Tensor:
    """The ids of ``score_select`` (exact top-k of the bf16 keys), found by scanning the
    8-bit sketch and rescoring the rows that can still matter."""
    kptr, b, h, hd, sb, sh, sr = _score_select_args(store_k, q, lo, n_rows, q_group)
    k_eff = min(budget, n_rows)
    if idx_out is None:
        idx_out = torch.empty((b * h, max(k_eff, 1)), dtype=torch.int32, device=store_k.device)
    if workspace is None:
        workspace = alloc_workspace(sketch_select_workspace_bytes(b * h, n_rows, budget), store_k.device)
    c = sketch.codes
    ev0 = ev1 = None
    if scan_events is not None:
        ev0, ev1 = scan_events[0].cuda_event, scan_events[1].cuda_event
    _check(lib.dc_score_select_sketch_bf16(
        kptr, _dev(c, "codes") + lo * c.stride(2), _dev(sketch.scale, "scale"), _dev(sketch.resid, "resid"),
        _dev(q, "q"), _dev(idx_out, "idx_out"), idx_out.stride(0), b, h, n_rows, hd, sb, sh, sr,
        c.stride(0), c.stride(1), c.stride(2), q_group, budget, mode, order, int(state_ready),
        _dev(workspace, "workspace"), workspace.numel(), ev0, ev1, _stream()))
    return idx_out[:, :k_eff]


def gather_rows(store_k: Optional[torch.Tensor], store_v: Optional[torch.Tensor], idx: torch.Tensor,
                out_k: Optional[torch.Tensor], out_v: Optional[torch.Tensor], row_offset: int = 0,
                n_idx: Optional[int] = None) -> None:
    """out[b, h, j, :] = store[b, h, row_offset + idx[b*H + h, j], :] for j < n_idx."""
    ref = store_k if store_k is not None else store_v
    sb, sh, sr = _store_strides(ref)
    b, h, _, hd = ref.shape
    dst = out_k if out_k is not None else out_v
    db, dh, dr = _store_strides(dst)
    n_idx = idx.shape[1] if n_idx is None else n_idx
    require(idx.dim() == 2 and idx.shape[0] == b * h and idx.shape[1] >= n_idx and idx.element_size() == 4,
            "idx must be a 32-bit (bsz * kv_heads, >= n_idx) tensor")
    for o in (out_k, out_v):
        require(o is None or (o.shape[0] == b and o.shape[1] == h and o.shape[2] >= n_idx and o.shape[3] == hd),
                "out_k / out_v must be (bsz, kv_heads, >= n_idx, head_dim)")
    _check(lib.dc_gather_rows_bf16(_opt(store_k, "store_k"), _opt(store_v, "store_v"), _dev(idx, "idx"),
                                   _opt(out_k, "out_k"), _opt(out_v, "out_v"), b, h, n_idx,
                                   idx.stride(0), hd, row_offset, sb, sh, sr, db, dh, dr, _stream()))


def gather_attn(q: torch.Tensor, store_k: torch.Tensor, store_v: torch.Tensor,
                idx: Optional[torch.Tensor], n_idx: int, region_lo: int, n_sink: int, recent_lo: int,
                n_recent: int, new_k: Optional[torch.Tensor] = None,
                new_v: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                workspace: Optional[torch.Tensor] = None,
                n_idx_unit: Optional[torch.Tensor] = None,
                n_recent_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q (b, h*group, hd) bf16 -> out (b, h*group, hd) bf16.  ``n_idx_unit`` (b*h) int32:
    per-unit number of leading ids to attend to (see ``kcheck``).  ``n_recent_dev``: one
    int32 on the device holding the current suffix length (``n_recent`` is then its capacity)."""
    ksb, ksh, ksr = _store_strides(store_k)
    vsb, vsh, vsr = _store_strides(store_v)
    b, h, _, hd = store_k.shape
    q = q.contiguous()
    group = q.numel() // (b * h * hd)
    if out is None:
        out = torch.empty((b, h * group, hd), dtype=torch.bfloat16, device=q.device)
    scale = 1.0 / math.sqrt(hd) if scale is None else scale
    n_total = n_idx + n_sink + n_recent + (1 if new_k is not None else 0)
    need = lib.dc_attn_workspace_bytes(b * h, group, hd, n_total)
    if workspace is None:
        workspace = alloc_workspace(need, q.device)
    if new_k is not None:
        new_k, new_v = new_k.contiguous(), new_v.contiguous()
    _check(lib.dc_gather_attn_bf16(
        _dev(q, "q"), _dev(store_k, "store_k"), _dev(store_v, "store_v"), _opt(idx, "idx"),
        _opt(new_k, "new_k"), _opt(new_v, "new_v"), _dev(out, "out"), _opt(lse, "lse"), b, h, group,
        hd, n_idx, 0 if idx is None else idx.stride(0), _opt(n_idx_unit, "n_idx_unit"), region_lo, n_sink,
        recent_lo, n_recent, _counter(n_recent_dev), ksb, ksh, ksr, vsb, vsh, vsr, scale,
        _dev(workspace, "workspace"), workspace.numel(), _stream()))
    return out


def gather_attn_static(q: torch.Tensor, store_k: torch.Tensor, store_v: torch.Tensor,
                       idx: Optional[torch.Tensor], n_idx: int, region_lo: int, n_sink: int, recent_lo: int,
                       n_recent: int, out: torch.Tensor, new_k: Optional[torch.Tensor] = None,
                       new_v: Optional[torch.Tensor] = None, scale: Optional[float] = None,
                       lse: Optional[torch.Tensor] = None,
                       n_idx_unit: Optional[torch.Tensor] = None,
                       n_recent_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gather_attn`` without a workspace and without any allocation (dc_gather_attn_static_bf16):
    the split partials live in a static device array of the library.  q, new_k, new_v must be
    contiguous and ``out`` is the caller's; sizes beyond the array raise DiffCacheError."""
    ksb, ksh, ksr = _store_strides(store_k)
    vsb, vsh, vsr = _store_strides(store_v)
    b, h, _, hd = store_k.shape
    for t, name in ((q, "q"), (new_k, "new_k"), (new_v, "new_v"), (out, "out")):
        if t is not None and not t.is_contiguous():
            raise DiffCacheError(f"{name} must be contiguous")
    group = q.numel() // (b * h * hd)
    if out.dtype != torch.bfloat16 or out.numel() < q.numel():
        raise DiffCacheError("out must be a bf16 tensor of the size of q")
    scale = 1.0 / math.sqrt(hd) if scale is None else scale
    _check(lib.dc_gather_attn_static_bf16(
        _dev(q, "q"), _dev(store_k, "store_k"), _dev(store_v, "store_v"), _opt(idx, "idx"),
        _opt(new_k, "new_k"), _opt(new_v, "new_v"), _dev(out, "out"), _opt(lse, "lse"), b, h, group,
        hd, n_idx, 0 if idx is None else idx.stride(0), _opt(n_idx_unit, "n_idx_unit"), region_lo, n_sink,
        recent_lo, n_recent, _counter(n_recent_dev), ksb, ksh, ksr, vsb, vsh, vsr, scale, _stream()))
    return out


def kcheck(scores: torch.Tensor, n_sel: int, hd: int, k_check_seq, attn_mass_threshold: float,
           mode: int = MODE_REF_DIST, n_eff: Optional[torch.Tensor] = None, want_stats: bool = False):
    """k-check of nsw.rs:198-296 on the exact, best-first scores (n_units, >= n_sel) fp32 of the
    selected rows: n_eff (n_units) int32 = the first size of ``k_check_seq`` (below n_sel)
    whose top rows already hold ``attn_mass_threshold`` of the estimated softmax mass, else
    n_sel.  With ``want_stats`` also (alpha, mass), each (n_units, len(k_check_seq)) fp32."""
    if scores.dtype != torch.float32 or scores.dim() != 2 or scores.stride(1) != 1:
        raise DiffCacheError("scores must be a 2-d fp32 tensor with contiguous rows")
    n_units = scores.shape[0]
    seq = [int(x) for x in k_check_seq]
    if len(seq) > 16:
        raise DiffCacheError(f"k_check_seq holds {len(seq)} sizes; dc_kcheck_f32 takes at most 16")
    arr = (C.c_int * max(len(seq), 1))(*seq)
    if n_eff is None:
        n_eff = torch.empty((n_units,), dtype=torch.int32, device=scores.device)
    alpha = mass = None
    if want_stats:
        alpha = torch.empty((n_units, len(seq)), dtype=torch.float32, device=scores.device)
        mass = torch.empty_like(alpha)
    _check(lib.dc_kcheck_f32(_dev(scores, "scores"), scores.stride(0), n_units, n_sel, hd, mode, arr,
                             len(seq), float(attn_mass_threshold), _dev(n_eff, "n_eff"),
                             _opt(alpha, "alpha"), _opt(mass, "mass"), _stream()))
    return (n_eff, alpha, mass) if want_stats else n_eff


def append_kv(store_k: torch.Tensor, store_v: torch.Tensor, new_k: torch.Tensor,
              new_v: torch.Tensor, pos: int, pos_dev: Optional[torch.Tensor] = None,
              pos_end: Optional[int] = None) -> None:
    """store[b, h, pos (+ pos_dev[0]), :] = new_k / new_v[b, h, :]; ``pos_dev``: an int32
    counter on the device added to ``pos`` when the kernel runs; rows at or beyond
    ``pos_end`` (default: the store's length) are not written."""
    sb, sh, sr = _store_strides(store_k)
    if _store_strides(store_v) != (sb, sh, sr):
        raise DiffCacheError("K and V stores must share their strides")
    b, h, n_max, hd = store_k.shape
    if not 0 <= pos < n_max:
        raise DiffCacheError(f"append position {pos} outside the store of {n_max} rows")
    new_k, new_v = new_k.contiguous(), new_v.contiguous()
    if new_k.numel() != b * h * hd or new_v.numel() != b * h * hd:
        raise DiffCacheError("new_k/new_v must hold (b, h, hd) values")
    _check(lib.dc_append_kv_bf16(_dev(store_k, "store_k"), _dev(store_v, "store_v"),
                                 _dev(new_k, "new_k"), _dev(new_v, "new_v"), b, h, hd, pos,
                                 _counter(pos_dev), n_max if pos_end is None else min(pos_end, n_max),
                                 sb, sh, sr, _stream()))


def step_advance(counter: torch.Tensor, delta: int = 1, limit: int = 2 ** 31 - 1) -> None:
    """counter[0] = clamp(counter[0] + delta, 0, limit), enqueued on the current stream."""
    _check(lib.dc_step_advance(_counter(counter), delta, limit, _stream()))


def step_state_advance(state: torch.Tensor, delta: int = 1, limit: int = 2 ** 31 - 1) -> None:
    """dc_step_state_advance on a 4-element int32 device tensor [n_recent, region_hi, append_pos, overflow]."""
    if not state.is_cuda or state.dtype != torch.int32 or state.numel() < 4 or not state.is_contiguous():
        raise DiffCacheError("the step state must be a contiguous int32 tensor of 4 elements in GPU memory")
    _check(lib.dc_step_state_advance(state.data_ptr(), delta, limit, _stream()))


def step_state_rollover(state: torch.Tensor, moved: int, keep: int) -> None:
    """dc_step_state_rollover: region_hi += moved, n_recent = keep, append_pos follows."""
    if not state.is_cuda or state.dtype != torch.int32 or state.numel() < 4 or not state.is_contiguous():
        raise DiffCacheError("the step state must be a contiguous int32 tensor of 4 elements in GPU memory")
    _check(lib.dc_step_state_rollover(state.data_ptr(), moved, keep, _stream()))


def ingest_kv(store: torch.Tensor, src: torch.Tensor, dst_pos: int = 0) -> None:
    """src (b, seq, h, hd) bf16 -> store[b, h, dst_pos + s, :]."""
    sb, sh, sr = _store_strides(store)
    b, h, n_max, hd = store.shape
    src = src.contiguous()
    if src.dtype != torch.bfloat16 or src.dim() != 4 or src.shape[0] != b or src.shape[2] != h \
            or src.shape[3] != hd:
        raise DiffCacheError("src must be a (b, seq, h, hd) bf16 tensor matching the store")
    seq = src.shape[1]
    if dst_pos < 0 or dst_pos + seq > n_max:
        raise DiffCacheError(f"rows [{dst_pos}, {dst_pos + seq}) outside the store of {n_max} rows")
    _check(lib.dc_ingest_kv_bf16(_dev(store, "store"), _dev(src, "src"), b, seq, h, hd, dst_pos, sb, sh,
                                 sr, _stream()))


def layer_workspace_bytes(n_units: int, n_region: int, budget: int, group: int, hd: int,
                          n_attended: int) -> int:
    return int(lib.dc_layer_workspace_bytes(n_units, n_region, budget, group, hd, n_attended))


def _layer_args(q, store_k, store_v, n_sink, recent_lo, n_recent, budget, scores, idx_out, out, workspace,
                new_k=None, new_v=None, lse=None, mode=MODE_REF_DIST, order=ORDER_ANY, scale=None,
                select_state_ready=False, scan_events=None, sketch=None, n_recent_dev=None,
                one_kernel=ONE_KERNEL_AUTO, region_hi_dev=None) -> "LayerArgs":
    """struct dc_layer_args from tensors (the arguments of decode_layer), with their checks."""
    sb, sh, sr = _store_strides(store_k)
    if _store_strides(store_v) != (sb, sh, sr):
        raise DiffCacheError("K and V stores must share their strides")
    b, h, n_max, hd = store_k.shape
    if recent_lo + n_recent > n_max:
        raise DiffCacheError("recent window runs past the end of the store")
    if not q.is_contiguous():
        raise DiffCacheError("q must be contiguous")
    group = q.numel() // (b * h * hd)
    if group < 1 or q.numel() != b * h * group * hd:
        raise DiffCacheError("q must hold (b, h * group, hd) values")
    if out.numel() < q.numel() or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise DiffCacheError("out must be a contiguous bf16 tensor of the size of q")
    if idx_out.dim() != 2 or idx_out.shape[0] < b * h or idx_out.element_size() != 4:
        raise DiffCacheError("idx_out must be a 32-bit (b * h, >= budget) tensor")
    a = LayerArgs()
    a.q, a.k, a.v = _dev(q, "q"), _dev(store_k, "store_k"), _dev(store_v, "store_v")
    a.new_k, a.new_v = _opt(new_k, "new_k"), _opt(new_v, "new_v")
    a.out, a.lse = _dev(out, "out"), _opt(lse, "lse")
    a.scores, a.idx_out = _opt(scores, "scores"), _dev(idx_out, "idx_out")
    a.workspace, a.workspace_bytes = _dev(workspace, "workspace"), workspace.numel()
    a.kv_batch_stride, a.kv_head_stride, a.kv_row_stride = sb, sh, sr
    a.scores_unit_stride = 0 if scores is None else scores.stride(0)
    a.idx_unit_stride = idx_out.stride(0)
    a.recent_lo = recent_lo
    a.n_b, a.n_h, a.group, a.hd = b, h, group, hd
    a.n_sink, a.n_recent, a.budget = n_sink, n_recent, budget
    a.mode, a.order = mode, order
    a.scale = 1.0 / math.sqrt(hd) if scale is None else scale
    a.select_state_ready = 1 if select_state_ready else 0
    if scan_events is not None:
        # torch creates the underlying event lazily: both must have been recorded once before
        a.ev_scan_begin, a.ev_scan_end = scan_events[0].cuda_event, scan_events[1].cuda_event
    if sketch is not None:
        c = sketch.codes
        if c.shape != store_k.shape:
            raise DiffCacheError("the sketch does not belong to this store")
        a.sketch_codes, a.sketch_scale = _dev(c, "codes"), _dev(sketch.scale, "scale")
        a.sketch_resid = _dev(sketch.resid, "resid")
        a.sketch_batch_stride, a.sketch_head_stride, a.sketch_row_stride = c.stride(0), c.stride(1), c.stride(2)
    a.n_recent_dev = _counter(n_recent_dev)
    a.one_kernel = one_kernel
    a.region_hi_dev = _counter(region_hi_dev)
    a._keep = (q, store_k, store_v, new_k, new_v, out, lse, scores, idx_out, workspace, sketch, n_recent_dev)
    return a


def decode_layer(q: torch.Tensor, store_k: torch.Tensor, store_v: torch.Tensor, n_sink: int,
                 recent_lo: int, n_recent: int, budget: int, scores: Optional[torch.Tensor],
                 idx_out: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor,
                 new_k: Optional[torch.Tensor] = None, new_v: Optional[torch.Tensor] = None,
                 lse: Optional[torch.Tensor] = None, mode: int = MODE_REF_DIST,
                 order: int = ORDER_ANY, scale: Optional[float] = None,
                 select_state_ready: bool = False,
                 scan_events: Optional[Tuple[torch.cuda.Event, torch.cuda.Event]] = None,
                 sketch: Optional["Sketch"] = None,
                 n_recent_dev: Optional[torch.Tensor] = None,
                 one_kernel: int = ONE_KERNEL_AUTO,
                 region_hi_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """score -> select -> attend for one layer, enqueued on the current stream.
    ``n_recent_dev``: the suffix length as a device-side int32 (``n_recent`` = capacity).
    ``select_state_ready``: see dc_layer_args in the header (skips the init kernel).
    ``sketch``: scan the 8-bit sketch of the keys instead of the keys (same result).
    ``one_kernel``: ONE_KERNEL_* policy for short contexts (see the header).
    ``region_hi_dev``: the end of the retrieval region as a device-side int32 (``recent_lo`` = its
    largest value), for captured steps that outlive a rollover of the recent window."""
    a = _layer_args(q, store_k, store_v, n_sink, recent_lo, n_recent, budget, scores, idx_out, out, workspace,
                    new_k, new_v, lse, mode, order, scale, select_state_ready, scan_events, sketch, n_recent_dev,
                    one_kernel, region_hi_dev)
    _check(lib.dc_decode_layer(C.byref(a), _stream()))
    return out


class LayerCall:
    """A decode_layer call with its argument struct built once: a serving loop that calls the same
    layer with the same tensors every step pays the checks of decode_layer once and a bare
    dc_decode_layer call afterwards.  The tensors are kept alive by the object."""

    def __init__(self, *args, **kwargs) -> None:
        self.args = _layer_args(*args, **kwargs)

    def __call__(self, select_state_ready: Optional[bool] = None,
                 scan_events: Optional[Tuple[torch.cuda.Event, torch.cuda.Event]] = None) -> None:
        a = self.args
        if select_state_ready is not None:
            a.select_state_ready = 1 if select_state_ready else 0
        if scan_events is not None:
            a.ev_scan_begin, a.ev_scan_end = scan_events[0].cuda_event, scan_events[1].cuda_event
        else:
            a.ev_scan_begin, a.ev_scan_end = None, None
        _check(lib.dc_decode_layer(C.byref(a), _stream()))

    def route(self) -> int:
        return int(lib.dc_decode_layer_route(C.byref(self.args)))


ROUTE_ATTEND_ONLY, ROUTE_DENSE, ROUTE_STREAM, ROUTE_SKETCH, ROUTE_ONE_KERNEL = range(5)


def last_route() -> int:
    """The route the last decode_layer call of this thread actually took (a ROUTE_* value)."""
    return int(lib.dc_last_route())


def decode_layer_errors() -> int:
    """Failures of the one-kernel route seen so far in this process (no synchronisation)."""
    return int(lib.dc_decode_layer_errors())


def decode_layer_route(*args, **kwargs) -> int:
    """Which kernels a decode_layer call with these arguments runs: a ROUTE_* value."""
    a = _layer_args(*args, **kwargs)
    rc = lib.dc_decode_layer_route(C.byref(a))
    if rc < 0:
        _check(rc)
    return rc


def decode_layer_status(*args, **kwargs) -> None:
    """Waits for the current stream and raises if a kernel of the last decode_layer calls on this
    workspace gave up a bounded wait between its blocks (dc_decode_layer_status).  Arguments as
    in the decode_layer call that it checks."""
    a = _layer_args(*args, **kwargs)
    _check(lib.dc_decode_layer_status(C.byref(a), _stream()))


# ---- PQ baseline ----

def pq_build_lut(q: torch.Tensor, books: torch.Tensor, n_b: int) -> torch.Tensor:
    """q (n_b*n_h, hd) bf16, books (n_h, M, 256, ds) fp32 -> lut (n_b*n_h, M, 256) fp32."""
    n_h, m, nc, ds = books.shape
    if nc != 256 or books.dtype != torch.float32:
        raise DiffCacheError("books must be (n_h, M, 256, ds) fp32")
    q, books = q.contiguous(), books.contiguous()
    lut = torch.empty((n_b * n_h, m, 256), dtype=torch.float32, device=q.device)
    _check(lib.dc_pq_build_lut(_dev(q, "q"), _dev(books, "books"), _dev(lut, "lut"), n_b, n_h, m * ds, m,
                               _stream()))
    return lut


def pq_adc_scan(codes: torch.Tensor, lut: torch.Tensor, hist: Optional[torch.Tensor] = None
                ) -> torch.Tensor:
    """codes (n_units, n_rows, M) uint8, lut (n_units, M, 256) -> scores (n_units, n_rows) fp32."""
    n_units, n_rows, m = codes.shape
    codes, lut = codes.contiguous(), lut.contiguous()
    scores = torch.empty((n_units, n_rows), dtype=torch.float32, device=codes.device)
    _check(lib.dc_pq_adc_scan(_dev(codes, "codes"), _dev(lut, "lut"), _dev(scores, "scores"),
                              _opt(hist, "hist"), n_units, n_rows, m, scores.stride(0), _stream()))
    return scores


def pq_search(store_k: torch.Tensor, codes: torch.Tensor, lut: torch.Tensor, q: torch.Tensor,
              n_cand: int, topk: int, idx_out: Optional[torch.Tensor] = None,
              workspace: Optional[torch.Tensor] = None, state_ready: bool = False,
              scan_events: Optional[Tuple[torch.cuda.Event, torch.cuda.Event]] = None) -> torch.Tensor:
    """ADC scan -> n_cand candidates -> exact rerank -> topk ids, best first, in one call
    (dc_pq_search_bf16).  store_k (b, h, n, hd) bf16, codes (b*h, n, M) uint8,
    lut (b*h, M, 256) fp32, q (b*h, hd) bf16 -> int32 (b*h, min(topk, n))."""
    sb, sh, sr = _store_strides(store_k)
    b, h, n, hd = store_k.shape
    n_units, n_rows, m = codes.shape
    if n_units != b * h or n_rows != n:
        raise ValueError("codes do not match the key store")
    codes, lut, q = codes.contiguous(), lut.contiguous(), q.contiguous()
    k2 = min(topk, n_cand, n)
    if idx_out is None:
        idx_out = torch.empty((n_units, k2), dtype=torch.int32, device=q.device)
    need = lib.dc_pq_search_workspace_bytes(n_units, n, n_cand)
    if workspace is None:
        workspace = alloc_workspace(need, q.device)
    _check(lib.dc_pq_search_bf16(_dev(store_k, "store_k"), _dev(codes, "codes"), _dev(lut, "lut"),
                                 _dev(q, "q"), _dev(idx_out, "idx_out"), idx_out.stride(0), b, h, n, hd, m,
                                 sb, sh, sr, n_cand, topk, int(state_ready), _dev(workspace, "workspace"),
                                 workspace.numel() * workspace.element_size(),
                                 scan_events[0].cuda_event if scan_events else None,
                                 scan_events[1].cuda_event if scan_events else None, _stream()))
    return idx_out


def score_gathered(store_k: torch.Tensor, q: torch.Tensor, idx: torch.Tensor, row_offset: int = 0,
                   scores: Optional[torch.Tensor] = None) -> torch.Tensor:
    sb, sh, sr = _store_strides(store_k)
    b, h, _, hd = store_k.shape
    q = q.contiguous()
    n_idx = idx.shape[1]
    if scores is None:
        scores = torch.empty((b * h, n_idx), dtype=torch.float32, device=q.device)
    _check(lib.dc_score_gathered_bf16(_dev(store_k, "store_k"), _dev(q, "q"), _dev(idx, "idx"),
                                      _dev(scores, "scores"), b, h, n_idx, idx.stride(0), hd, row_offset,
                                      sb, sh, sr, scores.stride(0), _stream()))
    return scores


def compose_idx(outer: torch.Tensor, inner: torch.Tensor) -> torch.Tensor:
    n_units, n_inner = inner.shape
    out = torch.empty((n_units, n_inner), dtype=torch.int32, device=inner.device)
    _check(lib.dc_compose_idx(_dev(outer, "outer"), outer.stride(0), _dev(inner, "inner"),
                              inner.stride(0), _dev(out, "out"), out.stride(0), n_units, n_inner,
                              _stream()))
    return out
