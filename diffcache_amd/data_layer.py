"""``DiffCacheHIP``: the HBM-resident counterpart of the reference's native data
layer ``diffcache._cpu.DiffCacheCPU`` (diffcache_cpu/src/lib.rs:523-660).

Same constructor, method names, argument meaning and failure behaviour; what
differs is where the data lives and how a query is answered:

* K and V of every (batch, kv-head) unit stay in GPU memory as bf16
  ``(bsz, kv_heads, max_ctx_len, head_dim)`` instead of host hugepages
  (lib.rs:83-150, nsw.rs:680-698);
* ``query`` is always the exact scan the reference runs with
  ``use_bruteforce=True`` (nsw.rs:592-630) -- score, exact top-``ef``, rows
  returned best first -- executed by the HIP kernels; no graph is built, so
  ``neighbours``, ``m`` and ``ef_cons`` are accepted and ignored.

bf16 crosses this boundary as raw ``uint16`` exactly as in the reference
(lib.rs:529-544); torch tensors (bf16 / int16 / uint16, on any device) are
accepted as well.  There is no CPU fallback: every computation runs in
``libdiffcache_hip.so``.
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional, Sequence, Union

import numpy as np
import torch

from . import _hip as hip
from . import snapshot

ArrayLike = Union[np.ndarray, torch.Tensor]

_DEFAULTS = dict(  # lib.rs:556-566
    max_ctx_len=1000000, m=16, ef_cons=200, r_sq=None, batch_search=False, name="l0",
    use_bruteforce=False, attn_mass_threshold=0.9,
    k_check_seq=[100, 200, 300, 400, 800, 1600, 3200, 6400, 12800, 25600],
)
_EXTRA = dict(device="cuda", key_mode="ref_dist", storage=None, key_sketch=False)  # not in the reference

_metrics: Dict[str, int] = {}
_metrics_on = False


def init_metrics() -> None:
    """Counterpart of ``_cpu.init_metrics`` (lib.rs:546-549,662-665).  The
    reference installs a TCP exporter; here the counters are kept in process
    and read with :func:`metrics`.  Calling it twice is harmless."""
    global _metrics_on
    _metrics_on = True


def metrics() -> Dict[str, int]:
    """Counters named as in the reference: ``<name>_num_searches``,
    ``<name>_total_query_latency`` (microseconds from the start of a query to the end of its
    search on the device: with metrics on, a query with device outputs waits for its stream)."""
    return dict(_metrics)


def _count(name: str, inc: int) -> None:
    if _metrics_on:
        _metrics[name] = _metrics.get(name, 0) + int(inc)


def _as_bf16(x: ArrayLike, device: torch.device) -> torch.Tensor:
    """uint16/int16 numpy or torch, or bf16 torch, to a bf16 tensor on ``device``."""
    if isinstance(x, np.ndarray):
        if x.dtype != np.uint16:
            raise TypeError(f"bf16 data must be passed as uint16, got {x.dtype}")
        t = torch.from_numpy(np.ascontiguousarray(x).view(np.int16)).view(torch.bfloat16)
    elif isinstance(x, torch.Tensor):
        if x.dtype == torch.bfloat16:
            t = x
        elif x.dtype in (torch.int16, torch.uint16):
            t = x.contiguous().view(torch.bfloat16)
        else:
            raise TypeError(f"bf16 data must be bfloat16/int16/uint16, got {x.dtype}")
    else:
        raise TypeError(f"unsupported array type {type(x)}")
    return t.to(device, non_blocking=True)


class DiffCacheHIP:
    def __init__(self, bsz: int, q_head_num: int, kv_head_num: int, head_dim: int, **kwargs) -> None:
        opt = dict(_DEFAULTS)
        opt.update(_EXTRA)
        for key, value in kwargs.items():
            if key not in opt:
                raise ValueError(f"Unknown option {key}")      # lib.rs:579
            opt[key] = value
        if q_head_num % kv_head_num != 0:
            raise AssertionError("q_head_num must be multiple of kv_head_num")   # lib.rs:294
        if head_dim not in (64, 128, 256):
            raise ValueError(f"head_dim {head_dim} is not supported by the HIP kernels (64, 128, 256)")
        if opt["key_mode"] not in ("ref_dist", "ip"):
            raise ValueError("key_mode must be 'ref_dist' or 'ip'")
        self.bsz, self.q_head_num, self.kv_head_num, self.head_dim = bsz, q_head_num, kv_head_num, head_dim
        self.max_ctx_len = int(opt["max_ctx_len"])
        self.m, self.ef_cons = int(opt["m"]), int(opt["ef_cons"])
        self.r_sq: List[float] = list(opt["r_sq"]) if opt["r_sq"] is not None else [4.0] * kv_head_num
        self.batch_search = bool(opt["batch_search"])
        self.name = str(opt["name"])
        self.use_bruteforce = bool(opt["use_bruteforce"])   # the scan here is always exact
        self.attn_mass_threshold = float(opt["attn_mass_threshold"])
        self.k_check_seq = [int(x) for x in opt["k_check_seq"]]
        self.mode = hip.MODE_REF_DIST if opt["key_mode"] == "ref_dist" else hip.MODE_IP
        self.device = torch.device(opt["device"])
        if self.device.type != "cuda":
            raise hip.DiffCacheError("DiffCacheHIP needs a GPU device; there is no CPU path")
        self.ctx_len = 0
        storage = opt["storage"]
        if storage is None:
            shape = (bsz, kv_head_num, self.max_ctx_len, head_dim)
            self.keys = torch.zeros(shape, dtype=torch.bfloat16, device=self.device)
            self.vals = torch.zeros(shape, dtype=torch.bfloat16, device=self.device)
        else:
            # rows of an existing HBM store, e.g. the retrieval region of a layer's K/V
            self.keys, self.vals = storage
            want = (bsz, kv_head_num, self.max_ctx_len, head_dim)
            hip.require(tuple(self.keys.shape) == want and tuple(self.vals.shape) == want,
                        f"storage must be two {want} bf16 tensors")
        self._ws: Optional[torch.Tensor] = None
        self._ws_key = None
        self._idx: Optional[torch.Tensor] = None
        # optional 8-bit sketch of the keys: queries scan it instead of the bf16 rows and
        # rescore the rows that can still matter; the ids are the same
        self.sketch: Optional[hip.Sketch] = hip.Sketch(self.keys) if opt["key_sketch"] else None

    def _resketch(self) -> None:
        if self.sketch is not None and self.ctx_len > 0:
            self.sketch.build(self.keys, 0, self.ctx_len)

    # ------------------------------------------------------------------ ingest
    def prefill(self, keys: ArrayLike, vals: ArrayLike, neighbours: Optional[ArrayLike] = None) -> None:
        """keys, vals (bsz, kv_heads, seq, hd) bf16-as-u16 (lib.rs:329-347).
        ``neighbours`` is the kNN graph the reference needs; unused here."""
        k = _as_bf16(keys, self.device)
        v = _as_bf16(vals, self.device)
        seq = k.shape[2] if k.dim() == 4 else -1
        want = (self.bsz, self.kv_head_num, seq, self.head_dim)
        hip.require(tuple(k.shape) == want, f"keys shape {tuple(k.shape)} != {want}")        # lib.rs:332
        hip.require(tuple(v.shape) == want, f"vals shape {tuple(v.shape)} != {want}")        # lib.rs:333
        hip.require(seq <= self.max_ctx_len, "sequence longer than max_ctx_len")
        self.keys[:, :, :seq].copy_(k)
        self.vals[:, :, :seq].copy_(v)
        self.ctx_len = seq
        self._resketch()

    def prefill_bshd(self, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        """Ingest straight from the model layout (bsz, seq, kv_heads, hd) with the
        layout-transform kernel (what diffcache.py:142-147 does through the host)."""
        seq = key_states.shape[1]
        hip.require(seq <= self.max_ctx_len, "sequence longer than max_ctx_len")
        hip.ingest_kv(self.keys, key_states, 0)
        hip.ingest_kv(self.vals, value_states, 0)
        self.ctx_len = seq
        self._resketch()

    def insert(self, keys: ArrayLike, vals: ArrayLike) -> None:
        """keys, vals (bsz, kv_heads, hd): append one token (lib.rs:352-369)."""
        k = _as_bf16(keys, self.device)
        v = _as_bf16(vals, self.device)
        want = (self.bsz, self.kv_head_num, self.head_dim)
        hip.require(tuple(k.shape) == want, f"keys shape {tuple(k.shape)} != {want}")        # lib.rs:353
        hip.require(tuple(v.shape) == want, f"vals shape {tuple(v.shape)} != {want}")        # lib.rs:354
        hip.require(self.ctx_len < self.max_ctx_len, "index is full")
        hip.append_kv(self.keys, self.vals, k, v, self.ctx_len)
        if self.sketch is not None:
            if self.ctx_len == 0:
                self.sketch.build(self.keys, 0, 1)
            else:   # keep the fitted scales; the residual bounds grow if the row lies outside them
                self.sketch.build(self.keys, self.ctx_len, 1, keep_scale=True)
        self.ctx_len += 1

    # ------------------------------------------------------------------ query
    def _workspace(self, n_rows: int, ef: int) -> torch.Tensor:
        key = (n_rows, ef)
        if self._ws is None or self._ws_key != key:
            n_units = self.bsz * self.kv_head_num
            self._ws = hip.alloc_workspace(hip.score_select_workspace_bytes(n_units, n_rows, ef), self.device)
            self._idx = torch.empty((n_units, max(ef, 1)), dtype=torch.int32, device=self.device)
            self._ws_key = key
        return self._ws

    def query_ids(self, queries: ArrayLike, ef: int, return_scores: bool = False):
        """Node ids (bsz*kv_heads, ef') best first, as int32 on the device; with
        ``return_scores`` also the dense fp32 scores (bsz*kv_heads, ctx_len)."""
        ef = min(ef, self.ctx_len)
        q = _as_bf16(queries, self.device)
        want = (self.bsz, self.kv_head_num, self.head_dim)
        hip.require(tuple(q.shape) == want, f"queries shape {tuple(q.shape)} != {want}")     # lib.rs:376
        if ef <= 0:
            empty = torch.empty((self.bsz * self.kv_head_num, 0), dtype=torch.int32, device=self.device)
            return (empty, None) if return_scores else empty
        if return_scores:
            scores = hip.score(self.keys, q, 0, self.ctx_len, self.mode)
            ids = hip.topk_select(scores, ef, self.mode, hip.ORDER_BEST)
            return ids, scores
        ws = self._workspace(self.ctx_len, ef)
        if self.sketch is not None:
            return hip.score_select_sketch(self.keys, self.sketch, q.contiguous(), 0, self.ctx_len, ef,
                                           self.mode, hip.ORDER_BEST, idx_out=self._idx, workspace=ws)
        return hip.score_select(self.keys, q.contiguous(), 0, self.ctx_len, ef, self.mode, hip.ORDER_BEST,
                                idx_out=self._idx, workspace=ws)

    def query(self, out_keys: ArrayLike, out_vals: ArrayLike, queries: ArrayLike, ef: int) -> None:
        """Write the ``min(ef, ctx_len)`` best K and V rows of every unit, best
        first, into ``out_keys`` / ``out_vals`` (bsz, kv_heads, >= ef', hd)
        (lib.rs:373-404, nsw.rs:592-630).  Host arrays are filled after a
        device-to-host copy; GPU tensors are written in place without a sync."""
        t0 = time.perf_counter()
        ef_eff = min(ef, self.ctx_len)
        ids = self.query_ids(queries, ef)
        _count(f"{self.name}_num_searches", self.bsz * self.kv_head_num)
        if ef_eff <= 0:
            return
        dev_out = isinstance(out_keys, torch.Tensor) and out_keys.is_cuda
        if dev_out:
            ok = out_keys if out_keys.dtype == torch.bfloat16 else out_keys.view(torch.bfloat16)
            ov = out_vals if out_vals.dtype == torch.bfloat16 else out_vals.view(torch.bfloat16)
        else:
            shape = (self.bsz, self.kv_head_num, ef_eff, self.head_dim)
            ok = torch.empty(shape, dtype=torch.bfloat16, device=self.device)
            ov = torch.empty(shape, dtype=torch.bfloat16, device=self.device)
        hip.require(ok.shape[0] == self.bsz and ok.shape[1] == self.kv_head_num and ok.shape[2] >= ef_eff
                    and ok.shape[3] == self.head_dim, "out_keys must be (bsz, kv_heads, >= ef, head_dim)")
        hip.require(ov.shape == ok.shape, "out_vals must match out_keys")
        hip.gather_rows(self.keys, self.vals, ids, ok, ov, row_offset=0, n_idx=ef_eff)
        if not dev_out:
            for dst, src in ((out_keys, ok), (out_vals, ov)):
                host = src.cpu().view(torch.int16).numpy().view(np.uint16)
                if isinstance(dst, np.ndarray):
                    dst[:, :, :ef_eff, :] = host
                else:
                    dst.view(torch.int16)[:, :, :ef_eff, :] = torch.from_numpy(host.view(np.int16))
        if _metrics_on:
            # the reference's counter is the time of the search itself (lib.rs:373-404 runs it to the
            # end before it returns); with device outputs the call above only enqueued it
            if dev_out:
                torch.cuda.current_stream(self.device).synchronize()
            _count(f"{self.name}_total_query_latency", (time.perf_counter() - t0) * 1e6)

    def query_streaming(self, cuda_stream: int, out_keys_gpu: int, out_vals_gpu: int,
                        queries: ArrayLike, ef: int) -> None:
        """Raw-pointer variant (lib.rs:626-636): rows go to the device buffers
        ``out_*_gpu`` (bsz, kv_heads, ef', hd) on stream ``cuda_stream``.  The
        reference streams chunks over PCIe as the graph search stabilises; here
        the rows are already on the device, so this is one gather."""
        ef_eff = min(ef, self.ctx_len)
        if ef_eff <= 0:
            return
        ext = torch.cuda.ExternalStream(cuda_stream, device=self.device)
        with torch.cuda.stream(ext):
            ids = self.query_ids(queries, ef)
            sb, sh, sr = self.keys.stride(0), self.keys.stride(1), self.keys.stride(2)
            hd = self.head_dim
            rc = hip.lib.dc_gather_rows_bf16(
                self.keys.data_ptr(), self.vals.data_ptr(), ids.data_ptr(), out_keys_gpu, out_vals_gpu,
                self.bsz, self.kv_head_num, ef_eff, ids.stride(0), hd, 0, sb, sh, sr,
                self.kv_head_num * ef_eff * hd, ef_eff * hd, hd, cuda_stream)
            hip._check(rc)

    # ------------------------------------------------------------------ misc
    def get_keys(self) -> np.ndarray:
        """(bsz, kv_heads, ctx_len, hd) float32 (lib.rs:646-649)."""
        return self.keys[:, :, :self.ctx_len].float().cpu().numpy()

    def update_r_sq(self, r_sq: Sequence[float]) -> None:
        hip.require(len(r_sq) == self.kv_head_num, "r_sq length must match kv_head_num")     # lib.rs:652
        self.r_sq = [float(x) for x in r_sq]

    def save(self, path: str) -> None:
        """One snapshot per unit named ``<path>b%03d_h%03d.idx`` -- the prefix is
        concatenated without a separator, as lib.rs:484-494 does -- in the
        reference's bincode layout (nsw.rs:58-72,704-733) with empty edge lists."""
        k = self.keys[:, :, :self.ctx_len].float().cpu().numpy()
        v = self.vals[:, :, :self.ctx_len].float().cpu().numpy()
        for b in range(self.bsz):
            for h in range(self.kv_head_num):
                snapshot.write(f"{path}b{b:03d}_h{h:03d}.idx", k[b, h], v[b, h], m=self.m,
                               ef_cons=self.ef_cons, n_max=self.max_ctx_len, r_sq=self.r_sq[h],
                               name=f"{self.name}b{b * self.kv_head_num + h:03d}h{h:03d}",
                               attn_mass_threshold=self.attn_mass_threshold,
                               k_check_seq=self.k_check_seq)

    def load(self, path: str, ctx_len: int) -> None:
        """lib.rs:496-506.  ``ctx_len`` becomes the context length as in the
        reference, which passes the full prompt length (diffcache.py:264,291);
        the scan never goes past the nodes the snapshots hold."""
        n_min = None
        for b in range(self.bsz):
            for h in range(self.kv_head_num):
                snap = snapshot.read(f"{path}b{b:03d}_h{h:03d}.idx")
                hip.require(snap["dim"] == self.head_dim, "snapshot dimension does not match")
                n = snap["n_nodes_stored"]
                hip.require(n <= self.max_ctx_len, "snapshot longer than max_ctx_len")
                n_min = n if n_min is None else min(n_min, n)
                self.keys[b, h, :n].copy_(torch.from_numpy(snap["keys"]).to(torch.bfloat16))
                self.vals[b, h, :n].copy_(torch.from_numpy(snap["vals"]).to(torch.bfloat16))
                self.r_sq[h] = snap["options"]["r_sq"]
        # the reference scans valid nodes only (nsw.rs:601-605), whatever ctx_len says
        self.ctx_len = min(int(ctx_len), n_min if n_min is not None else 0)
        self._resketch()
