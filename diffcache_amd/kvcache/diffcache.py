"""``DiffCache``: the reference's KV-cache operator API on an HBM-resident store.

Constructor and method names, argument meaning and call order are those of
``src/diffcache/kvcache/diffcache.py:15-300`` so the model harness
(``src/diffcache/base.py:83,125,133,151-154,174,210,242``) can use it unchanged:

    prefill_update_kv_cache(key_states, value_states, layer_idx)
    get_kvcache(layer_idx)
    decode_pre_query_operation(queries)      # inside the captured pre-attention graph
    decode_query_kvcache(layer_idx)          # between the two graphs
    decode_post_query_operation(layer_idx)   # inside the captured post-attention graph
    seq_len / seq_len_gpu, save_prefill_cache / load_prefill_cache

What changed underneath.  The reference keeps only ``budget + prefix +
suffix_max`` rows per head on the GPU and sends every decode query through the
host (D2H, device sync, Rust search, H2D).  Here all K/V rows of every layer
stay in HBM as bf16 ``(bsz, kv_heads, max_length, head_dim)``; the three hooks
enqueue the group-mean, the exact scan + top-k, and a device-side row gather on
the current stream, with no host synchronisation and no allocation, so they
are capturable.  ``kbuf`` / ``vbuf`` keep the reference's geometry
``[retrieved (right aligned) | prefix | suffix]`` for harnesses that run their
own attention over ``get_kvcache()``.

``decode_attention`` is the native path that has no counterpart in the
reference: score -> select -> attention straight from the store (one C call),
replacing the ``flash_attn_with_kvcache`` call of ``base.py:134-142`` as well.

Step state.  The length of the recent window, the row at which the retrieval region ends
and the row the next token is appended at live in a small int32 tensor on the device
(``dc_step_state`` of the header; ``step_state`` is the view of its first word), like the
``cache_seqlens`` tensor the reference hands to flash-attn (``base.py:134-142,150-152``):
a captured ``decode_attention`` appends at, scans up to and attends over the rows those
words name, and advances them after the last layer.  A call captured in a HIP graph
therefore stays right on every replay; after replays the host's mirror
(``kvbuf_suffix_len``) is brought up to date with ``advance_host_step``.

Rollover.  The reference never moves tokens out of the recent window into its index
(``diffcache.py:221`` asserts instead, although ``lib.rs:352-369`` exists for it), so a
sequence ends after ``kvbuf_suffix_maxlen - kvbuf_suffix_len`` tokens.  Here the rows are
already in the store, so when the window is full the region boundary simply moves: the
oldest rows of the window join the retrieval region (their sketch rows are added with the
fitted scales kept) and the window shrinks back to its initial length (``rollover``;
``generation`` counts them).  The call only enqueues work on the stream -- sketch rows, two
device words -- so it may sit between two replays of a captured step, and a step that was
captured while the region held at least ``retrieval_budget`` rows stays valid across it,
as the reference's graphs do for a whole generation (``base.py:46-55``); one captured with
a shorter region, or with ``use_k_check``, has the region's end as a launch parameter and
must be captured again (``captured_region_on_device`` tells which).

Two options beyond the reference's arguments.  ``key_sketch`` (default on): an
8-bit sketch of the keys is built at prefill and the scans read it instead of
the bf16 keys, rescoring only the rows that can still reach the top-k; the ids
are the same, the scan moves half the bytes (+25 % memory).  ``use_k_check``
(default off): ``decode_attention`` applies the reference's k-check
(``nsw.rs:198-296``, ``attn_mass_threshold``, ``k_check_seq``) to every unit's
best-first result and attends only to the rows it finds sufficient.
"""
from __future__ import annotations

import json
import os
from typing import List, Optional

import torch

from .. import _hip as hip
from ..data_layer import DiffCacheHIP, init_metrics


class DiffCache:
    def __init__(
        self,
        num_layers: int,
        batch_size: int,
        max_length: int,
        num_kv_heads: int,
        num_q_heads: int,
        head_dim: int,
        retrieval_budget: int,
        nsw_m: int,
        nsw_ef_cons: int,
        kvbuf_prefix_len: int,
        kvbuf_suffix_len: int,
        kvbuf_suffix_maxlen: int,
        attn_mass_threshold: float,
        k_check_seq: List[int],
        r_sq: List[List[float]],
        key_mode: str = "ref_dist",
        device: str = "cuda",
        key_sketch: bool = True,
        use_k_check: bool = False,
        hook_order: int = hip.ORDER_BEST,
        exclusive_gpu: bool = False,
    ) -> None:
        # hook_order: order of the ids that decode_query_kvcache selects, hence of the rows that
        # decode_post_query_operation gathers into kbuf/vbuf.  ORDER_BEST is the reference's
        # (best first, nsw.rs:592-630); attention over the buffer does not depend on the order, so
        # a caller that only attends may pass hip.ORDER_ANY and save the sort.
        # exclusive_gpu: the caller vouches that nothing else keeps CUs of this GPU busy while this
        # cache decodes (no second cache decoding on another stream, no long-lived kernels).  Short
        # contexts then run as one kernel under graph capture too; without it a captured step takes
        # the kernel chain, and an eager one does whenever another cache's one-kernel launch is
        # still in flight on another stream.
        hip.require(hook_order in (hip.ORDER_ANY, hip.ORDER_BEST, hip.ORDER_INDEX), "bad hook_order")
        self.hook_order = hook_order
        self.one_kernel = hip.ONE_KERNEL_EXCLUSIVE if exclusive_gpu else hip.ONE_KERNEL_AUTO
        self._errors_seen = hip.decode_layer_errors()
        self.failed_steps = 0         # decode steps whose one-kernel launch reported a wait that ran out
        self.num_layers = num_layers
        self.batch_size = batch_size
        self.max_length = max_length
        self.num_kv_heads = num_kv_heads
        self.num_q_heads = num_q_heads
        self.head_dim = head_dim
        self.retrieval_budget = retrieval_budget
        self.nsw_m = nsw_m
        self.nsw_ef_cons = nsw_ef_cons
        self.r_sq = r_sq
        self.attn_mass_threshold = attn_mass_threshold
        self.k_check_seq = k_check_seq
        self.key_mode = key_mode
        self.mode = hip.MODE_REF_DIST if key_mode == "ref_dist" else hip.MODE_IP
        self.device = torch.device(device)
        self.data_layers: List[Optional[DiffCacheHIP]] = [None for _ in range(num_layers)]
        self.retrieval_region_len = 0

        # kvbuf geometry of the reference (diffcache.py:48-66):
        #   [ retrieval_budget | prefix_len | suffix_maxlen ], layout (bsz, kh, seq, hd)
        self.kvbuf_suffix_maxlen = kvbuf_suffix_maxlen
        self.kvbuf_prefix_len = kvbuf_prefix_len
        self.kvbuf_suffix_len = kvbuf_suffix_len
        kvbuf_len = retrieval_budget + kvbuf_prefix_len + kvbuf_suffix_maxlen
        shape = (batch_size, num_kv_heads, kvbuf_len, head_dim)
        self.kbuf = [torch.empty(shape, device=self.device, dtype=torch.bfloat16) for _ in range(num_layers)]
        self.vbuf = [torch.empty(shape, device=self.device, dtype=torch.bfloat16) for _ in range(num_layers)]

        # the HBM-resident store that replaces the host index: every row of every layer
        # One allocation for all layers' keys and one for all values: on MI355X a scan of
        # a single large allocation runs about 3 % faster than scans of per-layer buffers.
        store = (num_layers, batch_size, num_kv_heads, max_length, head_dim)
        self._vslab = torch.zeros(store, device=self.device, dtype=torch.bfloat16)
        self._kslab = torch.zeros(store, device=self.device, dtype=torch.bfloat16)
        self.kstore = [self._kslab[l] for l in range(num_layers)]
        self.vstore = [self._vslab[l] for l in range(num_layers)]
        # 8-bit sketch of the keys (one byte per element, +25 % memory): the scan reads it
        # instead of the bf16 keys and rescores the rows that can still matter, with the same
        # result.  Allocated last: it is the buffer every decode step streams.
        self.key_sketch = key_sketch
        self.sketch: List[Optional[hip.Sketch]] = [None] * num_layers
        if key_sketch:
            self._cslab = torch.zeros(store, device=self.device, dtype=torch.uint8)
            self.sketch = [hip.Sketch(self.kstore[l], codes=self._cslab[l]) for l in range(num_layers)]

        n_units = batch_size * num_kv_heads
        self.group = num_q_heads // num_kv_heads
        # group-mean query of the current layer (the reference's pinned qbuf_cpu, diffcache.py:80)
        self.qbuf = torch.zeros((batch_size, num_kv_heads, head_dim), device=self.device, dtype=torch.bfloat16)
        # selected node ids of every layer, relative to the retrieval region, best first
        self.idx = [torch.zeros((n_units, max(retrieval_budget, 1)), device=self.device, dtype=torch.int32)
                    for _ in range(num_layers)]
        self._ws: Optional[torch.Tensor] = None
        self._ws_rows = -1
        # The select state inside the workspace is laid out differently by dc_decode_layer and
        # by the stand-alone select calls, so each route keeps its own "left ready" flag and
        # clears the other's.
        self._ws_ready = False        # a decode_attention call has left its select state ready
        self._ws_order = None         # ... for calls of this id order
        self._hook_ws_ready = False   # a decode_query_kvcache call (sketch route) has
        self._attn_out: Optional[torch.Tensor] = None
        # k-check (nsw.rs:198-296): with use_k_check, decode_attention attends only to the
        # leading rows of each unit's best-first list that the check finds sufficient
        # (attn_mass_threshold, k_check_seq); n_eff[layer] holds the sizes it chose.
        self.use_k_check = use_k_check
        self.n_eff = [torch.zeros((n_units,), device=self.device, dtype=torch.int32)
                      for _ in range(num_layers)] if use_k_check else []
        self._kc_scores: Optional[torch.Tensor] = None
        self._attn_ws: Optional[torch.Tensor] = None
        self._prefix0 = kvbuf_prefix_len
        self._suffix0 = kvbuf_suffix_len
        # device-side step state [n_recent, region_hi, append_pos, overflow] (dc_step_state); the
        # host mirrors are kvbuf_suffix_len and _region()
        self._state = torch.zeros((4,), device=self.device, dtype=torch.int32)
        self.step_state = self._state[0:1]
        self.captured_region_on_device: Optional[bool] = None   # of the last captured decode_attention
        # suffix rows that are present in kstore / vstore: all of them on the native route,
        # only the prompt's on the hook route (the harness's attention call writes the new
        # tokens into kbuf / vbuf, as flash_attn_with_kvcache does for the reference)
        self._store_suffix_rows = kvbuf_suffix_len
        self.generation = 0           # number of rollovers so far

        init_metrics()

    # ------------------------------------------------------------------ helpers
    def _region(self):
        lo = self.kvbuf_prefix_len
        return lo, lo + self.retrieval_region_len

    def _ensure_workspace(self) -> torch.Tensor:
        """Scratch for one layer call, sized once for the longest region the store can hold
        (the region grows at every rollover)."""
        region = self.retrieval_region_len
        if self._ws is None or self._ws_rows < region:
            n_units = self.batch_size * self.num_kv_heads
            cap = max(region, self.max_length - self.kvbuf_prefix_len - min(self._suffix0, self.kvbuf_suffix_maxlen))
            attended = min(cap, self.retrieval_budget) + self.kvbuf_prefix_len + self.kvbuf_suffix_maxlen + 1
            self._ws = hip.alloc_workspace(
                hip.layer_workspace_bytes(n_units, cap, self.retrieval_budget, self.group,
                                          self.head_dim, attended), self.device)
            self._ws_rows = cap
            self._ws_ready = False
            self._hook_ws_ready = False
        return self._ws

    def _set_suffix_len(self, n: int) -> None:
        """Window length and, from the host's view of the region, the whole device-side state."""
        self.kvbuf_suffix_len = n
        _, hi = self._region()
        self._state[0:1].fill_(n)
        self._state[1:2].fill_(hi)
        self._state[2:3].fill_(hi + n)

    def check_status(self) -> None:
        """Waits for the device and raises if a decoded token was dropped because the recent
        window was full when its step ran (replays of a captured step beyond the window's
        capacity without ``rollover()``), or if a one-kernel launch gave up a wait."""
        n_recent, region_hi, append_pos, overflow = self._state.tolist()
        hip.require(overflow == 0, "a decode step ran with a full recent window: its token was not stored "
                                   "(call rollover() before the step that finds the window full)")
        self._note_failures()
        hip.require(self.failed_steps == 0, f"{self.failed_steps} one-kernel launches gave up a wait; their outputs were NaN")

    def advance_host_step(self, steps: int = 1) -> None:
        """After ``steps`` replays of a captured decode step: bring the host's mirror of the
        recent-window length up to the device's counter (no synchronisation)."""
        self.kvbuf_suffix_len += steps
        self._store_suffix_rows += steps
        hip.require(self.kvbuf_suffix_len <= self.kvbuf_suffix_maxlen,
                    "more steps were replayed than the recent window holds; call rollover() in time")

    def window_full(self) -> bool:
        return self.kvbuf_suffix_len >= self.kvbuf_suffix_maxlen

    def rollover(self) -> int:
        """Move the oldest rows of the recent window into the retrieval region (see the module
        docstring).  Between two decode steps (or two replays of a captured one), never under
        graph capture; only enqueues work on the current stream.  Returns the number of rows
        moved."""
        hip.require(not torch.cuda.is_current_stream_capturing(), "rollover() cannot be captured in a graph")
        keep = min(self._suffix0, self.kvbuf_suffix_maxlen - 1)
        moved = self.kvbuf_suffix_len - keep
        if moved <= 0:
            return 0
        lo, hi = self._region()
        p, s, b0 = self.kvbuf_prefix_len, self.kvbuf_suffix_len, self.retrieval_budget
        hip.require(hi + s <= self.max_length, "store is full")
        for l in range(self.num_layers):
            ks, vs = self.kstore[l], self.vstore[l]
            have = self._store_suffix_rows
            if have < s:    # hook route: the decoded tokens live in kbuf / vbuf only
                ks[:, :, hi + have:hi + s].copy_(self.kbuf[l][:, :, b0 + p + have:b0 + p + s])
                vs[:, :, hi + have:hi + s].copy_(self.vbuf[l][:, :, b0 + p + have:b0 + p + s])
            if self.key_sketch:
                first = self.retrieval_region_len == 0       # nothing was sketched yet: fit the scales
                self.sketch[l].build(ks, hi if not first else lo, moved, keep_scale=not first)
            # the assembled buffer's suffix = the rows that stay in the window
            self.kbuf[l][:, :, b0 + p:b0 + p + keep].copy_(ks[:, :, hi + moved:hi + s])
            self.vbuf[l][:, :, b0 + p:b0 + p + keep].copy_(vs[:, :, hi + moved:hi + s])
        self.retrieval_region_len += moved
        self.kvbuf_suffix_len = keep
        hip.step_state_rollover(self._state, moved, keep)      # the device's view, in stream order
        self._store_suffix_rows = keep
        self._ws_ready = False
        self._hook_ws_ready = False
        self.generation += 1
        for l in range(self.num_layers):
            if self.data_layers[l] is not None:
                self._bind_data_layer(l)
        return moved

    # ------------------------------------------------------------------ prefill
    def prefill_update_kv_cache(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int):
        """key_states / value_states (bsz, seq_len, num_kv_heads, head_dim) bf16 on the
        GPU (diffcache.py:149-184)."""
        seq_len = key_states.size(1)
        hip.require(seq_len <= self.max_length, "prompt longer than max_length")

        # r_sq from the prefill keys, as the reference does; only the graph build needed it
        r_sq = torch.einsum("bshd,bshd->bsh", key_states, key_states).max(dim=1).values.max(dim=0).values.tolist()
        self.r_sq[layer_idx] = r_sq

        # all rows into the store, (b, s, h, d) -> (b, h, s, d)
        hip.ingest_kv(self.kstore[layer_idx], key_states, 0)
        hip.ingest_kv(self.vstore[layer_idx], value_states, 0)

        prefix_len = min(self._prefix0, seq_len)                    # diffcache.py:163
        suffix_len = min(self._suffix0, seq_len - prefix_len)       # diffcache.py:169
        self.kvbuf_prefix_len = prefix_len
        self.retrieval_region_len = seq_len - prefix_len - suffix_len
        self._set_suffix_len(suffix_len)
        self._store_suffix_rows = suffix_len
        if self.key_sketch and self.retrieval_region_len > 0:
            self.sketch[layer_idx].build(self.kstore[layer_idx], prefix_len, self.retrieval_region_len)

        # prefix and suffix rows of the assembled buffer (diffcache.py:164-171)
        b0 = self.retrieval_budget
        ks, vs = self.kstore[layer_idx], self.vstore[layer_idx]
        self.kbuf[layer_idx][:, :, b0:b0 + prefix_len].copy_(ks[:, :, :prefix_len])
        self.vbuf[layer_idx][:, :, b0:b0 + prefix_len].copy_(vs[:, :, :prefix_len])
        s0 = seq_len - suffix_len
        self.kbuf[layer_idx][:, :, b0 + prefix_len:b0 + prefix_len + suffix_len].copy_(ks[:, :, s0:seq_len])
        self.vbuf[layer_idx][:, :, b0 + prefix_len:b0 + prefix_len + suffix_len].copy_(vs[:, :, s0:seq_len])

        self._bind_data_layer(layer_idx)
        return key_states, value_states

    def _bind_data_layer(self, layer_idx: int) -> None:
        """The layer's retrieval region seen through the reference's data-layer API."""
        lo, hi = self._region()
        n = hi - lo
        self.data_layers[layer_idx] = DiffCacheHIP(
            bsz=self.batch_size, q_head_num=self.num_q_heads, kv_head_num=self.num_kv_heads,
            head_dim=self.head_dim, max_ctx_len=n, m=self.nsw_m, ef_cons=self.nsw_ef_cons,
            r_sq=self.r_sq[layer_idx], name=f"l{layer_idx:03d}",
            attn_mass_threshold=self.attn_mass_threshold, k_check_seq=self.k_check_seq,
            key_mode=self.key_mode, device=str(self.device),
            storage=(self.kstore[layer_idx][:, :, lo:hi], self.vstore[layer_idx][:, :, lo:hi]))
        self.data_layers[layer_idx].ctx_len = n

    def get_kvcache(self, layer_idx: int):
        retrieval_len = min(self.retrieval_region_len, self.retrieval_budget)
        start = self.retrieval_budget - retrieval_len
        return (self.kbuf[layer_idx][:, :, start:, :].permute(0, 2, 1, 3),
                self.vbuf[layer_idx][:, :, start:, :].permute(0, 2, 1, 3))

    # ------------------------------------------------------------------ decode hooks
    def decode_pre_query_operation(self, queries: torch.Tensor) -> None:
        """GQA-group mean of the layer's queries (diffcache.py:191-194), kept on the device."""
        hip.group_mean(queries, self.group, out=self.qbuf.view(-1, self.head_dim), hd=self.head_dim)

    def decode_query_kvcache(self, layer_idx: int) -> None:
        """Exact scan + top-k of the retrieval region with the mean query
        (diffcache.py:211-223 -> lib.rs:373-404 -> nsw.rs:592-630)."""
        if layer_idx == 0 and self.window_full():
            self.rollover()                                                  # diffcache.py:221 asserts instead
        retrieval_len = min(self.retrieval_region_len, self.retrieval_budget)
        if retrieval_len > 0:
            lo, hi = self._region()
            ws = self._ensure_workspace()
            if self.key_sketch:
                hip.score_select_sketch(self.kstore[layer_idx], self.sketch[layer_idx], self.qbuf, lo, hi - lo,
                                        retrieval_len, self.mode, self.hook_order, idx_out=self.idx[layer_idx],
                                        workspace=ws, state_ready=self._hook_ws_ready)
                self._hook_ws_ready = True
            else:
                hip.score_select(self.kstore[layer_idx], self.qbuf, lo, hi - lo, retrieval_len, self.mode,
                                 self.hook_order, idx_out=self.idx[layer_idx], workspace=ws)
                self._hook_ws_ready = False   # the one-shot call does not leave the state initialised
            self._ws_ready = False
        hip.require(self.kvbuf_suffix_len < self.kvbuf_suffix_maxlen,
                    "the recent window is full (kvbuf_suffix_maxlen)")       # diffcache.py:221
        if layer_idx == self.num_layers - 1:
            self.kvbuf_suffix_len += 1                                       # diffcache.py:222-223
            hip.step_state_advance(self._state, 1, self.kvbuf_suffix_maxlen)

    def decode_post_query_operation(self, layer_idx: int) -> None:
        """Selected rows into kbuf/vbuf[:, :, budget - len : budget] (diffcache.py:196-209)."""
        retrieval_len = min(self.retrieval_region_len, self.retrieval_budget)
        if retrieval_len <= 0:
            return
        lo, _ = self._region()
        b0 = self.retrieval_budget
        hip.gather_rows(self.kstore[layer_idx], self.vstore[layer_idx], self.idx[layer_idx],
                        self.kbuf[layer_idx][:, :, b0 - retrieval_len:b0],
                        self.vbuf[layer_idx][:, :, b0 - retrieval_len:b0], row_offset=lo, n_idx=retrieval_len)

    # ------------------------------------------------------------------ native decode path
    def decode_attention(self, layer_idx: int, queries: torch.Tensor, key_states: torch.Tensor,
                         value_states: torch.Tensor, out: Optional[torch.Tensor] = None,
                         order: int = hip.ORDER_ANY) -> torch.Tensor:
        """One layer of the decode path in one call: append the token's k/v to the
        store, score the retrieval region with the group-mean query, select the
        exact top-``retrieval_budget``, attend over [selected | prefix | suffix +
        this token].  queries (bsz, 1, Hq*hd) or (bsz, Hq, hd); key/value_states
        (bsz, 1, Hkv, hd).  Returns (bsz, Hq, hd) bf16.  Call it for every layer of
        a step; the suffix grows by one after the last layer."""
        b, hq, hkv, hd = self.batch_size, self.num_q_heads, self.num_kv_heads, self.head_dim
        capturing = torch.cuda.is_current_stream_capturing()
        if layer_idx == 0:
            self._note_failures()
        if layer_idx == 0 and self.window_full() and not capturing:
            self.rollover()                                                  # diffcache.py:221 asserts instead
        hip.require(self.kvbuf_suffix_len < self.kvbuf_suffix_maxlen,
                    "the recent window is full (kvbuf_suffix_maxlen): call rollover() between steps")
        lo, hi = self._region()
        hip.require(hi + self.kvbuf_suffix_len < self.max_length, "store is full")
        q = queries.reshape(b, hq, hd)
        if not q.is_contiguous():
            q = q.contiguous()
        nk, nv = key_states.reshape(b, hkv, hd), value_states.reshape(b, hkv, hd)
        if not nk.is_contiguous():
            nk = nk.contiguous()
        if not nv.is_contiguous():
            nv = nv.contiguous()
        # Under capture the region's end is read from the device wherever the path allows it (a
        # region of at least `budget` rows, no k-check), so that the graph outlives a rollover:
        # launches and workspace are then laid out for the longest region the store can hold.
        dev_region = capturing and not self.use_k_check and hi - lo >= self.retrieval_budget > 0
        if capturing:
            self.captured_region_on_device = dev_region
        hi_cap = self.max_length - self.kvbuf_suffix_maxlen
        if dev_region:
            # the token's row is the device's append position; never past the end of the store
            hip.append_kv(self.kstore[layer_idx], self.vstore[layer_idx], nk, nv, 0, pos_dev=self._state[2:3],
                          pos_end=self.max_length)
        else:
            # the token's row: hi + (device-side window length); never past the window's capacity
            hip.append_kv(self.kstore[layer_idx], self.vstore[layer_idx], nk, nv, hi, pos_dev=self.step_state,
                          pos_end=min(hi + self.kvbuf_suffix_maxlen, self.max_length))
        if out is None:
            if self._attn_out is None:
                self._attn_out = torch.empty((b, hq, hd), device=self.device, dtype=torch.bfloat16)
            out = self._attn_out
        ws = self._ensure_workspace()
        if self.use_k_check and min(hi - lo, self.retrieval_budget) > 0:
            self._decode_attention_k_check(layer_idx, q, nk, nv, out, ws)
        else:
            # attended: [selected | prefix | the window's rows before this token | this token]
            # (a call with the region's end on the device has other launch sizes than one without:
            #  neither leaves the select state ready for the other)
            tag = (order, dev_region)
            hip.decode_layer(q, self.kstore[layer_idx], self.vstore[layer_idx], lo, hi_cap if dev_region else hi,
                             self.kvbuf_suffix_maxlen, self.retrieval_budget, None, self.idx[layer_idx], out, ws,
                             nk, nv, mode=self.mode, order=order,
                             select_state_ready=self._ws_ready and self._ws_order == tag,
                             sketch=self.sketch[layer_idx], n_recent_dev=self.step_state,
                             one_kernel=self.one_kernel,
                             region_hi_dev=self._state[1:2] if dev_region else None)
            self._ws_ready = True
            self._ws_order = tag        # the state is left ready for a call of the same kind only
            self._hook_ws_ready = False
        if layer_idx == self.num_layers - 1:
            hip.step_state_advance(self._state, 1, self.kvbuf_suffix_maxlen)
            if not capturing:       # a captured step is counted when it is replayed (advance_host_step)
                self.kvbuf_suffix_len += 1
                self._store_suffix_rows += 1
        return out

    def _note_failures(self) -> None:
        """A one-kernel launch of this process reported a wait between its blocks that ran out
        (read from pinned host memory, no synchronisation): that step's outputs were NaN.  The
        select state of the workspace is initialised again on the next call, and this cache
        stays on the kernel chain from here on: whatever starved the kernel of CUs may still be
        there."""
        n = hip.decode_layer_errors()
        if n != self._errors_seen:
            self.failed_steps += n - self._errors_seen
            self._errors_seen = n
            self._ws_ready = False
            self._hook_ws_ready = False
            self.one_kernel = hip.ONE_KERNEL_NEVER

    def _decode_attention_k_check(self, layer_idx: int, q: torch.Tensor, nk: torch.Tensor, nv: torch.Tensor,
                                  out: torch.Tensor, ws: torch.Tensor) -> None:
        """select (best first) -> exact scores of the selected rows -> k-check -> attention over
        the leading n_eff rows of every unit plus the always-kept rows."""
        lo, hi = self._region()
        n_sel = min(hi - lo, self.retrieval_budget)
        n_units = self.batch_size * self.num_kv_heads
        ks, vs, idx = self.kstore[layer_idx], self.vstore[layer_idx], self.idx[layer_idx]
        if self.key_sketch:
            hip.score_select_sketch(ks, self.sketch[layer_idx], q, lo, hi - lo, n_sel, self.mode,
                                    hip.ORDER_BEST, q_group=self.group, idx_out=idx, workspace=ws,
                                    state_ready=self._hook_ws_ready)
            self._hook_ws_ready = True
        else:
            hip.score_select(ks, q, lo, hi - lo, n_sel, self.mode, hip.ORDER_BEST, q_group=self.group,
                             idx_out=idx, workspace=ws)
            self._hook_ws_ready = False
        self._ws_ready = False
        hip.group_mean(q, self.group, out=self.qbuf.view(-1, self.head_dim), hd=self.head_dim)
        if self._kc_scores is None or self._kc_scores.shape[1] != n_sel:
            self._kc_scores = torch.empty((n_units, n_sel), device=self.device, dtype=torch.float32)
        hip.score_gathered(ks, self.qbuf, idx[:, :n_sel], row_offset=lo, scores=self._kc_scores)
        hip.kcheck(self._kc_scores, n_sel, self.head_dim, self.k_check_seq, self.attn_mass_threshold,
                   self.mode, n_eff=self.n_eff[layer_idx])
        need = hip.lib.dc_attn_workspace_bytes(n_units, self.group, self.head_dim,
                                               n_sel + self.kvbuf_prefix_len + self.kvbuf_suffix_maxlen + 1)
        if self._attn_ws is None or self._attn_ws.numel() < need:
            self._attn_ws = hip.alloc_workspace(need, self.device)
        hip.gather_attn(q, ks, vs, idx, n_sel, lo, lo, hi, self.kvbuf_suffix_maxlen, nk, nv, out=out,
                        workspace=self._attn_ws, n_idx_unit=self.n_eff[layer_idx], n_recent_dev=self.step_state)

    # ------------------------------------------------------------------ prefill cache
    def save_prefill_cache(self, prefill_cache_path: str) -> None:
        """Same directory layout as diffcache.py:225-259."""
        path = os.path.join(prefill_cache_path, "metadata.txt")
        metadata = {
            "r_sq": self.r_sq,
            "kvbuf_prefix_len": self.kvbuf_prefix_len,
            "kvbuf_suffix_len": self.kvbuf_suffix_len,
            "retrieval_region_len": self.retrieval_region_len,
        }
        with open(path, "w") as f:
            json.dump(metadata, f)
        b0, p, s = self.retrieval_budget, self.kvbuf_prefix_len, self.kvbuf_suffix_len
        _, hi = self._region()
        for layer_idx in range(self.num_layers):
            layer_path = os.path.join(prefill_cache_path, f"p_l_{layer_idx:03d}")
            os.makedirs(layer_path, exist_ok=False)
            torch.save(self.kbuf[layer_idx][:, :, b0:b0 + p, :], os.path.join(layer_path, "k.pt"))
            torch.save(self.vbuf[layer_idx][:, :, b0:b0 + p, :], os.path.join(layer_path, "v.pt"))
        for layer_idx in range(self.num_layers):
            layer_path = os.path.join(prefill_cache_path, f"s_l_{layer_idx:03d}")
            os.makedirs(layer_path, exist_ok=False)
            # The window's rows: from the store where it has them (the native route appends
            # there and never touches kbuf / vbuf), else from the assembled buffer (hook route).
            have = min(self._store_suffix_rows, s)
            sk = torch.cat([self.kstore[layer_idx][:, :, hi:hi + have],
                            self.kbuf[layer_idx][:, :, b0 + p + have:b0 + p + s]], dim=2)
            sv = torch.cat([self.vstore[layer_idx][:, :, hi:hi + have],
                            self.vbuf[layer_idx][:, :, b0 + p + have:b0 + p + s]], dim=2)
            torch.save(sk, os.path.join(layer_path, "k.pt"))
            torch.save(sv, os.path.join(layer_path, "v.pt"))
        for layer_idx in range(self.num_layers):
            layer_path = os.path.join(prefill_cache_path, f"d_l_{layer_idx:03d}")
            os.makedirs(layer_path, exist_ok=False)
            self.data_layers[layer_idx].save(layer_path)

    def load_prefill_cache(self, inputs_ids: torch.Tensor, prefill_cache_path: str) -> None:
        """diffcache.py:261-293; the K/V rows come back into the HBM store."""
        ctx_len = inputs_ids.size(1)
        with open(os.path.join(prefill_cache_path, "metadata.txt"), "r") as f:
            metadata = json.load(f)
        self.r_sq = metadata["r_sq"]
        self.kvbuf_prefix_len = metadata["kvbuf_prefix_len"]
        self.retrieval_region_len = metadata["retrieval_region_len"]
        self._set_suffix_len(metadata["kvbuf_suffix_len"])
        self._store_suffix_rows = self.kvbuf_suffix_len
        b0, p, s = self.retrieval_budget, self.kvbuf_prefix_len, self.kvbuf_suffix_len
        lo, hi = self._region()
        for layer_idx in range(self.num_layers):
            pp = os.path.join(prefill_cache_path, f"p_l_{layer_idx:03d}")
            sp = os.path.join(prefill_cache_path, f"s_l_{layer_idx:03d}")
            pk = torch.load(os.path.join(pp, "k.pt"), weights_only=True).to(self.device)
            pv = torch.load(os.path.join(pp, "v.pt"), weights_only=True).to(self.device)
            sk = torch.load(os.path.join(sp, "k.pt"), weights_only=True).to(self.device)
            sv = torch.load(os.path.join(sp, "v.pt"), weights_only=True).to(self.device)
            self.kbuf[layer_idx][:, :, b0:b0 + p, :] = pk
            self.vbuf[layer_idx][:, :, b0:b0 + p, :] = pv
            self.kbuf[layer_idx][:, :, b0 + p:b0 + p + s, :] = sk
            self.vbuf[layer_idx][:, :, b0 + p:b0 + p + s, :] = sv
            self.kstore[layer_idx][:, :, :p] = pk
            self.vstore[layer_idx][:, :, :p] = pv
            self.kstore[layer_idx][:, :, hi:hi + s] = sk
            self.vstore[layer_idx][:, :, hi:hi + s] = sv
        for layer_idx in range(self.num_layers):
            self._bind_data_layer(layer_idx)
            layer_path = os.path.join(prefill_cache_path, f"d_l_{layer_idx:03d}")
            self.data_layers[layer_idx].load(layer_path, ctx_len)
            self.data_layers[layer_idx].update_r_sq(self.r_sq[layer_idx])
            if self.key_sketch and hi > lo:
                self.sketch[layer_idx].build(self.kstore[layer_idx], lo, hi - lo)

    def seq_len(self, layer_idx: int) -> int:
        return self.kvbuf_prefix_len + self.kvbuf_suffix_len + self.retrieval_region_len

    def seq_len_gpu(self, layer_idx: int) -> int:
        retrieval_len = min(self.retrieval_region_len, self.retrieval_budget)
        return self.kvbuf_prefix_len + self.kvbuf_suffix_len + retrieval_len
