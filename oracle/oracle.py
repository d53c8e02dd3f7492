"""CPU oracle for the decode-time retrieval path (TEST INFRASTRUCTURE ONLY).

This module is a checker.  It restates, in numpy, what the reference computes
on its decode path so that the HIP kernels can be compared against it.  It is
imported only by tests, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; the product (``diffcache_amd``) never
imports it and has no CPU fallback.

What each function follows in the reference (paths relative to the reference
checkout):

=====================  =====================================================
function               reference
=====================  =====================================================
group_mean_bf16        src/diffcache/kvcache/diffcache.py:191-194
scores_f64/scores_f32  diffcache_cpu/src/nsw.rs:129-139, lib.rs:65-69
ref_dist               diffcache_cpu/src/nsw.rs:138
pack_neighbour         diffcache_cpu/src/nsw.rs:74-80
search_bruteforce      diffcache_cpu/src/nsw.rs:592-630
topk_select            same set/order as search_bruteforce, vectorised
data_layer_query       diffcache_cpu/src/lib.rs:373-404
DualHeap               diffcache_cpu/src/dualheap.rs:4-87
region_split           src/diffcache/kvcache/diffcache.py:163-176,
                       tools/topk_test.py:355-364
assemble_kvbuf         src/diffcache/kvcache/diffcache.py:48-66,186-209
sparse_attention       src/diffcache/base.py:134-142 (flash-attn decode call,
                       default scale 1/sqrt(hd), new token appended)
decode_layer           src/diffcache/base.py:150-155 call order
fit_alpha_from_logits  diffcache_cpu/src/nsw.rs:198-241
estimate_top_h_mass    diffcache_cpu/src/nsw.rs:243-278
k_check_early_stoppable diffcache_cpu/src/nsw.rs:280-296
k_check_budget         the epoch loop of nsw.rs:302-303,339,367-379 applied to
                       the exact, sorted result list
pq_*                   no reference source (evaluation/impl/pqcache is an
                       empty directory): PARITY UNPINNED at the reference;
                       pinned by closed forms in tests/test_oracle_pq.py
                       (pq_adc_scores_f32 restates the HIP kernels' documented
                       fp32 order of additions and is compared bit for bit)
=====================  =====================================================

Parity status.  The reference holds golden vectors only for ``DualHeap``
(dualheap.rs:191-358); ``tests/test_oracle_dualheap.py`` replays them.  For
every other function the reference has no tests, so they are pinned by closed
forms, brute force and library routines (see ``tests/test_oracle_*.py``).  Two
third-party routines are absent from the reference tree and are restated from
their published contract: simsimd 6.5.3 ``dot`` for bf16 (fp32 accumulate,
order unspecified) and flash-attn ``flash_attn_with_kvcache`` (softmax(q.k *
scale) . v with fp32 accumulate).  Bit-level agreement with simsimd's
accumulation order is "parity unpinned"; the bar used instead is 1e-5
relative on scores.
"""
from __future__ import annotations

import heapq
from typing import Optional, Sequence, Tuple

import numpy as np

MODE_IP = 0        # order by raw inner product, descending
MODE_REF_DIST = 1  # order by f32(65536 - ip) exactly as nsw.rs:138 does

# --------------------------------------------------------------------------
# bf16 <-> f32 on raw uint16 (the reference carries bf16 as u16, lib.rs:529-544)
# --------------------------------------------------------------------------


def bf16_to_f32(u16: np.ndarray) -> np.ndarray:
    u16 = np.asarray(u16, dtype=np.uint16)
    return (u16.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 (raw uint16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    b = x.view(np.uint32)
    lsb = (b >> np.uint32(16)) & np.uint32(1)
    rounded = (b + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    out = rounded.astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


# --------------------------------------------------------------------------
# A1: GQA-group mean query
# --------------------------------------------------------------------------


def group_mean_bf16(q_u16: np.ndarray, num_kv_heads: int) -> np.ndarray:
    """queries (b, Hq, hd) bf16 -> (b, Hkv, hd) bf16.

    diffcache.py:193: ``queries.view(b, Hkv, G, hd).mean(dim=2)`` in bf16, which
    torch evaluates as an fp32 sum over the group followed by one division and
    one rounding to bf16.
    """
    q = bf16_to_f32(q_u16)
    b, hq, hd = q.shape
    g = hq // num_kv_heads
    q = q.reshape(b, num_kv_heads, g, hd)
    acc = np.zeros((b, num_kv_heads, hd), dtype=np.float32)
    for i in range(g):
        acc = (acc + q[:, :, i, :]).astype(np.float32)
    mean = (acc / np.float32(g)).astype(np.float32)
    return f32_to_bf16(mean)


# --------------------------------------------------------------------------
# A2: scores and the reference's ordering key
# --------------------------------------------------------------------------


def scores_f64(q_u16: np.ndarray, k_u16: np.ndarray) -> np.ndarray:
    """Exact inner products: q (hd,), K (n, hd) -> (n,) float64.

    bf16 x bf16 products are exact in fp32, so the float64 sum is the value
    every fp32 accumulation order approximates (nsw.rs:138, lib.rs:65-69).
    """
    q = bf16_to_f32(q_u16).astype(np.float64)
    k = bf16_to_f32(k_u16).astype(np.float64)
    return k @ q


def scores_f32(q_u16: np.ndarray, k_u16: np.ndarray) -> np.ndarray:
    return scores_f64(q_u16, k_u16).astype(np.float32)


def ref_dist(scores: np.ndarray) -> np.ndarray:
    """nsw.rs:138: ``65536.0 - dot`` evaluated in f32."""
    return (np.float32(65536.0) - np.asarray(scores, dtype=np.float32)).astype(np.float32)


def _f2ord(x: np.ndarray) -> np.ndarray:
    """Order-preserving map f32 -> u32 (ascending)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    neg = (b >> np.uint32(31)).astype(bool)
    return np.where(neg, ~b, b | np.uint32(0x80000000)).astype(np.uint32)


def key32(scores: np.ndarray, mode: int) -> np.ndarray:
    """32-bit ordering key: smaller key = better match.

    MODE_REF_DIST: order-preserving bits of ``f32(65536 - s)``; for the positive
    distances the reference assumes (nsw.rs:127,136) this orders exactly like
    the raw ``to_bits()`` the reference packs (nsw.rs:76).
    MODE_IP: order-preserving bits of ``-s`` with -0.0 folded onto +0.0.
    """
    s = np.asarray(scores, dtype=np.float32)
    if mode == MODE_REF_DIST:
        return _f2ord(ref_dist(s))
    s = (s + np.float32(0.0)).astype(np.float32)
    return _f2ord((-s).astype(np.float32))


def pack_neighbour(dist: np.ndarray, node: np.ndarray) -> np.ndarray:
    """nsw.rs:74-80: u64 = (dist.to_bits() << 32) | node."""
    d = np.ascontiguousarray(dist, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (d << np.uint64(32)) | np.asarray(node, dtype=np.uint64)


# --------------------------------------------------------------------------
# A3: exact top-ef
# --------------------------------------------------------------------------


def search_bruteforce(scores: np.ndarray, ef: int) -> np.ndarray:
    """Literal restatement of the scan loop of nsw.rs:600-621 on given scores.

    A size-``ef`` max-heap of packed u64 keys; a new node replaces the heap's
    maximum only when its distance is strictly smaller (nsw.rs:612); the result
    is the heap sorted ascending (nsw.rs:621).  Returns node ids, best first.
    Pure-Python loop: small inputs only.
    """
    dist = ref_dist(scores)
    packed = pack_neighbour(dist, np.arange(len(dist), dtype=np.uint64))
    heap: list = []  # max-heap via negated ints
    for node in range(len(dist)):
        key = int(packed[node])
        if len(heap) < ef:
            heapq.heappush(heap, -key)
        elif ef > 0 and dist[node] < np.uint32((-heap[0]) >> 32).view(np.float32):
            heapq.heapreplace(heap, -key)
    out = sorted(-k for k in heap)
    return np.array([k & 0xFFFFFFFF for k in out], dtype=np.uint32)


def topk_select(scores: np.ndarray, k: int, mode: int) -> np.ndarray:
    """The ``min(k, n)`` smallest (key32, index) pairs, ascending.

    Same set and order as ``search_bruteforce`` in MODE_REF_DIST (checked in
    tests); in MODE_IP it is "highest score first, ties to the lower index".
    """
    s = np.asarray(scores, dtype=np.float32)
    n = s.shape[0]
    k = min(k, n)
    if k <= 0:
        return np.zeros((0,), dtype=np.uint32)
    key = key32(s, mode).astype(np.uint64)
    packed = (key << np.uint64(32)) | np.arange(n, dtype=np.uint64)
    if k < n:
        part = np.partition(packed, k - 1)[:k]
    else:
        part = packed
    part = np.sort(part)
    return (part & np.uint64(0xFFFFFFFF)).astype(np.uint32)


def data_layer_query(keys_u16: np.ndarray, vals_u16: np.ndarray, queries_u16: np.ndarray,
                     ef: int, mode: int = MODE_REF_DIST
                     ) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """lib.rs:373-404: per (b, kv-head) exact search + row gather.

    keys/vals (b, Hkv, ctx, hd) u16, queries (b, Hkv, hd) u16.
    Returns (out_keys, out_vals) shaped (b, Hkv, ef', hd) with ef' = min(ef, ctx)
    and the selected node ids (b, Hkv, ef'), rows sorted best first.
    """
    b, h, ctx, hd = keys_u16.shape
    ef = min(ef, ctx)
    out_k = np.zeros((b, h, ef, hd), dtype=np.uint16)
    out_v = np.zeros((b, h, ef, hd), dtype=np.uint16)
    ids = np.zeros((b, h, ef), dtype=np.uint32)
    for bi in range(b):
        for hi in range(h):
            s = scores_f32(queries_u16[bi, hi], keys_u16[bi, hi])
            sel = topk_select(s, ef, mode)
            ids[bi, hi] = sel
            out_k[bi, hi] = keys_u16[bi, hi][sel]
            out_v[bi, hi] = vals_u16[bi, hi][sel]
    return out_k, out_v, ids


# --------------------------------------------------------------------------
# A5: DualHeap (dualheap.rs:4-87), kept literal so its own tests can be replayed
# --------------------------------------------------------------------------


class DualHeap:
    """Keeps the smallest ``cap`` items; exposes the d-th smallest."""

    def __init__(self, d: int, cap: int) -> None:
        assert d >= 1, "d must be >= 1"
        assert cap >= d, "cap must be >= d"
        self.d = d
        self.cap = cap
        self.small: list = []  # max-heap (negated): the d smallest
        self.rest: list = []   # max-heap (negated): the next cap - d
        self.small_replace_count = 0

    def __len__(self) -> int:
        return len(self.small) + len(self.rest)

    def dth_min(self):
        if len(self) < self.d:
            return None
        return -self.small[0]

    def kept_max(self):
        if self.rest:
            return -self.rest[0]
        if self.small:
            return -self.small[0]
        return None

    def push(self, item) -> None:
        if len(self.small) < self.d:
            heapq.heappush(self.small, -item)
            return
        if -self.small[0] > item:
            self.small_replace_count += 1
            item = -heapq.heapreplace(self.small, -item)
        if self.cap == self.d:
            return
        if len(self.rest) < self.cap - self.d:
            heapq.heappush(self.rest, -item)
            return
        if -self.rest[0] <= item:
            return
        heapq.heapreplace(self.rest, -item)

    def extend(self, items) -> None:
        for it in items:
            self.push(it)

    def into_sorted_vec(self) -> list:
        return sorted(-x for x in self.small) + sorted(-x for x in self.rest)


# --------------------------------------------------------------------------
# A6: regions and the assembled buffer
# --------------------------------------------------------------------------


def region_split(seq_len: int, prefix_len: int, suffix_len: int) -> Tuple[int, int, int, int]:
    """diffcache.py:163,169,175 / topk_test.py:359-364.

    Returns (p_len, s_len, retrieval_start, retrieval_end).
    """
    p_len = max(0, min(prefix_len, seq_len))
    s_len = max(0, min(suffix_len, seq_len - p_len))
    return p_len, s_len, p_len, seq_len - s_len


def attended_rows(sel_region_ids: np.ndarray, p_len: int, region_end: int, n_ctx: int) -> np.ndarray:
    """Absolute row numbers in the order the reference lays them out in kbuf:
    [retrieved best-first | prefix | suffix] (diffcache.py:48-52,202-209)."""
    sel = np.asarray(sel_region_ids, dtype=np.int64) + p_len
    return np.concatenate([sel, np.arange(p_len, dtype=np.int64),
                           np.arange(region_end, n_ctx, dtype=np.int64)])


def assemble_kvbuf(k_u16: np.ndarray, v_u16: np.ndarray, rows: np.ndarray
                   ) -> Tuple[np.ndarray, np.ndarray]:
    return k_u16[rows], v_u16[rows]


# --------------------------------------------------------------------------
# A7: attention over the selected rows
# --------------------------------------------------------------------------


def sparse_attention(q_u16: np.ndarray, k_rows_u16: np.ndarray, v_rows_u16: np.ndarray,
                     new_k_u16: Optional[np.ndarray] = None,
                     new_v_u16: Optional[np.ndarray] = None,
                     scale: Optional[float] = None) -> Tuple[np.ndarray, np.ndarray]:
    """q (G, hd) bf16; K/V rows (S, hd) bf16; optional current-token k/v (hd,).

    float64 softmax(q.K^T * scale) . V over the rows plus the current token
    (base.py:134-142: flash_attn_with_kvcache appends k/v at cache_seqlens and
    the single query sees every row).  Returns (out f64 (G, hd), lse f64 (G,)).
    """
    q = bf16_to_f32(q_u16).astype(np.float64)
    k = bf16_to_f32(k_rows_u16).astype(np.float64)
    v = bf16_to_f32(v_rows_u16).astype(np.float64)
    if new_k_u16 is not None:
        k = np.concatenate([k, bf16_to_f32(new_k_u16).astype(np.float64)[None, :]], axis=0)
        v = np.concatenate([v, bf16_to_f32(new_v_u16).astype(np.float64)[None, :]], axis=0)
    hd = q.shape[-1]
    if scale is None:
        scale = 1.0 / np.sqrt(hd)
    if k.shape[0] == 0:
        return np.zeros_like(q), np.full((q.shape[0],), -np.inf)
    logits = (q @ k.T) * scale
    m = logits.max(axis=1, keepdims=True)
    p = np.exp(logits - m)
    l = p.sum(axis=1, keepdims=True)
    out = (p @ v) / l
    lse = (m + np.log(l))[:, 0]
    return out, lse


def decode_layer(q_u16: np.ndarray, k_u16: np.ndarray, v_u16: np.ndarray,
                 num_kv_heads: int, budget: int, prefix_len: int, suffix_len: int,
                 mode: int = MODE_REF_DIST,
                 new_k_u16: Optional[np.ndarray] = None,
                 new_v_u16: Optional[np.ndarray] = None,
                 scores_override: Optional[np.ndarray] = None):
    """One layer of the decode path for one batch element.

    q (Hq, hd); K, V (Hkv, n_ctx, hd); new_k/new_v (Hkv, hd) or None.
    Returns dict(qmean (Hkv,hd) u16, scores list, sel list, out (Hq,hd) f64).
    ``scores_override`` (Hkv, region) lets a caller select on scores it
    measured elsewhere ("identical scores" parity).
    """
    hq, hd = q_u16.shape
    g = hq // num_kv_heads
    n_ctx = k_u16.shape[1]
    p_len, s_len, lo, hi = region_split(n_ctx, prefix_len, suffix_len)
    qmean = group_mean_bf16(q_u16[None], num_kv_heads)[0]
    out = np.zeros((hq, hd), dtype=np.float64)
    lse = np.zeros((hq,), dtype=np.float64)
    all_scores, all_sel = [], []
    for h in range(num_kv_heads):
        if scores_override is not None:
            s = np.asarray(scores_override[h], dtype=np.float32)
        else:
            s = scores_f32(qmean[h], k_u16[h, lo:hi])
        sel = topk_select(s, budget, mode)
        rows = attended_rows(sel, p_len, hi, n_ctx)
        kr, vr = assemble_kvbuf(k_u16[h], v_u16[h], rows)
        o, l = sparse_attention(q_u16[h * g:(h + 1) * g], kr, vr,
                                None if new_k_u16 is None else new_k_u16[h],
                                None if new_v_u16 is None else new_v_u16[h])
        out[h * g:(h + 1) * g] = o
        lse[h * g:(h + 1) * g] = l
        all_scores.append(s)
        all_sel.append(sel)
    return {"qmean": qmean, "scores": all_scores, "sel": all_sel, "out": out, "lse": lse}


# --------------------------------------------------------------------------
# A9: product quantisation, asymmetric distance (no reference source)
# --------------------------------------------------------------------------


def pq_train(keys_f32: np.ndarray, m: int, n_centroids: int, iters: int, seed: int) -> np.ndarray:
    """Seeded Lloyd k-means per subspace.  keys (n, hd) f32 -> codebooks
    (m, n_centroids, hd/m) f32.  Initial centroids = a seeded sample of the
    keys; empty cells keep their previous centroid."""
    n, hd = keys_f32.shape
    ds = hd // m
    rng = np.random.RandomState(seed)
    books = np.zeros((m, n_centroids, ds), dtype=np.float32)
    for j in range(m):
        x = keys_f32[:, j * ds:(j + 1) * ds].astype(np.float32)
        c = x[rng.choice(n, size=n_centroids, replace=n < n_centroids)].copy()
        for _ in range(iters):
            d = (x * x).sum(1)[:, None] - 2.0 * (x @ c.T) + (c * c).sum(1)[None, :]
            a = d.argmin(1)
            sums = np.zeros_like(c, dtype=np.float64)
            np.add.at(sums, a, x)
            cnt = np.bincount(a, minlength=n_centroids)
            nz = cnt > 0
            c[nz] = (sums[nz] / cnt[nz, None]).astype(np.float32)
        books[j] = c
    return books


def pq_encode(keys_f32: np.ndarray, books: np.ndarray) -> np.ndarray:
    """Nearest centroid (squared L2, ties to the lower code) per subspace."""
    m, nc, ds = books.shape
    n = keys_f32.shape[0]
    codes = np.zeros((n, m), dtype=np.uint8)
    for j in range(m):
        x = keys_f32[:, j * ds:(j + 1) * ds].astype(np.float64)
        c = books[j].astype(np.float64)
        d = (x * x).sum(1)[:, None] - 2.0 * (x @ c.T) + (c * c).sum(1)[None, :]
        codes[:, j] = d.argmin(1).astype(np.uint8)
    return codes


def pq_build_lut(q_u16: np.ndarray, books: np.ndarray) -> np.ndarray:
    """LUT[m][c] = q[m*ds:(m+1)*ds] . centroid[m][c], float64."""
    m, nc, ds = books.shape
    q = bf16_to_f32(q_u16).astype(np.float64).reshape(m, ds)
    return np.einsum("md,mcd->mc", q, books.astype(np.float64))


def pq_adc_scores(codes: np.ndarray, lut: np.ndarray) -> np.ndarray:
    """s_i = sum_m LUT[m][codes[i, m]], float64."""
    m = lut.shape[0]
    return lut[np.arange(m)[None, :], codes.astype(np.int64)].sum(axis=1)


def pq_adc_scores_f32(codes: np.ndarray, lut_f32: np.ndarray) -> np.ndarray:
    """The same sums in fp32 and in the order the HIP kernels document: key i adds
    subspaces (i mod M), (i mod M) + 1, ... cyclically, starting from 0.0f."""
    n, m = codes.shape
    lut_f32 = lut_f32.astype(np.float32)
    rows = np.arange(n)
    acc = np.zeros(n, dtype=np.float32)
    for j in range(m):
        s = (rows + j) % m
        acc = (acc + lut_f32[s, codes[rows, s].astype(np.int64)]).astype(np.float32)
    return acc


def pq_reconstruct(codes: np.ndarray, books: np.ndarray) -> np.ndarray:
    m, nc, ds = books.shape
    return books[np.arange(m)[None, :], codes.astype(np.int64)].reshape(codes.shape[0], m * ds)


def pq_search(q_u16: np.ndarray, k_u16: np.ndarray, codes: np.ndarray, lut_f32: np.ndarray,
              n_cand: int, k: int) -> Tuple[np.ndarray, np.ndarray]:
    """ADC scan -> n_cand candidates (MODE_IP order on fp32 ADC scores) ->
    exact bf16 rerank to top-k (ties to the lower key index).  Returns
    (candidates best-ADC first, top-k key ids best first)."""
    adc = pq_adc_scores(codes, lut_f32.astype(np.float64)).astype(np.float32)
    cand = topk_select(adc, n_cand, MODE_IP)
    exact = scores_f32(q_u16, k_u16[cand])
    packed = (key32(exact, MODE_IP).astype(np.uint64) << np.uint64(32)) | cand.astype(np.uint64)
    packed = np.sort(packed)[:min(k, len(cand))]
    return cand, (packed & np.uint64(0xFFFFFFFF)).astype(np.uint32)


# --------------------------------------------------------------------------
# k-check: does the top-H already hold the wanted attention mass?
# (nsw.rs:198-296; no tests in the reference -- pinned by closed forms in
# tests/test_oracle_kcheck.py)
# --------------------------------------------------------------------------

K_CHECK_MIN_RANK = 5  # nsw.rs:288
MAX_EF = 16384        # nsw.rs:15: length of the reference's ln(rank) table


def fit_alpha_from_logits(logits_sorted: np.ndarray, min_rank: int) -> Optional[np.float32]:
    """Least-squares slope of logit against ln(rank) over ranks min_rank..H; alpha = -slope
    (nsw.rs:198-241).  Sums in f64 in rank order, result cast to f32."""
    z = np.asarray(logits_sorted, dtype=np.float32)
    h = len(z)
    if h == 0 or min_rank == 0 or min_rank >= h:
        return None
    if h > MAX_EF:      # the reference's ln(rank) table ends there (nsw.rs:15,207-210)
        return None
    n = float(h - min_rank + 1)
    if n < 2.0:
        return None
    sx = sy = sxx = sxy = 0.0
    for idx in range(min_rank - 1, h):
        x = float(np.log(np.float64(idx + 1)))
        y = float(z[idx])
        sx += x
        sy += y
        sxx += x * x
        sxy += x * y
    denom = n * sxx - sx * sx
    if abs(denom) < 1e-12:
        return None
    b = (n * sxy - sx * sy) / denom
    return np.float32(-b)


def estimate_top_h_mass(logits_sorted: np.ndarray, h: int, alpha: np.float32) -> Optional[np.float32]:
    """Share of the softmax mass the first h logits hold when the rest follows a power law
    with exponent alpha: head / (head + v_h * h / (alpha - 1)), all in f32, sums in rank
    order (nsw.rs:243-278)."""
    z = np.asarray(logits_sorted, dtype=np.float32)
    if h == 0 or h > len(z):
        return None
    alpha = np.float32(alpha)
    if alpha <= np.float32(1.0):
        return None
    head = z[:h]
    mx = np.float32(head.max())
    head_sum = np.float32(0.0)
    for v in head:
        head_sum = np.float32(head_sum + np.exp(np.float32(v - mx), dtype=np.float32))
    v_h = np.exp(np.float32(head[h - 1] - mx), dtype=np.float32)
    tail = np.float32(np.float32(v_h * np.float32(h)) / np.float32(alpha - np.float32(1.0)))
    denom = np.float32(head_sum + tail)
    if denom <= 0:
        return None
    return np.float32(head_sum / denom)


def k_check_logits(dists: np.ndarray, dim: int) -> np.ndarray:
    """(65536 - dist) / sqrt(dim) in f32 (nsw.rs:282-286)."""
    d = np.asarray(dists, dtype=np.float32)
    return ((np.float32(65536.0) - d) / np.float32(np.sqrt(np.float32(dim)))).astype(np.float32)


def k_check_early_stoppable(dists_sorted: np.ndarray, dim: int, attn_mass_threshold: float) -> bool:
    """nsw.rs:280-296 on the ascending distances of the current best H."""
    logits = k_check_logits(dists_sorted, dim)
    alpha = fit_alpha_from_logits(logits, K_CHECK_MIN_RANK)
    if alpha is None:
        return False
    mass = estimate_top_h_mass(logits, len(logits), alpha)
    if mass is None:
        return False
    return bool(mass >= np.float32(attn_mass_threshold))


def k_check_budget(dists_sorted: np.ndarray, dim: int, k_check_seq: Sequence[int],
                   attn_mass_threshold: float) -> int:
    """The number of best rows worth attending to: the first H of k_check_seq (H < ef, taken
    in order, nsw.rs:302-303,377-378) whose top-H passes the k-check, else ef = len(dists).
    The reference runs this inside its graph search on the H best found so far; on the exact,
    complete result list those are the first H entries."""
    ef = len(dists_sorted)
    for h in k_check_seq:
        if h >= ef:
            break
        if k_check_early_stoppable(np.asarray(dists_sorted)[:h], dim, attn_mass_threshold):
            return int(h)
    return ef


# --------------------------------------------------------------------------
# Checking aid for the HIP select's internal histogram (no reference
# counterpart): the 12-bit monotone bucket of an ordering key.
# --------------------------------------------------------------------------


def coarse_bucket(scores: np.ndarray, mode: int) -> np.ndarray:
    """Bucket (smaller = better) of each score: positive scores in [2^-20, 2^20) get
    8 buckets per binade, clamped outside; negative scores two per binade."""
    s = np.asarray(scores, dtype=np.float32)
    if mode == MODE_REF_DIST:
        d = ref_dist(s)
        s = (np.float32(65536.0) - d).astype(np.float32)
    s = (s + np.float32(0.0)).astype(np.float32)
    b = s.view(np.uint32)
    mag = b & np.uint32(0x7FFFFFFF)
    binades, sub_bits = 40, 3
    pos_buckets = np.uint32(binades << sub_bits)
    lo = np.uint32((127 - 20) << 23)
    hi = np.uint32(((127 - 20 + binades) << 23) - 1)
    m = np.clip(mag, lo, hi)
    pos = (pos_buckets - np.uint32(1)) - ((m - lo) >> np.uint32(23 - sub_bits))
    neg = pos_buckets + (mag >> np.uint32(22))
    return np.where((b >> np.uint32(31)) != 0, neg, pos).astype(np.uint32)
