"""PQ baseline on the HBM store: codebook training, encoding and the search
pipeline ADC scan -> candidates -> exact bf16 rerank.

The reference's PQ baseline directory (evaluation/impl/pqcache) is empty, so
this follows the benchmark configuration only: M subspaces x 256 centroids,
8-bit codes, per-query fp32 lookup tables, 4096 candidates reranked to top-k.
Training and encoding are one-off preparation and use torch ops on the device;
everything a query touches runs in libdiffcache_hip.so.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _hip as hip


def train_codebooks(keys: torch.Tensor, m: int, iters: int = 8, seed: int = 0,
                    n_centroids: int = 256) -> torch.Tensor:
    """Seeded Lloyd k-means per subspace.  keys (n, hd) on the GPU ->
    (m, n_centroids, hd/m) fp32.  Initial centroids are a seeded sample of the
    keys; an empty cell keeps its centroid."""
    x = keys.float()
    n, hd = x.shape
    ds = hd // m
    g = torch.Generator(device=x.device).manual_seed(seed)
    books = torch.empty((m, n_centroids, ds), dtype=torch.float32, device=x.device)
    for j in range(m):
        xs = x[:, j * ds:(j + 1) * ds].contiguous()
        c = xs[torch.randint(0, n, (n_centroids,), generator=g, device=x.device)].clone()
        for _ in range(iters):
            a = torch.cdist(xs, c).argmin(dim=1)
            sums = torch.zeros_like(c).index_add_(0, a, xs)
            cnt = torch.bincount(a, minlength=n_centroids).to(xs.dtype)
            nz = cnt > 0
            c[nz] = sums[nz] / cnt[nz, None]
        books[j] = c
    return books


def encode(keys: torch.Tensor, books: torch.Tensor, chunk: int = 1 << 18) -> torch.Tensor:
    """keys (n, hd) bf16/fp32, books (m, 256, ds) -> codes (n, m) uint8: nearest
    centroid by squared L2 per subspace."""
    m, nc, ds = books.shape
    n = keys.shape[0]
    codes = torch.empty((n, m), dtype=torch.uint8, device=keys.device)
    for s in range(0, n, chunk):
        x = keys[s:s + chunk].float()
        for j in range(m):
            d = torch.cdist(x[:, j * ds:(j + 1) * ds].contiguous(), books[j])
            codes[s:s + chunk, j] = d.argmin(dim=1).to(torch.uint8)
    return codes


class PQIndex:
    """Codes and codebooks of every (batch, kv-head) unit over an HBM key store
    (bsz, kv_heads, n, hd); codebooks are shared by the batch elements of a head."""

    def __init__(self, store_k: torch.Tensor, books: torch.Tensor, codes: torch.Tensor,
                 n_cand: int = 4096, topk: int = 1024) -> None:
        b, h, n, hd = store_k.shape
        hip.require(books.shape[0] == h and books.shape[2] == 256 and books.dtype == torch.float32,
                    "books must be (kv_heads, M, 256, hd / M) fp32")
        hip.require(codes.shape == (b * h, n, books.shape[1]) and codes.dtype == torch.uint8,
                    "codes must be (bsz * kv_heads, n, M) uint8")
        self.store_k, self.books, self.codes = store_k, books.contiguous(), codes.contiguous()
        self.b, self.h, self.n, self.hd, self.m = b, h, n, hd, books.shape[1]
        self.n_cand, self.topk = min(n_cand, n), min(topk, n)
        dev = store_k.device
        nu = b * h
        self.ids = torch.empty((nu, self.topk), dtype=torch.int32, device=dev)
        self.ws = hip.alloc_workspace(hip.lib.dc_pq_search_workspace_bytes(nu, n, self.n_cand), dev)
        self._ws_ready = False      # every search leaves the workspace ready for the next one

    @classmethod
    def build(cls, store_k: torch.Tensor, m: int = 32, sample: int = 65536, iters: int = 8,
              seed: int = 0, **kw) -> "PQIndex":
        b, h, n, hd = store_k.shape
        books = torch.stack([train_codebooks(store_k[0, hh, :min(sample, n)], m, iters, seed + hh)
                             for hh in range(h)])
        codes = torch.stack([encode(store_k[bb, hh], books[hh]) for bb in range(b) for hh in range(h)])
        return cls(store_k, books, codes, **kw)

    def search(self, q: torch.Tensor) -> torch.Tensor:
        """q (b*h, hd) bf16 -> int32 ids (b*h, topk), best exact score first.  The returned
        tensor is reused by the next call."""
        lut = hip.pq_build_lut(q, self.books, self.b)
        ids = hip.pq_search(self.store_k, self.codes, lut, q, self.n_cand, self.topk,
                            idx_out=self.ids, workspace=self.ws, state_ready=self._ws_ready)
        self._ws_ready = True
        return ids

    def search_stepwise(self, q: torch.Tensor) -> torch.Tensor:
        """The same search through the separate entry points, with a dense ADC score array:
        dc_pq_adc_scan -> dc_topk_select -> dc_score_gathered_bf16 -> dc_topk_select ->
        dc_compose_idx.  Same ids as search()."""
        lut = hip.pq_build_lut(q, self.books, self.b)
        hist = hip.new_hist(self.b * self.h, q.device)
        adc = hip.pq_adc_scan(self.codes, lut, hist=hist)
        cand = hip.topk_select(adc, self.n_cand, hip.MODE_IP, hip.ORDER_INDEX, hist=hist)
        exact = hip.score_gathered(self.store_k, q, cand)
        pos = hip.topk_select(exact, self.topk, hip.MODE_IP, hip.ORDER_BEST)
        return hip.compose_idx(cand, pos)
