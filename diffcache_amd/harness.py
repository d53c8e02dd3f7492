"""Decode-step harness around ``DiffCache``: a Llama-shaped decoder with random weights.

The reference drives its KV cache from ``BaseModel.layer_decode``
(src/diffcache/base.py:116-155): RMSNorm, QKV projection and RoPE before the
cache query, attention over the assembled rows, then the output projection and
the MLP.  This module does the same around ``DiffCache.decode_attention`` with
synthetic weights and a synthetic prompt cache (hub checkpoints are not available
offline), so that the retrieval path can be timed inside a whole decode step:
tokens per second with the dense parts of the model in the loop.

    python -m diffcache_amd.harness --layers 32 --batch 8 --ctx 131072 --steps 20

Everything dense is plain PyTorch (hipBLASLt GEMMs); only the cache calls go to
the HIP library.
"""
from __future__ import annotations

import argparse
import json
import math
import time
from typing import List, Optional

import torch

from .kvcache.diffcache import DiffCache


class SyntheticLlama:
    """Llama-3-style decoder stack (pre-norm, GQA, RoPE, SwiGLU) with random bf16 weights."""

    def __init__(self, num_layers: int = 32, hidden: int = 4096, num_q_heads: int = 32,
                 num_kv_heads: int = 8, head_dim: int = 128, intermediate: int = 14336,
                 rope_theta: float = 500000.0, device: str = "cuda", seed: int = 0) -> None:
        self.num_layers, self.hidden = num_layers, hidden
        self.hq, self.hkv, self.hd = num_q_heads, num_kv_heads, head_dim
        self.inter, self.rope_theta = intermediate, rope_theta
        self.device = torch.device(device)
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(rows: int, cols: int) -> torch.Tensor:
            t = torch.randn((rows, cols), generator=g, device=self.device, dtype=torch.float32)
            return (t / math.sqrt(cols)).to(torch.bfloat16)

        qkv_out = (self.hq + 2 * self.hkv) * head_dim
        self.wqkv: List[torch.Tensor] = [w(qkv_out, hidden) for _ in range(num_layers)]
        self.wo: List[torch.Tensor] = [w(hidden, self.hq * head_dim) for _ in range(num_layers)]
        self.wgu: List[torch.Tensor] = [w(2 * intermediate, hidden) for _ in range(num_layers)]
        self.wd: List[torch.Tensor] = [w(hidden, intermediate) for _ in range(num_layers)]
        self.norm1 = [torch.ones(hidden, device=self.device, dtype=torch.bfloat16) for _ in range(num_layers)]
        self.norm2 = [torch.ones(hidden, device=self.device, dtype=torch.bfloat16) for _ in range(num_layers)]
        inv = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, device=self.device, dtype=torch.float32) / head_dim))
        self._inv_freq = inv

    def weight_bytes(self) -> int:
        per = sum(t.numel() for t in (self.wqkv[0], self.wo[0], self.wgu[0], self.wd[0]))
        return per * 2 * self.num_layers

    @staticmethod
    def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * weight

    def rope(self, x: torch.Tensor, pos) -> torch.Tensor:
        """x (b, heads, hd): rotate-half RoPE at one position (an int, or a one-element
        device tensor so that a captured graph can be replayed at other positions)."""
        ang = (pos.float() if isinstance(pos, torch.Tensor) else float(pos)) * self._inv_freq
        cos = torch.cat([ang.cos(), ang.cos()]).to(x.dtype)
        sin = torch.cat([ang.sin(), ang.sin()]).to(x.dtype)
        half = x.shape[-1] // 2
        rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
        return x * cos + rot * sin

    def qkv(self, layer: int, x: torch.Tensor, pos):
        """x (b, hidden) -> q (b, hq, hd), k (b, hkv, hd), v (b, hkv, hd) with RoPE on q and k."""
        b = x.shape[0]
        h = self.rmsnorm(x, self.norm1[layer])
        y = h @ self.wqkv[layer].t()
        q, k, v = torch.split(y, [self.hq * self.hd, self.hkv * self.hd, self.hkv * self.hd], dim=-1)
        q = self.rope(q.view(b, self.hq, self.hd), pos)
        k = self.rope(k.view(b, self.hkv, self.hd), pos)
        return q.contiguous(), k.contiguous(), v.reshape(b, self.hkv, self.hd).contiguous()

    def post_attention(self, layer: int, x: torch.Tensor, attn: torch.Tensor) -> torch.Tensor:
        """attn (b, hq, hd) -> new residual stream (b, hidden): o_proj + SwiGLU MLP."""
        b = x.shape[0]
        x = x + attn.reshape(b, self.hq * self.hd) @ self.wo[layer].t()
        h = self.rmsnorm(x, self.norm2[layer])
        gu = h @ self.wgu[layer].t()
        gate, up = gu[:, :self.inter], gu[:, self.inter:]
        return x + (torch.nn.functional.silu(gate) * up) @ self.wd[layer].t()

    def decode_step(self, cache: DiffCache, x: torch.Tensor) -> torch.Tensor:
        """One token for every sequence of the batch: x (b, hidden) -> (b, hidden)."""
        pos = cache.seq_len(0)
        for layer in range(self.num_layers):
            q, k, v = self.qkv(layer, x, pos)
            attn = cache.decode_attention(layer, q, k.unsqueeze(1), v.unsqueeze(1))
            x = self.post_attention(layer, x, attn)
        return x


class GraphedDecoder:
    """The reference's arrangement (base.py:116-155): per layer one captured graph for what
    precedes the cache query (norm, QKV, RoPE) and one for what follows the attention
    (o_proj, MLP), with the cache call in between, which only enqueues kernels."""

    def __init__(self, model: SyntheticLlama, cache: DiffCache, batch: int) -> None:
        self.model, self.cache = model, cache
        dev, dt = model.device, torch.bfloat16
        self.x = torch.zeros((batch, model.hidden), device=dev, dtype=dt)
        self.q = torch.zeros((batch, model.hq, model.hd), device=dev, dtype=dt)
        self.k = torch.zeros((batch, 1, model.hkv, model.hd), device=dev, dtype=dt)
        self.v = torch.zeros((batch, 1, model.hkv, model.hd), device=dev, dtype=dt)
        self.attn = torch.zeros((batch, model.hq, model.hd), device=dev, dtype=dt)
        self.pos = torch.zeros((1,), device=dev, dtype=torch.int64)
        self.pre: List[torch.cuda.CUDAGraph] = []
        self.post: List[torch.cuda.CUDAGraph] = []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):               # warm the GEMM paths up before capture
            for layer in range(model.num_layers):
                self._pre(layer)
                self._post(layer)
        torch.cuda.current_stream().wait_stream(side)
        self.x.zero_()
        for layer in range(model.num_layers):
            g1, g2 = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
            with torch.cuda.graph(g1):
                self._pre(layer)
            with torch.cuda.graph(g2):
                self._post(layer)
            self.pre.append(g1)
            self.post.append(g2)
        self.x.zero_()

    def _pre(self, layer: int) -> None:
        q, k, v = self.model.qkv(layer, self.x, self.pos)
        self.q.copy_(q)
        self.k.copy_(k.unsqueeze(1))
        self.v.copy_(v.unsqueeze(1))

    def _post(self, layer: int) -> None:
        self.x.copy_(self.model.post_attention(layer, self.x, self.attn))

    def decode_step(self, x: torch.Tensor) -> torch.Tensor:
        self.x.copy_(x)
        self.pos.fill_(self.cache.seq_len(0))
        for layer in range(self.model.num_layers):
            self.pre[layer].replay()
            self.cache.decode_attention(layer, self.q, self.k, self.v, out=self.attn)
            self.post[layer].replay()
        return self.x


def synthetic_prompt_cache(cache: DiffCache, ctx: int, seed: int = 1) -> None:
    """Fill every layer of the cache with a random prompt of ``ctx`` tokens (keys with
    per-channel log-normal scales, as in the benchmark's configuration 3)."""
    dev = cache.device
    g = torch.Generator(device=dev).manual_seed(seed)
    b, hkv, hd = cache.batch_size, cache.num_kv_heads, cache.head_dim
    for layer in range(cache.num_layers):
        k = torch.randn((b, ctx, hkv, hd), generator=g, device=dev, dtype=torch.bfloat16)
        k.mul_(torch.exp(torch.randn((1, 1, hkv, hd), generator=g, device=dev)).to(torch.bfloat16))
        v = torch.randn((b, ctx, hkv, hd), generator=g, device=dev, dtype=torch.bfloat16)
        cache.prefill_update_kv_cache(k, v, layer)
        del k, v


def run(layers: int, batch: int, ctx: int, budget: int, steps: int, warmup: int, key_sketch: bool,
        graphs: bool = True, hidden: int = 4096, hq: int = 32, hkv: int = 8, hd: int = 128, inter: int = 14336,
        sink: int = 4, recent: int = 64) -> dict:
    dev = "cuda"
    model = SyntheticLlama(layers, hidden, hq, hkv, hd, inter, device=dev)
    room = warmup + steps + 8
    cache = DiffCache(num_layers=layers, batch_size=batch, max_length=ctx + room, num_kv_heads=hkv,
                      num_q_heads=hq, head_dim=hd, retrieval_budget=budget, nsw_m=16, nsw_ef_cons=200,
                      kvbuf_prefix_len=sink, kvbuf_suffix_len=recent, kvbuf_suffix_maxlen=recent + room,
                      attn_mass_threshold=0.9, k_check_seq=[1 << 30],
                      r_sq=[[4.0] * hkv for _ in range(layers)], key_sketch=key_sketch)
    synthetic_prompt_cache(cache, ctx)
    x = torch.randn((batch, hidden), device=dev, dtype=torch.bfloat16)
    dec = GraphedDecoder(model, cache, batch) if graphs else None

    def one_step(t: torch.Tensor) -> torch.Tensor:
        t = dec.decode_step(t) if dec is not None else model.decode_step(cache, t)
        return t / t.float().pow(2).mean(-1, keepdim=True).sqrt().to(t.dtype)   # keep the stream bounded

    for _ in range(warmup):
        x = one_step(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        x = one_step(x)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return {
        "metric": "decode_tokens_per_s_synthetic_llama",
        "value": batch / dt,
        "unit": "tokens/s",
        "ms_per_step": dt * 1e3,
        "config": {"layers": layers, "batch": batch, "ctx": ctx, "budget": budget, "hidden": hidden,
                   "q_heads": hq, "kv_heads": hkv, "head_dim": hd, "intermediate": inter,
                   "key_sketch": key_sketch, "graphs": graphs, "weights": "random bf16",
                   "prompt": "synthetic K/V"},
        "weight_bytes": model.weight_bytes(),
        "finite": bool(torch.isfinite(x.float()).all()),
    }


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--ctx", type=int, default=131072)
    ap.add_argument("--budget", type=int, default=2048)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-sketch", action="store_true", help="stream the bf16 keys instead of the 8-bit sketch")
    ap.add_argument("--eager", action="store_true", help="no captured graphs around the dense halves")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("harness: no GPU visible")
        return 2
    print(json.dumps(run(args.layers, args.batch, args.ctx, args.budget, args.steps, args.warmup,
                         not args.no_sketch, graphs=not args.eager)))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
