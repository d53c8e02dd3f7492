#!/usr/bin/env python3
"""Benchmark of the decode-time retrieval path on one MI355X.

Workload (default): benchmark configuration 3 -- a full 32-layer Llama-3-8B-shaped
decode step, batch 8, context 131072 per sequence, 32 query / 8 kv heads,
head_dim 128, bf16 K/V resident in HBM (~137 GB), top-k 2048 plus 4 sink tokens
and a 64-token recent window.  One "step" = for every layer: score the whole
retrieval region with the GQA-mean query, select the exact top-k, run the
gathered attention (including the current token's k/v).  Inputs are synthetic
and already in HBM when the timed region starts.

By default the scan reads the 8-bit sketch of the keys and rescans the rows that can
still reach the top-k from the bf16 keys (same ids); --scan bf16 streams the bf16
keys themselves.

Prints ONE JSON line.  `value` is the latency of one whole decode step in
microseconds (lower is better); `roofline` describes the scan kernel (bytes it must
stream per launch over its measured duration, against the 8 TB/s HBM peak);
`cpu_baseline` is the C restatement of the reference's exact scan timed on this
machine's host cores.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes one scan launch of config 3 moves, from rocprofv3 FETCH_SIZE and WRITE_SIZE scaled
# by a known-size copy kernel (the figures and commands are kept with the other profile
# summaries of this repository): counts x 2 KiB read + counts x 1 KiB written.
SCAN_TRAFFIC_BYTES_C3 = {"sketch": 524_722 * 2048 + 13_249 * 1024,
                         "bf16": 1_053_933 * 2048 + 12_570 * 1024}

CONFIGS = {
    # name: layers, batch, q heads, kv heads, hd, context, budget, sinks, recent
    "c3": dict(layers=32, batch=8, hq=32, hkv=8, hd=128, ctx=131072, budget=2048, sink=4, recent=64,
               desc="config3: 32-layer Llama-3-8B-shaped decode step, batch 8, ctx 131072, "
                    "32q/8kv heads, hd 128, bf16 K/V in HBM, top-k 2048 + 4 sinks + 64 recent"),
    "c2": dict(layers=1, batch=1, hq=32, hkv=8, hd=128, ctx=32768, budget=1024, sink=4, recent=64,
               desc="config2: one Llama-3-8B-shaped decode layer, batch 1, ctx 32768, "
                    "top-k 1024 + 4 sinks + 64 recent"),
    "c5": dict(layers=32, batch=1, hq=32, hkv=8, hd=128, ctx=1048576, budget=4096, sink=4, recent=64,
               desc="config5: 32 layers, batch 1, ctx 1048576, top-k 4096 + 4 sinks + 64 recent"),
}


def algorithmic_bytes_per_unit(n_region: int, attended: int, group: int, hd: int) -> int:
    """K streamed once + gathered K and V rows + q in / out (bf16)."""
    return n_region * hd * 2 + 2 * attended * hd * 2 + group * hd * 2 * 2


def make_layer(torch, cfg, layer: int, cfg_id: int, dev, k, v):
    """Synthetic K, V, q, new k/v of one layer, generated on the device into the
    layer's views k, v of the store.  Seed = 1000 * config + layer.
    config 2: keys N(0,1) x per-channel log-normal scale, queries N(0,1);
    config 3: the same keys, queries 0.7 * mean of a random 32-key cluster + 0.3 * N(0,1);
    config 5: keys in 256 Gaussian clusters (centres N(0,1), std 0.1), every query head
              aimed at the mean of 1-4 cluster centres."""
    g = torch.Generator(device=dev).manual_seed(1000 * cfg_id + layer)
    b, hkv, hq, hd, n = cfg["batch"], cfg["hkv"], cfg["hq"], cfg["hd"], cfg["ctx"]
    grp = hq // hkv
    v.normal_(generator=g)
    if cfg_id == 5:
        n_cl = 256
        centres = torch.randn((b, hkv, n_cl, hd), generator=g, device=dev)
        k.normal_(generator=g)
        k.mul_(0.1)
        member = torch.randint(0, n_cl, (b, hkv, n), generator=g, device=dev)
        for bi in range(b):
            for hi in range(hkv):     # one unit at a time: 256 MB of fp32 centres per gather
                k[bi, hi].add_(centres[bi, hi][member[bi, hi]].to(torch.bfloat16))
        n_t = torch.randint(1, 5, (b, hq), generator=g, device=dev)
        pick = torch.randint(0, n_cl, (b, hq, 4), generator=g, device=dev)
        use = (torch.arange(4, device=dev).view(1, 1, 4) < n_t.unsqueeze(-1)).float()
        bi = torch.arange(b, device=dev).view(b, 1, 1).expand(b, hq, 4)
        hi = (torch.arange(hq, device=dev) // grp).view(1, hq, 1).expand(b, hq, 4)
        target = (centres[bi, hi, pick] * use.unsqueeze(-1)).sum(2) / n_t.unsqueeze(-1).float()
        q = (target + 0.1 * torch.randn((b, hq, hd), generator=g, device=dev)).to(torch.bfloat16)
    else:
        k.normal_(generator=g)
        # per-channel log-normal scale (sigma 1), one vector per kv head: outlier channels
        scale = torch.exp(torch.randn((1, hkv, 1, hd), generator=g, device=dev)).to(torch.bfloat16)
        k.mul_(scale)
        if cfg_id == 2:
            q = torch.randn((b, hq, hd), generator=g, device=dev).to(torch.bfloat16)
        else:
            # queries: 0.7 * mean of a random 32-key cluster + 0.3 * N(0,1), per query head
            pick = torch.randint(0, n, (b, hq, 32), generator=g, device=dev)
            bi = torch.arange(b, device=dev).view(b, 1, 1).expand(b, hq, 32)
            hi = (torch.arange(hq, device=dev) // grp).view(1, hq, 1).expand(b, hq, 32)
            centre = k[bi, hi, pick].float().mean(dim=2)
            q = (0.7 * centre + 0.3 * torch.randn((b, hq, hd), generator=g, device=dev)).to(torch.bfloat16)
    new_k = torch.randn((b, hkv, hd), generator=g, device=dev).to(torch.bfloat16)
    new_v = torch.randn((b, hkv, hd), generator=g, device=dev).to(torch.bfloat16)
    return k, v, q.contiguous(), new_k, new_v


def cpu_baseline(torch, cfg, layers_data, target_s: float = 10.0):
    """The C restatement of the reference's exact-scan path, timed on this box's
    host cores on a bounded sample: layer 0, batch element 0 (hkv units), one
    thread per unit like rayon's fan-out, repeated until ~target_s of work."""
    import numpy as np
    from oracle import cpu_ref
    k, v, q, nk, nv = layers_data[0]
    hkv, hq, hd, n = cfg["hkv"], cfg["hq"], cfg["hd"], cfg["ctx"]
    grp = hq // hkv

    def host(t):
        return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)

    k0, v0 = host(k[0]), host(v[0])                       # (hkv, n, hd)
    q0 = host(q[0]).reshape(hkv, grp, hd)
    nk0, nv0 = host(nk[0]), host(nv[0])
    cores = os.cpu_count() or 1
    # the GPU box gives one GPU's share of the host: 16 cores
    threads = min(hkv, cores, 16)
    cpu_ref.lib()
    reps, total = 0, 0.0
    t_first = None
    while total < target_s and reps < 20000:
        t0 = time.perf_counter()
        cpu_ref.decode_layer(q0, k0, v0, cfg["budget"], cfg["sink"], cfg["recent"], n_ctx=n,
                             new_k_u16=nk0, new_v_u16=nv0, n_threads=threads, want_ids=False)
        dt = time.perf_counter() - t0
        t_first = dt if t_first is None else t_first
        total += dt
        reps += 1
    per_sample = total / reps
    units_total = cfg["layers"] * cfg["batch"] * hkv
    step_us = per_sample * (units_total / hkv) * 1e6
    return {
        "value": step_us, "unit": "us", "cores": threads, "kind": "port",
        "sample": (f"oracle/cpu_ref.c decode_layer on layer 0, batch element 0 ({hkv} units x {n} rows), "
                   f"{threads} threads, mean of {reps} runs = {per_sample * 1e3:.1f} ms; scaled x"
                   f"{units_total // hkv} to the full step ({cfg['layers']} layers x batch {cfg['batch']}); "
                   f"host reports {cores} cpus"),
    }


def make_pq_index(torch, hip, dev, store=None):
    """Benchmark configuration 4: 8 kv heads x 1,048,576 keys ~ N(0,1), hd 128, M 32 x 256 centroids
    from seeded k-means on a 65,536-key sample, 8-bit codes, 4096 candidates, top-k 1024.
    Returns (index, key store, queries).  `store`: a (1, 8, 2^20, 128) bf16 buffer to fill."""
    from diffcache_amd.pq import PQIndex
    h, n, hd, m, n_cand, topk = 8, 1 << 20, 128, 32, 4096, 1024
    g = torch.Generator(device=dev).manual_seed(4000)
    if store is None:
        store = torch.empty((1, h, n, hd), dtype=torch.bfloat16, device=dev)
    store.normal_(generator=g)
    q = torch.randn((h, hd), generator=g, device=dev).to(torch.bfloat16)
    index = PQIndex.build(store, m=m, sample=65536, iters=8, seed=4000, n_cand=n_cand, topk=topk)
    return index, store, q


def run_pq(args, torch, hip, dev) -> int:
    """Benchmark configuration 4: PQ baseline, one layer, 8 kv heads x 1,048,576 keys, M 32 x 8-bit
    codes, ADC scan -> 4096 candidates -> exact bf16 rerank to top-k 1024."""
    h, n, hd, m, n_cand, topk = 8, 1 << 20, 128, 32, 4096, 1024
    t_gen = time.perf_counter()
    index, store, q = make_pq_index(torch, hip, dev)
    torch.cuda.synchronize()
    t_gen = time.perf_counter() - t_gen
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(args.steps)]

    def step(e=None):
        if args.stepwise:
            return step_stepwise(e)
        lut = hip.pq_build_lut(q, index.books, 1)
        ids = hip.pq_search(store, index.codes, lut, q, n_cand, topk, idx_out=index.ids,
                            workspace=index.ws, state_ready=index._ws_ready, scan_events=e)
        index._ws_ready = True
        return ids

    hist = hip.new_hist(h, dev)

    def step_stepwise(e=None):
        # the separate entry points, with a dense ADC score array
        lut = hip.pq_build_lut(q, index.books, 1)
        hist.zero_()
        if e is not None:
            e[0].record()
        adc = hip.pq_adc_scan(index.codes, lut, hist=hist)
        if e is not None:
            e[1].record()
        cand = hip.topk_select(adc, n_cand, hip.MODE_IP, hip.ORDER_INDEX, hist=hist)
        exact = hip.score_gathered(store, q, cand)
        pos = hip.topk_select(exact, topk, hip.MODE_IP, hip.ORDER_BEST)
        return hip.compose_idx(cand, pos)

    for e in ev:            # events must exist before the library records them
        e[0].record()
        e[1].record()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        step(ev[s])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    scan_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / len(ev)
    scan_bytes = h * n * m
    ach = scan_bytes / (scan_ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "pq_adc_search_latency_us", "value": ms * 1e3, "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8 codes, fp32 tables, bf16 rerank",
        "data": "synthetic",
        "config": {"workload": "config4: PQ baseline, 8 kv heads x 1048576 keys, hd 128, M 32 x 256 centroids, "
                               "ADC scan -> 4096 candidates -> exact rerank to top-k 1024"},
        "roofline": {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": ach / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "pq_adc_kernel<32>" if args.stepwise else "pq_prune_kernel<32>",
                     "algorithmic_bytes_per_launch": scan_bytes, "avg_launch_us": scan_ms * 1e3},
        "cpu_baseline": None, "setup_s": t_gen}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS) + ["c4"])
    ap.add_argument("--mode", default="ref_dist", choices=["ref_dist", "ip"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--split", action="store_true",
                    help="issue the scan, select and attention as separate C calls with an event between "
                         "each (per-stage breakdown) instead of one dc_decode_layer call per layer")
    ap.add_argument("--event-stride", type=int, default=4,
                    help="one-call path: time the scan kernel in place on every N-th layer")
    ap.add_argument("--streams", type=int, default=1,
                    help="pipeline the batch as this many independent micro-batches, one HIP stream each "
                         "(the units of a layer are independent, so one micro-batch's select/attention "
                         "overlaps the other's scan)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="before the steps, run a plain elementwise kernel that reads 1 GiB and writes "
                         "1 GiB three times (a known-size reference for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--dense", action="store_true",
                    help="materialise the fp32 scores (dc_score_bf16 + dc_topk_select) instead of the "
                         "streaming score + select")
    ap.add_argument("--stepwise", action="store_true",
                    help="config c4 only: the PQ search through the separate entry points (dense ADC "
                         "score array) instead of dc_pq_search_bf16")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one decode step (all layers) in a HIP graph and time its replays; "
                         "reported as graph_step_us next to the eager figure")
    ap.add_argument("--scan", default=None, choices=["sketch", "bf16"],
                    help="sketch (default): scan the 8-bit sketch of the keys and rescore the surviving "
                         "rows exactly from the bf16 keys (same ids, half the bytes); bf16: stream the "
                         "bf16 keys themselves")
    args = ap.parse_args()
    other_path = args.dense or args.split or args.streams != 1
    if args.scan == "sketch" and other_path:
        print("bench.py: --scan sketch goes with the default one-call path only", file=sys.stderr)
        return 2
    args.sketch = (args.scan or ("bf16" if other_path else "sketch")) == "sketch"
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              "use --gpus 1", file=sys.stderr)
        return 2

    import torch
    from diffcache_amd import _hip as hip

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.config == "c4":
        return run_pq(args, torch, hip, dev)
    cfg = CONFIGS[args.config]
    cfg_id = {"c2": 2, "c3": 3, "c5": 5}[args.config]
    mode = hip.MODE_REF_DIST if args.mode == "ref_dist" else hip.MODE_IP
    L, b, hq, hkv, hd, n = cfg["layers"], cfg["batch"], cfg["hq"], cfg["hkv"], cfg["hd"], cfg["ctx"]
    grp = hq // hkv
    n_units = b * hkv
    sink, recent, budget = cfg["sink"], cfg["recent"], cfg["budget"]
    lo, hi = sink, n - recent
    region = hi - lo
    k_eff = min(budget, region)
    attended = k_eff + sink + recent + 1

    t_gen = time.perf_counter()
    # One allocation holds every layer's keys and one every layer's values, as the KV
    # store of diffcache_amd.DiffCache does: scans of a single large allocation run
    # about 3 % faster on MI355X than scans of per-layer allocations.
    vslab = torch.empty((L, b, hkv, n, hd), dtype=torch.bfloat16, device=dev)
    kslab = torch.empty((L, b, hkv, n, hd), dtype=torch.bfloat16, device=dev)
    layers = [make_layer(torch, cfg, l, cfg_id, dev, kslab[l], vslab[l]) for l in range(L)]
    sketches = None
    if args.sketch:
        # the sketch of the retrieval region of every layer (prefill-time work, untimed)
        cslab = torch.empty((L, b, hkv, n, hd), dtype=torch.uint8, device=dev)
        sketches = [hip.Sketch(kslab[l], codes=cslab[l]).build(kslab[l], lo, hi - lo) for l in range(L)]
    torch.cuda.synchronize()
    t_gen = time.perf_counter() - t_gen

    if args.streams < 1 or b % args.streams != 0:
        print("bench.py: --streams must divide the batch size", file=sys.stderr)
        return 2
    args.fused = not args.split

    class Pipe:
        """One micro-batch: its slice of every layer's tensors, its buffers, its stream."""

        def __init__(self, b0, b1):
            self.nb = b1 - b0
            self.n_units = self.nb * hkv
            self.layers = [(k[b0:b1], v[b0:b1], q[b0:b1], nk[b0:b1], nv[b0:b1]) for (k, v, q, nk, nv) in layers]
            nu = self.n_units
            self.scores = torch.empty((nu, region), dtype=torch.float32, device=dev) if args.dense else None
            self.idx = torch.empty((nu, budget), dtype=torch.int32, device=dev)
            self.out = torch.empty((self.nb, hq, hd), dtype=torch.bfloat16, device=dev)
            self.hist = hip.new_hist(nu, dev)
            self.ws_topk = hip.alloc_workspace(hip.lib.dc_topk_workspace_bytes(nu, region, budget), dev)
            self.ws_attn = hip.alloc_workspace(hip.lib.dc_attn_workspace_bytes(nu, grp, hd, attended), dev)
            self.ws_layer = hip.alloc_workspace(hip.layer_workspace_bytes(nu, region, budget, grp, hd, attended), dev)
            self.ws_sel = hip.alloc_workspace(hip.score_select_workspace_bytes(nu, region, budget), dev)
            self.stream = torch.cuda.Stream(device=dev)     # default priority
            self.clean = False

        def layer(self, l, ev=None, wait_for=None):
            k, v, q, nk, nv = self.layers[l]
            nu = self.n_units
            if wait_for is not None:
                # scans of different micro-batches take turns: this layer call starts once the
                # other micro-batch's scan has finished, so its select/attention overlap our scan
                torch.cuda.current_stream().wait_event(wait_for)
            if args.fused:
                hip.decode_layer(q, k, v, sink, hi, recent, budget, self.scores, self.idx, self.out,
                                 self.ws_layer, nk, nv, mode=mode, order=hip.ORDER_ANY,
                                 select_state_ready=self.clean and not args.dense,
                                 scan_events=None if ev is None or l % stride else
                                 (ev[4 * l], ev[4 * l + 1]),
                                 sketch=None if sketches is None else sketches[l])
                self.clean = True
                return
            if args.dense:
                self.hist.zero_()
            elif not self.clean:
                hip.select_state_init(nu, region, budget, self.ws_sel)
                self.clean = True   # dc_sparse_select(reinit) keeps it so from here on
            if ev is not None:
                ev[4 * l + 0].record()
            if args.dense:
                hip.score(k, q, lo, region, mode, q_group=grp, scores=self.scores, hist=self.hist)
            else:
                hip.score_prune(k, q, lo, region, budget, self.ws_sel, mode, q_group=grp)
            if ev is not None:
                ev[4 * l + 1].record()
            if args.dense:
                hip.topk_select(self.scores, budget, mode, hip.ORDER_ANY, hist=self.hist, idx_out=self.idx,
                                workspace=self.ws_topk)
            else:
                hip.sparse_select(self.idx, nu, region, budget, self.ws_sel, mode, hip.ORDER_ANY, reinit=True)
            if ev is not None:
                ev[4 * l + 2].record()
            hip.gather_attn(q, k, v, self.idx, k_eff, lo, sink, hi, recent, nk, nv, out=self.out,
                            workspace=self.ws_attn)
            if ev is not None:
                ev[4 * l + 3].record()

    per = b // args.streams
    pipes = [Pipe(i * per, (i + 1) * per) for i in range(args.streams)]

    def new_events(count):
        return [torch.cuda.Event(enable_timing=True) for _ in range(count)]

    stride = 1 if args.streams > 1 else args.event_stride

    def step(evs):
        """One decode step: every layer in order; the micro-batches are independent of
        each other and each runs its layers in order on its own stream.  With several
        streams the scans are chained through their end events so that only one scan
        streams from HBM at a time."""
        prev_scan_end = None
        for l in range(L):
            for pi, pipe in enumerate(pipes):
                with torch.cuda.stream(pipe.stream):
                    pipe.layer(l, evs[pi], wait_for=prev_scan_end if args.streams > 1 else None)
                if args.streams > 1:
                    prev_scan_end = evs[pi][4 * l + 1]

    if args.pmc_calibration:
        ca = torch.ones((256 << 20,), dtype=torch.float32, device=dev)      # 1 GiB
        cb = torch.empty_like(ca)
        for _ in range(3):
            torch.add(ca, 1.0, out=cb)
        torch.cuda.synchronize()
        del ca, cb

    events = [[new_events(4 * L) for _ in pipes] for _ in range(args.steps + 1)]
    # torch creates the native event on first record; the C side needs the handle
    for per_step in events:
        for pi, evs in enumerate(per_step):
            for e in evs:
                e.record(pipes[pi].stream)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step(events[-1])
    torch.cuda.synchronize()
    events = events[:-1]
    # one more event after every step on the first micro-batch's stream: the spread of the
    # step times (with several streams the boundaries are only approximate)
    marks = new_events(args.steps + 1)
    for e in marks:
        e.record(pipes[0].stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks[0].record(pipes[0].stream)
    for s in range(args.steps):
        step(events[s])
        marks[s + 1].record(pipes[0].stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    per_step_us = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 for i in range(args.steps))

    def pct(p):
        return per_step_us[min(len(per_step_us) - 1, int(p * len(per_step_us)))]

    # Small configurations fit in the 256 MB Infinity Cache, so the loop above measures a
    # warm cache.  Cold: a 1 GiB buffer is overwritten before every step (untimed) and each
    # step is timed on its own.
    cold_step_us = None
    if n_units * L * region * hd * 2 < (512 << 20) and args.streams == 1:
        flush = torch.empty((1 << 30,), dtype=torch.uint8, device=dev)
        c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        cold = []
        for s_i in range(min(args.steps, 30)):
            with torch.cuda.stream(pipes[0].stream):
                flush.fill_(s_i & 0xff)
                c0.record()
            step(events[s_i])
            with torch.cuda.stream(pipes[0].stream):
                c1.record()
            torch.cuda.synchronize()
            cold.append(c0.elapsed_time(c1) * 1e3)
        cold.sort()
        cold_step_us = cold[len(cold) // 2]
        del flush

    graph_step_us = None
    if args.graph and args.streams == 1 and args.fused:
        # every call of the step only enqueues kernels on the stream, so the whole step can be
        # captured; the select state is already "left ready" by the eager steps above
        cap_stream = pipes[0].stream
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap_stream):
            for l in range(L):
                pipes[0].layer(l, None)
        torch.cuda.synchronize()
        for _ in range(max(args.warmup, 1)):
            graph.replay()
        torch.cuda.synchronize()
        tg = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_step_us = (time.perf_counter() - tg) * 1e6 / args.steps

    # per-kernel durations from the events of the timed region
    stage_us = None
    score_ms = None
    flat = [e for per_step in events for e in per_step]
    if args.fused:
        sc = [e[4 * l].elapsed_time(e[4 * l + 1]) for e in flat for l in range(0, L, stride)]
        score_ms = sum(sc) / len(sc)
        stage_us = {"score": score_ms * 1e3, "timed_launches": len(sc)}
    else:
        sc = [e[4 * l].elapsed_time(e[4 * l + 1]) for e in flat for l in range(L)]
        se = [e[4 * l + 1].elapsed_time(e[4 * l + 2]) for e in flat for l in range(L)]
        at = [e[4 * l + 2].elapsed_time(e[4 * l + 3]) for e in flat for l in range(L)]
        score_ms = sum(sc) / len(sc)
        stage_us = {"score": score_ms * 1e3, "select": sum(se) / len(se) * 1e3,
                    "attn": sum(at) / len(at) * 1e3, "timed_launches": len(sc)}

    unit_bytes = algorithmic_bytes_per_unit(region, k_eff + sink + recent, grp, hd)
    step_bytes = unit_bytes * n_units * L
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    # what the chosen path must move: the sketch scan reads hd bytes per key, not 2*hd
    step_path_bytes = step_bytes - (n_units * L * region * hd if args.sketch else 0)
    # bytes one scan launch has to stream: the bf16 K rows, or their one-byte-per-element sketch
    score_bytes = (n_units // args.streams) * region * hd * (1 if args.sketch else 2)
    roofline = {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": None,
                "traffic": None,
                "kernel": "sketch_prune_kernel<128>" if args.sketch else
                          "score_kernel<128>" if args.dense else "score_prune_kernel<128>",
                "algorithmic_bytes_per_launch": score_bytes}
    if args.config == "c3" and args.streams == 1 and not args.dense and args.mode == "ref_dist":
        roofline["traffic"] = SCAN_TRAFFIC_BYTES_C3["sketch" if args.sketch else "bf16"]
    if score_ms is not None:
        ach = score_bytes / (score_ms * 1e-3) / 1e9
        roofline.update(achieved=ach, frac=ach / HBM_PEAK_GBPS, avg_launch_us=score_ms * 1e3)

    result = {
        "metric": "decode_step_retrieval_sparse_attn_latency_us",
        "value": ms_per_step * 1e3,
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": cfg["desc"], "key_mode": args.mode, "streams": args.streams,
                   "call_path": ("dc_decode_layer" + (" (dense scores)" if args.dense else
                                                      " (sketch scan + exact rescoring)" if args.sketch else "")
                                 if args.fused else
                                 "dc_score_bf16/dc_topk_select/dc_gather_attn_bf16" if args.dense else
                                 "dc_select_state_init/dc_score_prune_bf16/dc_sparse_select/dc_gather_attn_bf16")},
        # bytes of the reference's exact algorithm per step (every bf16 key once + the gathered
        # K/V rows + q in/out) over the measured time.  With the sketch scan the path streams
        # one byte per key element instead of two, so this rate can exceed the HBM peak; the
        # bytes this call path has to move are in step_path_bytes.
        "step_hbm_gbps": step_gbps,
        "step_hbm_frac": step_gbps / HBM_PEAK_GBPS,
        "step_algorithmic_bytes": step_bytes,
        "step_path_bytes": step_path_bytes,
        "step_path_gbps": step_path_bytes / (ms_per_step * 1e-3) / 1e9,
        "keys_scored_per_s": n_units * L * region / (ms_per_step * 1e-3),
        "step_us_p10_p50_p90": [pct(0.10), pct(0.50), pct(0.90)],
        "graph_step_us": graph_step_us,
        "cold_cache_step_us_median": cold_step_us,
        "stage_us_per_layer": stage_us,
        "roofline": roofline,
        "setup_s": t_gen,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch, cfg, layers)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
