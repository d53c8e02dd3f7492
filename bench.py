#!/usr/bin/env python3
"""Benchmark of the decode-time retrieval path on one MI355X.

Headline workload: benchmark configuration 3 -- a full 32-layer Llama-3-8B-shaped decode
step, batch 8, context 131072 per sequence, 32 query / 8 kv heads, head_dim 128, bf16 K/V
resident in HBM (~137 GB), top-k 2048 plus 4 sink tokens and a 64-token recent window.
One "step" = for every layer: score the whole retrieval region with the GQA-mean query,
select the exact top-k, run the gathered attention (including the current token's k/v).
Inputs are synthetic and already in HBM when the timed region starts.

Two scan routes give the same ids: "sketch" (default) scans an 8-bit sketch of the keys
and rescans the rows that can still reach the top-k from the bf16 keys; "bf16" streams
the bf16 keys themselves, which is the byte count of the reference's algorithm
(every key row once).  A default run times both on configuration 3 and, beside it,
configurations 2 (one layer, 32K context), 5 (1M context) and 4 (PQ baseline).

Prints ONE JSON line.  `value` is the latency of one whole decode step of configuration 3
on the default route, in microseconds (lower is better).  `roofline` describes that route's
scan kernel: bytes it must stream per launch over its measured duration, against the
8 TB/s HBM peak (`frac`), and the same duration priced at the two bytes per key element of
the reference's algorithm (`frac_8d`, which can exceed 1 because the sketch reads one).
`routes.bf16` is the same step streaming the bf16 keys; `configs` holds the other
configurations; `cpu_baseline` is the C restatement of the reference's exact scan timed on
this machine's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the dominant kernels, from rocprofv3 FETCH_SIZE and WRITE_SIZE scaled by a
# known-size copy kernel.  Taken when the profile summaries kept with this repository were made,
# not in this run; the figures live in one file that the summaries quote as well.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def profiled_traffic(key: str):
    """HBM bytes per launch of `key` ("c3.sketch", "c3.bf16", "c2.one_kernel") from the tracked
    counter file, or None."""
    try:
        with open(TRAFFIC_FILE) as f:
            e = json.load(f)["kernels"][key]
        return int(e["fetch_counts"] * e["fetch_unit_bytes"] + e["write_counts"] * e["write_unit_bytes"])
    except (OSError, KeyError, ValueError):
        return None


def device_state() -> dict:
    """Clock levels, power and partition modes of the GPU as the driver's sysfs files report them
    (plain file reads; whatever is missing or unreadable is left out).  Read before and after a
    timed loop: the same binary has been seen at two speed levels of the scan on these boxes."""
    import glob
    out = {}
    for card in sorted(glob.glob("/sys/class/drm/card[0-9]*/device")):
        if not os.path.exists(os.path.join(card, "pp_dpm_sclk")) and \
                not os.path.exists(os.path.join(card, "current_compute_partition")):
            continue
        st = {}
        for name in ("pp_dpm_sclk", "pp_dpm_mclk", "pp_dpm_fclk", "pp_dpm_socclk", "current_compute_partition",
                     "current_memory_partition", "power_dpm_force_performance_level", "gpu_busy_percent",
                     "mem_busy_percent"):
            try:
                with open(os.path.join(card, name)) as f:
                    txt = f.read().strip()
            except OSError:
                continue
            if name.startswith("pp_dpm_"):      # keep the active level(s): the lines marked with '*'
                act = [ln.strip() for ln in txt.splitlines() if ln.rstrip().endswith("*")]
                txt = "; ".join(act) if act else txt.replace("\n", "; ")
            st[name] = txt
        for hw in glob.glob(os.path.join(card, "hwmon", "hwmon*")):
            # temp2: junction, temp3: memory (millidegrees), as their *_label files say on these boxes
            for name in ("power1_average", "power1_input", "power1_cap", "temp1_input", "temp2_input", "temp3_input",
                         "freq1_input", "freq2_input"):
                try:
                    with open(os.path.join(hw, name)) as f:
                        st[name] = f.read().strip()
                except OSError:
                    pass
        if st:
            out[os.path.basename(os.path.dirname(card))] = st
    return out

CONFIGS = {
    # name: layers, batch, q heads, kv heads, hd, context, budget, sinks, recent
    "c3": dict(id=3, layers=32, batch=8, hq=32, hkv=8, hd=128, ctx=131072, budget=2048, sink=4, recent=64,
               desc="config3: 32-layer Llama-3-8B-shaped decode step, batch 8, ctx 131072, "
                    "32q/8kv heads, hd 128, bf16 K/V in HBM, top-k 2048 + 4 sinks + 64 recent"),
    "c2": dict(id=2, layers=1, batch=1, hq=32, hkv=8, hd=128, ctx=32768, budget=1024, sink=4, recent=64,
               desc="config2: one Llama-3-8B-shaped decode layer, batch 1, ctx 32768, "
                    "top-k 1024 + 4 sinks + 64 recent"),
    "c5": dict(id=5, layers=32, batch=1, hq=32, hkv=8, hd=128, ctx=1048576, budget=4096, sink=4, recent=64,
               desc="config5: 32 layers, batch 1, ctx 1048576, top-k 4096 + 4 sinks + 64 recent"),
}
C4_DESC = ("config4: PQ baseline, 8 kv heads x 1048576 keys, hd 128, M 32 x 256 centroids, "
           "ADC scan -> 4096 candidates -> exact rerank to top-k 1024")


def algorithmic_bytes_per_unit(n_region: int, attended: int, group: int, hd: int) -> int:
    """Bytes of the reference's algorithm per (layer, batch, kv-head) unit and decode step:
    K streamed once + gathered K and V rows + q in / out (bf16)."""
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


class Slabs:
    """One allocation for every layer's values, one for the keys, one for the 8-bit key sketch,
    as diffcache_amd.DiffCache lays its store out (scans of one large allocation run about 3 %
    faster on MI355X than scans of per-layer allocations; the sketch, which every step streams,
    is allocated last).  Configurations of equal size (3 and 5) reuse them."""

    def __init__(self, torch, dev, numel: int, sketch: bool):
        self.v = torch.empty((numel,), dtype=torch.bfloat16, device=dev)
        self.k = torch.empty((numel,), dtype=torch.bfloat16, device=dev)
        self.c = torch.empty((numel,), dtype=torch.uint8, device=dev) if sketch else None
        self.numel = numel


class DecodeWorkload:
    """The data of one configuration in HBM, and timed decode steps over it."""

    def __init__(self, torch, hip, name: str, dev, slabs: Slabs = None, sketch: bool = True):
        self.torch, self.hip, self.name, self.dev = torch, hip, name, dev
        cfg = self.cfg = CONFIGS[name]
        L, b, hkv, n, hd = cfg["layers"], cfg["batch"], cfg["hkv"], cfg["ctx"], cfg["hd"]
        numel = L * b * hkv * n * hd
        if slabs is None or slabs.numel < numel:
            slabs = Slabs(torch, dev, numel, sketch)
        shape = (L, b, hkv, n, hd)
        t0 = time.perf_counter()
        kslab, vslab = slabs.k[:numel].view(shape), slabs.v[:numel].view(shape)
        self.layers = [make_layer(torch, cfg, l, cfg["id"], dev, kslab[l], vslab[l]) for l in range(L)]
        self.lo, self.hi = cfg["sink"], n - cfg["recent"]
        self.region = self.hi - self.lo
        self.sketches = None
        if sketch and slabs.c is not None:
            # the sketch of the retrieval region of every layer (prefill-time work, untimed)
            cslab = slabs.c[:numel].view(shape)
            self.sketches = [hip.Sketch(kslab[l], codes=cslab[l]).build(kslab[l], self.lo, self.region)
                             for l in range(L)]
        torch.cuda.synchronize()
        self.setup_s = time.perf_counter() - t0
        self.n_units = b * hkv
        self.grp = cfg["hq"] // hkv
        self.k_eff = min(cfg["budget"], self.region)
        self.attended = self.k_eff + cfg["sink"] + cfg["recent"] + 1
        nu, budget = self.n_units, cfg["budget"]
        self.idx = torch.empty((nu, budget), dtype=torch.int32, device=dev)
        self.out = torch.empty((b, cfg["hq"], hd), dtype=torch.bfloat16, device=dev)
        self.ws = hip.alloc_workspace(hip.layer_workspace_bytes(nu, self.region, budget, self.grp, hd,
                                                                self.attended), dev)
        self.scores = None
        self.stream = torch.cuda.Stream(device=dev)     # default priority
        self.clean = False
        self.calls = {}
        # this process has the GPU to itself and one stream: short contexts may run as one kernel
        # inside the captured step as well (--one-kernel never: the kernel chain at any size)
        self.one_kernel = hip.ONE_KERNEL_EXCLUSIVE

    def layer(self, l: int, scan: str, mode: int, ev=None, route_only: bool = False):
        """One dc_decode_layer call.  scan: "sketch", "bf16" or "dense" (fp32 scores +
        dc_topk_select).  ev: an event pair recorded around the scan kernel."""
        hip, cfg = self.hip, self.cfg
        k, v, q, nk, nv = self.layers[l]
        if scan == "dense" and self.scores is None:
            self.scores = self.torch.empty((self.n_units, self.region), dtype=self.torch.float32, device=self.dev)
        call = self.calls.get((l, scan, mode))
        if call is None:
            # the argument struct of a layer is built once; a step only calls dc_decode_layer
            call = self.calls[(l, scan, mode)] = hip.LayerCall(
                q, k, v, cfg["sink"], self.hi, cfg["recent"], cfg["budget"],
                self.scores if scan == "dense" else None, self.idx, self.out, self.ws, nk, nv,
                mode=mode, order=hip.ORDER_ANY, sketch=self.sketches[l] if scan == "sketch" else None,
                one_kernel=self.one_kernel)
        if route_only:
            return call.route()
        call(select_state_ready=self.clean and scan != "dense", scan_events=ev)
        self.clean = scan != "dense"

    def measure(self, scan: str, mode: int, steps: int, warmup: int, event_stride: int = 4,
                graph: bool = False, cold: bool = False) -> dict:
        torch, cfg = self.torch, self.cfg
        L = cfg["layers"]
        if scan == "sketch" and self.sketches is None:
            raise RuntimeError("this workload was built without a sketch")
        timed = list(range(0, L, max(1, event_stride)))

        def new_events(count):
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(count)]
            for e in evs:       # torch creates the native event on first record; the C side needs the handle
                e.record(self.stream)
            return evs

        def step(evs):
            for l in range(L):
                ev = None
                if evs is not None and l in timed:
                    j = timed.index(l)
                    ev = (evs[2 * j], evs[2 * j + 1])
                self.layer(l, scan, mode, ev)

        # A step of few layers is shorter than the events that time it cost (an event is a packet of
        # its own in the queue): then only every `group`-th step carries the in-place event pairs
        # and the per-step marks bracket `group` steps.
        group = 1 if L >= 8 else 8
        n_marks = steps // group if steps >= group else 1
        group = group if steps >= group else steps
        events = [new_events(2 * len(timed)) for _ in range(n_marks)]
        marks = new_events(n_marks + 1)
        torch.cuda.synchronize()
        with torch.cuda.stream(self.stream):
            for _ in range(warmup):
                step(None)
            torch.cuda.synchronize()
            state_before = device_state()
            t0 = time.perf_counter()
            marks[0].record()
            for s in range(steps):
                step(events[s // group] if s % group == 0 and s // group < n_marks else None)
                if (s + 1) % group == 0 and (s + 1) // group <= n_marks:
                    marks[(s + 1) // group].record()
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - t0
        state_after = device_state()
        ms_per_step = elapsed * 1e3 / steps
        per_step_us = sorted(marks[i].elapsed_time(marks[i + 1]) * 1e3 / group for i in range(n_marks))

        def pct(p):
            return per_step_us[min(len(per_step_us) - 1, int(p * len(per_step_us)))]

        sc = [e[2 * j].elapsed_time(e[2 * j + 1]) for e in events for j in range(len(timed))]
        scan_ms = sum(sc) / len(sc)

        # Small configurations fit in the 256 MB Infinity Cache, so the loop above measures a warm
        # cache.  Cold: a 1 GiB buffer is overwritten before every step (untimed) and each step is
        # timed on its own.
        cold_us = None
        if cold:
            flush = torch.empty((1 << 30,), dtype=torch.uint8, device=self.dev)
            c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            samples = []
            for s_i in range(min(steps, 30)):
                with torch.cuda.stream(self.stream):
                    flush.fill_(s_i & 0xff)
                    c0.record()
                    step(None)
                    c1.record()
                torch.cuda.synchronize()
                samples.append(c0.elapsed_time(c1) * 1e3)
            samples.sort()
            cold_us = samples[len(samples) // 2]
            del flush

        graph_us = None
        if graph:
            # every call of the step only enqueues kernels, so the whole step can be captured; the
            # select state is already "left ready" by the eager steps above
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=self.stream):
                for l in range(L):
                    self.layer(l, scan, mode, None)
            torch.cuda.synchronize()
            for _ in range(max(warmup, 1)):
                g.replay()
            torch.cuda.synchronize()
            tg = time.perf_counter()
            for _ in range(steps):
                g.replay()
            torch.cuda.synchronize()
            graph_us = (time.perf_counter() - tg) * 1e6 / steps

        hd, nu = cfg["hd"], self.n_units
        unit_bytes = algorithmic_bytes_per_unit(self.region, self.k_eff + cfg["sink"] + cfg["recent"], self.grp, hd)
        step_bytes = unit_bytes * nu * L                      # the reference's algorithm
        # what this route has to move: the sketch scan reads hd bytes per key, not 2 * hd
        path_bytes = step_bytes - (nu * L * self.region * hd if scan == "sketch" else 0)
        rows_bytes_8d = nu * self.region * hd * 2             # one launch, every bf16 key row once
        scan_bytes = rows_bytes_8d // 2 if scan == "sketch" else rows_bytes_8d + \
            (nu * self.region * 4 if scan == "dense" else 0)
        kernel = {"sketch": "sketch_prune_kernel", "bf16": "score_prune_kernel",
                  "dense": "score_kernel"}[scan] + "<%d>" % hd
        call_path = "dc_decode_layer" + {"sketch": " (sketch scan + exact rescoring)", "bf16": "",
                                         "dense": " (dense scores)"}[scan]
        if self.layer(0, scan, mode, route_only=True) == self.hip.ROUTE_ONE_KERNEL:
            # short context: the layer is one kernel that reads the bf16 keys (with or without a
            # sketch) and the event pair brackets all of it
            kernel = "small_layer_kernel<%d, %d>" % (hd, self.grp)
            call_path = "dc_decode_layer (short context: one kernel)"
            path_bytes = step_bytes
            scan_bytes = unit_bytes * nu
        ach = scan_bytes / (scan_ms * 1e-3) / 1e9
        roofline = {
            "bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBPS,
            "traffic": None,
            "kernel": kernel,
            "algorithmic_bytes_per_launch": scan_bytes, "avg_launch_us": scan_ms * 1e3,
            "timed_launches": len(sc),
            # the same launch priced at the reference algorithm's bytes (two per key element)
            "achieved_8d": rows_bytes_8d / (scan_ms * 1e-3) / 1e9,
            "frac_8d": rows_bytes_8d / (scan_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        }
        one_kernel = kernel.startswith("small_layer_kernel")
        key = "c2.one_kernel" if (self.name == "c2" and one_kernel) else f"{self.name}.{scan}"
        roofline["traffic"] = profiled_traffic(key)
        if roofline["traffic"] is not None:
            roofline["traffic_source"] = "profiles/hbm_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE when " \
                                         "the committed profile summaries were taken, not measured in this run"
        # The same binary has been seen at two levels of the scan's speed (about +10 %), constant
        # within a process: say which one this run was at (configuration 3 only, where it was seen).
        level = None
        if self.name == "c3" and not one_kernel and scan in ("sketch", "bf16"):
            level = "fast" if scan_ms * 1e3 < (185.0 if scan == "sketch" else 342.0) else "slow"
        s_per_step = ms_per_step * 1e-3
        return {
            "value": ms_per_step * 1e3, "unit": "us", "ms_per_step": ms_per_step, "steps": steps, "warmup": warmup,
            "workload": cfg["desc"], "scan": scan,
            # the arithmetic the route computes in: the sketch scan reads one byte per key element
            # and the rows that survive are rescored from the bf16 keys in fp32
            "dtype": "bf16" if (one_kernel or scan != "sketch") else "u8 sketch scan + bf16 exact rescoring",
            "level": level,
            "device_state": {"before": state_before, "after": state_after},
            "call_path": call_path,
            "step_us_p10_p50_p90": [pct(0.10), pct(0.50), pct(0.90)],
            "roofline": roofline,
            # bytes this route must move per step over the step time: the step-level HBM fraction
            "step_path_bytes": path_bytes,
            "step_path_gbps": path_bytes / s_per_step / 1e9,
            "step_path_frac": path_bytes / s_per_step / 1e9 / HBM_PEAK_GBPS,
            # bytes of the reference's algorithm (every bf16 key once + gathered rows) over the same time
            "step_8d_bytes": step_bytes,
            "step_8d_gbps": step_bytes / s_per_step / 1e9,
            "step_8d_frac": step_bytes / s_per_step / 1e9 / HBM_PEAK_GBPS,
            "keys_scored_per_s": nu * L * self.region / s_per_step,
            "cold_cache_step_us_median": cold_us,
            "graph_step_us": graph_us,
        }


def measure_pq(torch, hip, dev, steps: int, warmup: int, stepwise: bool = False, store=None) -> dict:
    """Benchmark configuration 4: tables + ADC scan -> 4096 candidates -> exact bf16 rerank -> top 1024."""
    h, n, m, n_cand, topk = 8, 1 << 20, 32, 4096, 1024
    t_gen = time.perf_counter()
    index, store, q = make_pq_index(torch, hip, dev, store)
    torch.cuda.synchronize()
    t_gen = time.perf_counter() - t_gen
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(steps)]
    hist = hip.new_hist(h, dev)

    def step(e=None):
        lut = hip.pq_build_lut(q, index.books, 1)
        if not stepwise:
            ids = hip.pq_search(store, index.codes, lut, q, n_cand, topk, idx_out=index.ids,
                                workspace=index.ws, state_ready=index._ws_ready, scan_events=e)
            index._ws_ready = True
            return ids
        # the separate entry points, with a dense ADC score array
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
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        step(ev[s])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    scan_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / len(ev)
    scan_bytes = h * n * m
    ach = scan_bytes / (scan_ms * 1e-3) / 1e9
    # the configuration's algorithmic bytes: codes + 4096 rerank rows + codebooks + tables, per unit
    algo = h * (n * m + n_cand * 256 + m * 256 * 4 * 4 + m * 256 * 4)
    return {
        "value": ms * 1e3, "unit": "us", "ms_per_step": ms, "steps": steps, "warmup": warmup,
        "workload": C4_DESC, "dtype": "u8 codes, fp32 tables, bf16 rerank",
        "call_path": "dc_pq_build_lut + " + ("the stepwise entry points" if stepwise else "dc_pq_search_bf16"),
        "roofline": {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": ach / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "pq_adc_kernel<32>" if stepwise else "pq_prune_kernel<32>",
                     "algorithmic_bytes_per_launch": scan_bytes, "avg_launch_us": scan_ms * 1e3,
                     "timed_launches": len(ev)},
        "step_8d_bytes": algo, "step_8d_frac": algo / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "setup_s": t_gen,
    }


def cpu_baseline(torch, work: DecodeWorkload, target_s: float = 12.0) -> dict:
    """The C restatement of the reference's exact-scan path (oracle/cpu_ref.c), timed on this
    box's host cores on a bounded sample of the same workload.  One thread per (batch, kv-head)
    unit, as rayon's fan-out over units does (lib.rs:387-401), with as many units in flight as
    the box gives cores to one GPU.  The sample rotates over several layers' K/V so that no pass
    finds its keys in the host's last-level cache."""
    import numpy as np
    from oracle import cpu_ref
    cfg = work.cfg
    hkv, hq, hd, n, b, L = cfg["hkv"], cfg["hq"], cfg["hd"], cfg["ctx"], cfg["batch"], cfg["layers"]
    grp = hq // hkv
    cores = os.cpu_count() or 1
    share = min(cores, 16)                      # a GPU box gives one GPU's share of the host: 16 cores
    nb = max(1, min(b, share // hkv))           # batch elements per pass
    units = nb * hkv
    threads = min(units, share)
    n_buf = min(L, 4)                           # distinct layers to rotate over (4 x 0.5 GB of keys)

    def host(t):
        return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)

    bufs = []
    for l in range(n_buf):
        k, v, q, nk, nv = work.layers[l]
        bufs.append((host(q[:nb]).reshape(units, grp, hd), host(k[:nb]).reshape(units, n, hd),
                     host(v[:nb]).reshape(units, n, hd), host(nk[:nb]).reshape(units, hd),
                     host(nv[:nb]).reshape(units, hd)))
    cpu_ref.lib()
    reps, total = 0, 0.0
    while total < target_s and reps < 20000:
        q0, k0, v0, nk0, nv0 = bufs[reps % n_buf]
        t0 = time.perf_counter()
        cpu_ref.decode_layer(q0, k0, v0, cfg["budget"], cfg["sink"], cfg["recent"], n_ctx=n,
                             new_k_u16=nk0, new_v_u16=nv0, n_threads=threads, want_ids=False)
        total += time.perf_counter() - t0
        reps += 1
    per_pass = total / reps
    units_total = L * b * hkv
    pass_bytes = units * n * hd * 2
    return {
        "value": per_pass * (units_total / units) * 1e6, "unit": "us", "cores": threads, "kind": "port",
        "sample": (f"oracle/cpu_ref.c decode_layer (scan + heap select + gather + attention) on {units} units "
                   f"({nb} batch element(s) of one layer, {n} rows each), {threads} threads, rotating over "
                   f"{n_buf} layers' K/V ({n_buf * pass_bytes / 1e9:.1f} GB of keys); mean of {reps} passes = "
                   f"{per_pass * 1e3:.2f} ms ({pass_bytes / per_pass / 1e9:.0f} GB/s of key bytes); scaled x"
                   f"{units_total // units} to the full step ({L} layers x batch {b}); host reports {cores} cpus"),
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="all", choices=["all", "c2", "c3", "c4", "c5"],
                    help="all (default): configuration 3 as the headline, both scan routes, with "
                         "configurations 2, 4 and 5 beside it; or one configuration alone")
    ap.add_argument("--scan", default=None, choices=["sketch", "bf16", "dense"],
                    help="one configuration alone: sketch (default; scan the 8-bit sketch of the keys and "
                         "rescore the surviving rows exactly from the bf16 keys), bf16 (stream the bf16 keys) "
                         "or dense (materialise fp32 scores: dc_score_bf16 + dc_topk_select)")
    ap.add_argument("--mode", default="ref_dist", choices=["ref_dist", "ip"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--event-stride", type=int, default=4,
                    help="time the scan kernel in place on every N-th layer")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="before the steps, run a plain elementwise kernel that reads 1 GiB and writes "
                         "1 GiB three times (a known-size reference for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--stepwise", action="store_true",
                    help="config c4 only: the PQ search through the separate entry points (dense ADC "
                         "score array) instead of dc_pq_search_bf16")
    ap.add_argument("--shape", default=None, metavar="KEY=VALUE,...",
                    help="a decode step of another shape, timed like a single --config: any of layers, batch, "
                         "hq, hkv, hd, ctx, budget, sink, recent (defaults: configuration 3 with 4 layers), "
                         "e.g. --shape batch=2,ctx=524288.  Not a BASELINE configuration: no CPU leg")
    ap.add_argument("--one-kernel", default="exclusive", choices=["exclusive", "never"],
                    help="single --config / --shape: never = take the kernel chain also where the context is "
                         "short enough for the one-kernel route")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one decode step (all layers) in a HIP graph and time its replays; "
                         "reported as graph_step_us (always done for configuration 2)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              "use --gpus 1", file=sys.stderr)
        return 2
    if args.shape is not None:
        cfg = dict(CONFIGS["c3"], id=6, layers=4)
        try:
            for item in args.shape.split(","):
                key, val = item.split("=")
                if key not in ("layers", "batch", "hq", "hkv", "hd", "ctx", "budget", "sink", "recent"):
                    raise ValueError(key)
                cfg[key] = int(val)
        except ValueError as e:
            print(f"bench.py: bad --shape ({e})", file=sys.stderr)
            return 2
        cfg["desc"] = ("other shape: {layers} layers, batch {batch}, ctx {ctx}, {hq}q/{hkv}kv heads, hd {hd}, "
                       "top-k {budget} + {sink} sinks + {recent} recent".format(**cfg))
        CONFIGS["shape"] = cfg
        args.config, args.no_cpu = "shape", True
    if args.config == "all" and args.scan is not None:
        print("bench.py: --scan goes with a single --config", file=sys.stderr)
        return 2

    import torch
    from diffcache_amd import _hip as hip

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    mode = hip.MODE_REF_DIST if args.mode == "ref_dist" else hip.MODE_IP
    steps, warmup = args.steps, args.warmup

    if args.pmc_calibration:
        ca = torch.ones((256 << 20,), dtype=torch.float32, device=dev)      # 1 GiB
        cb = torch.empty_like(ca)
        for _ in range(3):
            torch.add(ca, 1.0, out=cb)
        torch.cuda.synchronize()
        del ca, cb

    head = {"metric": "decode_step_retrieval_sparse_attn_latency_us", "n_gpus": 1, "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}

    def line(res: dict, extra_config: dict) -> dict:
        """The contract's keys first, then everything the measurement returned."""
        out = dict(head)
        out.update({"value": res["value"], "unit": res["unit"], "steps": res["steps"], "warmup": res["warmup"],
                    "ms_per_step": res["ms_per_step"]})
        if "dtype" in res:
            out["dtype"] = res["dtype"]
        out["config"] = dict({"workload": res["workload"], "call_path": res["call_path"]}, **extra_config)
        for k, v in res.items():
            if k not in ("value", "unit", "steps", "warmup", "ms_per_step", "workload", "call_path", "dtype"):
                out[k] = v
        return out

    if args.config == "c4":
        res = measure_pq(torch, hip, dev, steps, warmup, args.stepwise)
        out = line(res, {})
        out["metric"] = "pq_adc_search_latency_us"
        out["cpu_baseline"] = None
        print(json.dumps(out))
        return 0

    if args.config != "all":
        scan = args.scan or "sketch"
        work = DecodeWorkload(torch, hip, args.config, dev, sketch=scan == "sketch")
        if args.one_kernel == "never":
            work.one_kernel = hip.ONE_KERNEL_NEVER
        res = work.measure(scan, mode, steps, warmup, args.event_stride, graph=args.graph or args.config == "c2",
                           cold=args.config == "c2")
        out = line(res, {"key_mode": args.mode})
        out["setup_s"] = work.setup_s
        out["cpu_baseline"] = None if args.no_cpu else cpu_baseline(torch, work)
        print(json.dumps(out))
        return 0

    # ---- the default run: configuration 3 as the headline, the rest beside it -------------------
    c3 = CONFIGS["c3"]
    slabs = Slabs(torch, dev, c3["layers"] * c3["batch"] * c3["hkv"] * c3["ctx"] * c3["hd"], True)
    work = DecodeWorkload(torch, hip, "c3", dev, slabs)
    res = work.measure("sketch", mode, steps, warmup, args.event_stride)
    out = line(res, {"key_mode": args.mode})
    out["setup_s"] = work.setup_s
    out["routes"] = {"bf16": work.measure("bf16", mode, steps, max(2, warmup // 2), args.event_stride)}
    cpu = None if args.no_cpu else cpu_baseline(torch, work)
    del work
    configs = {}
    w5 = DecodeWorkload(torch, hip, "c5", dev, slabs)
    configs["c5"] = w5.measure("sketch", mode, steps, warmup, args.event_stride)
    configs["c5"]["routes"] = {"bf16": w5.measure("bf16", mode, steps, max(2, warmup // 2), args.event_stride)}
    del w5
    w2 = DecodeWorkload(torch, hip, "c2", dev)
    n2 = max(steps, 200)                        # one layer per step: more steps for a stable mean
    configs["c2"] = w2.measure("sketch", mode, n2, max(warmup, 20), 1, graph=True, cold=True)
    configs["c2"]["routes"] = {"bf16": w2.measure("bf16", mode, n2, max(warmup, 20), 1, graph=True, cold=True)}
    del w2
    store4 = slabs.k[:8 * (1 << 20) * 128].view(1, 8, 1 << 20, 128)
    configs["c4"] = measure_pq(torch, hip, dev, max(steps, 100), max(warmup, 10), False, store4)
    out["configs"] = configs
    out["cpu_baseline"] = cpu
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
