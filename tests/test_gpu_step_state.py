"""Device-side step state, rollover of the recent window, and saving after decode steps.

The reference keeps a captured attention call valid across steps through the device tensor
``cache_seqlens`` (src/diffcache/base.py:134-142,150-152); ``DiffCache.step_state`` plays
that role here.  The reference never lets tokens leave the recent window
(src/diffcache/kvcache/diffcache.py:221 asserts, although diffcache_cpu/src/lib.rs:352-369
exists for it); here the region boundary moves (``DiffCache.rollover``).  Every step is
checked against ``oracle.decode_layer`` on the history grown so far.
"""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from test_gpu_api import DEV, bf16_close, dev_bf16, make_cache, np_u16, rand_bf16

pytestmark = pytest.mark.gpu


class History:
    """Host copy of what a cache should hold: prompt rows plus every decoded token, per layer."""

    def __init__(self, K, V):
        self.k = [np.transpose(x, (0, 2, 1, 3)).copy() for x in K]      # (b, hkv, n, hd)
        self.v = [np.transpose(x, (0, 2, 1, 3)).copy() for x in V]

    def push(self, l, nk, nv):                                           # nk, nv (b, 1, hkv, hd)
        self.k[l] = np.concatenate([self.k[l], np.transpose(nk, (0, 2, 1, 3))], axis=2)
        self.v[l] = np.concatenate([self.v[l], np.transpose(nv, (0, 2, 1, 3))], axis=2)


def check_against_oracle(cache, hist, l, q, nk, nv, out, idx, suffix_len, mode=orc.MODE_REF_DIST):
    """ids and output of one decode_attention call == oracle.decode_layer over the history, the
    selection being judged on the GPU's own dense scores of the current region."""
    from diffcache_amd import _hip
    b, hkv, hq, hd, budget = cache.batch_size, cache.num_kv_heads, cache.num_q_heads, cache.head_dim, cache.retrieval_budget
    lo, hi = cache._region()
    n_now = hist.k[l].shape[2]
    assert hi + suffix_len == n_now, (hi, suffix_len, n_now)
    qmean = orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)
    sc = _hip.score(cache.kstore[l], dev_bf16(qmean), lo, hi - lo, _hip.MODE_REF_DIST).cpu().numpy()
    got = orc.bf16_to_f32(np_u16(out))
    ids = idx.cpu().numpy().astype(np.uint32)
    k_eff = min(budget, hi - lo)
    for bi in range(b):
        res = orc.decode_layer(q.reshape(b, hq, hd)[bi], hist.k[l][bi], hist.v[l][bi], hkv, budget,
                               cache.kvbuf_prefix_len, suffix_len, mode, nk[bi, 0], nv[bi, 0],
                               scores_override=sc[bi * hkv:(bi + 1) * hkv])
        for h in range(hkv):
            assert np.array_equal(ids[bi * hkv + h, :k_eff], res["sel"][h]), (l, bi, h)
        assert bf16_close(got[bi], res["out"]), (l, bi)


def test_decode_attention_captured_once_and_replayed_with_a_growing_window():
    """decode_attention of every layer captured ONCE in a HIP graph; ten replays with fresh
    inputs: the appended row, the attended window and the counter move on the device, and every
    replay equals the eager call on a twin cache and the oracle."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(70)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 2, 2, 8, 128, 96, 4, 8, 32, 1500
    K = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    caches = [make_cache(L, b, seq + 64, hkv, hq, hd, budget, p, s, smax) for _ in range(3)]
    for c in caches:
        for l in range(L):
            c.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    graphed, eager, warm = caches
    hist = History(K, V)
    qs = [torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    nks = [torch.zeros((b, 1, hkv, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    nvs = [torch.zeros((b, 1, hkv, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    outs = [torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    # every kernel runs once outside capture (on the third cache), buffers exist before capture
    for l in range(L):
        warm.decode_attention(l, qs[l], nks[l], nvs[l], order=_hip.ORDER_BEST)
    graphed._ensure_workspace()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for l in range(L):
            graphed.decode_attention(l, qs[l], nks[l], nvs[l], out=outs[l], order=_hip.ORDER_BEST)
    assert graphed.kvbuf_suffix_len == s                     # capturing ran nothing
    assert int(graphed.step_state.item()) == s
    for step in range(10):
        q_np = [rand_bf16(rng, b, hq, hd) for _ in range(L)]
        nk_np = [rand_bf16(rng, b, 1, hkv, hd) for _ in range(L)]
        nv_np = [rand_bf16(rng, b, 1, hkv, hd) for _ in range(L)]
        for l in range(L):
            qs[l].copy_(dev_bf16(q_np[l]))
            nks[l].copy_(dev_bf16(nk_np[l]))
            nvs[l].copy_(dev_bf16(nv_np[l]))
        print(f"replay {step}: window {s + step} rows", flush=True)
        g.replay()
        torch.cuda.synchronize()
        for l in range(L):
            want = eager.decode_attention(l, qs[l], nks[l], nvs[l], order=_hip.ORDER_BEST)
            torch.cuda.synchronize()
            assert torch.equal(outs[l], want), (step, l)
            assert torch.equal(graphed.idx[l], eager.idx[l]), (step, l)
            check_against_oracle(graphed, hist, l, q_np[l], nk_np[l], nv_np[l], outs[l], graphed.idx[l], s + step)
            hist.push(l, nk_np[l], nv_np[l])
        graphed.advance_host_step()
        assert int(graphed.step_state.item()) == s + step + 1 == graphed.kvbuf_suffix_len == eager.kvbuf_suffix_len
        lo, hi = graphed._region()
        for l in range(L):          # the appended rows are in the store
            assert np.array_equal(np_u16(graphed.kstore[l][:, :, hi:hi + s + step + 1]), hist.k[l][:, :, hi:])
        (torch.randn(1000, device=DEV) * 2).sum().item()    # unrelated eager work between replays


@pytest.mark.parametrize("with_sketch", [True, False])
@pytest.mark.parametrize("order", [0, 1])
def test_decode_layer_with_the_region_end_on_the_device(with_sketch, order):
    """dc_layer_args.region_hi_dev through the C ABI: launches laid out for the largest region,
    the live end read by the kernels.  For several live ends on ONE workspace (select state left
    ready from call to call) the ids and the output equal those of a call that passes the same end
    as a launch parameter."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(75)
    b, hkv, hq, hd, budget, p, n_max, cap_recent = 2, 2, 8, 128, 200, 4, 9000, 16
    g = hq // hkv
    k, v = rand_bf16(rng, b, hkv, n_max, hd), rand_bf16(rng, b, hkv, n_max, hd)
    kd, vd = dev_bf16(k), dev_bf16(v)
    hi_cap = n_max - cap_recent
    sk = _hip.Sketch(kd).build(kd, p, hi_cap - p) if with_sketch else None
    ws = _hip.alloc_workspace(_hip.layer_workspace_bytes(b * hkv, hi_cap - p, budget, g, hd, budget + p + cap_recent + 1), DEV)
    state = torch.zeros((4,), dtype=torch.int32, device=DEV)
    first = True
    for hi, n_recent in [(2000, 5), (2001, 16), (8984, 0), (300, 7), (204, 16)]:
        q = dev_bf16(rand_bf16(rng, b, hq, hd))
        nk, nv = dev_bf16(rand_bf16(rng, b, hkv, hd)), dev_bf16(rand_bf16(rng, b, hkv, hd))
        state.copy_(torch.tensor([n_recent, hi, hi + n_recent, 0], dtype=torch.int32))
        idx_d = torch.full((b * hkv, budget), -1, dtype=torch.int32, device=DEV)
        out_d = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
        print(f"region end on the device: hi={hi} n_recent={n_recent} sketch={with_sketch} order={order}", flush=True)
        _hip.decode_layer(q, kd, vd, p, hi_cap, cap_recent, budget, None, idx_d, out_d, ws, nk, nv, order=order,
                          select_state_ready=not first, sketch=sk, n_recent_dev=state[0:1], region_hi_dev=state[1:2])
        assert _hip.last_route() == (_hip.ROUTE_SKETCH if with_sketch else _hip.ROUTE_STREAM)
        first = False
        idx_h = torch.full((b * hkv, budget), -1, dtype=torch.int32, device=DEV)
        out_h = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
        ws_h = _hip.alloc_workspace(_hip.layer_workspace_bytes(b * hkv, hi - p, budget, g, hd, budget + p + n_recent + 1), DEV)
        _hip.decode_layer(q, kd, vd, p, hi, n_recent, budget, None, idx_h, out_h, ws_h, nk, nv, order=order,
                          sketch=sk, one_kernel=_hip.ONE_KERNEL_NEVER)
        torch.cuda.synchronize()
        if order == _hip.ORDER_BEST:
            assert torch.equal(idx_d, idx_h), (hi, n_recent)
        else:
            assert torch.equal(torch.sort(idx_d, dim=1).values, torch.sort(idx_h, dim=1).values), (hi, n_recent)
        assert torch.allclose(out_d.float(), out_h.float(), atol=2e-3, rtol=2.0 ** -7), (hi, n_recent)


@pytest.mark.parametrize("key_sketch", [True, False])
def test_captured_step_survives_rollovers(key_sketch):
    """Every layer's decode_attention captured ONCE; 3 x kvbuf_suffix_maxlen replays with
    rollover() between them whenever the window is full.  The region's end, the window's length
    and the append position are device words, so the one graph serves the whole generation (the
    reference's graphs do: src/diffcache/base.py:46-55; its data layer takes every token:
    diffcache_cpu/src/lib.rs:352-369).  Every step equals the eager call on a twin cache (which
    rolls over by itself) and the oracle on the grown history."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(74)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 2, 2, 8, 128, 96, 4, 6, 14, 1200
    steps = 3 * smax
    scale = np.exp(rng.standard_normal((1, 1, hkv, hd))).astype(np.float32)
    K = [orc.f32_to_bf16(rng.standard_normal((b, seq, hkv, hd)).astype(np.float32) * scale) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    caches = [make_cache(L, b, seq + steps + 8, hkv, hq, hd, budget, p, s, smax, key_sketch=key_sketch) for _ in range(3)]
    for c in caches:
        for l in range(L):
            c.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    graphed, eager, warm = caches
    hist = History(K, V)
    qs = [torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    nks = [torch.zeros((b, 1, hkv, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    nvs = [torch.zeros((b, 1, hkv, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    outs = [torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    for l in range(L):      # every kernel once outside capture (on the third cache)
        warm.decode_attention(l, qs[l], nks[l], nvs[l], order=_hip.ORDER_BEST)
    graphed._ensure_workspace()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for l in range(L):
            graphed.decode_attention(l, qs[l], nks[l], nvs[l], out=outs[l], order=_hip.ORDER_BEST)
    assert graphed.captured_region_on_device is True
    want_suffix, rollovers, region0 = s, 0, graphed.retrieval_region_len
    for step in range(steps):
        if graphed.window_full():           # between two replays: stream-ordered, no capture again
            assert graphed.rollover() == smax - s
            want_suffix, rollovers = s, rollovers + 1
        q_np = [rand_bf16(rng, b, hq, hd) for _ in range(L)]
        big = 25.0 if step % 7 == 3 else 1.0    # some keys far outside the range the sketch was fitted to
        nk_np = [rand_bf16(rng, b, 1, hkv, hd, scale=big) for _ in range(L)]
        nv_np = [rand_bf16(rng, b, 1, hkv, hd) for _ in range(L)]
        for l in range(L):
            qs[l].copy_(dev_bf16(q_np[l]))
            nks[l].copy_(dev_bf16(nk_np[l]))
            nvs[l].copy_(dev_bf16(nv_np[l]))
        print(f"replay {step}: region {graphed.retrieval_region_len} rows, window {want_suffix}", flush=True)
        g.replay()
        torch.cuda.synchronize()
        assert graphed.retrieval_region_len == region0 + rollovers * (smax - s)
        for l in range(L):
            want = eager.decode_attention(l, qs[l], nks[l], nvs[l], order=_hip.ORDER_BEST)
            torch.cuda.synchronize()
            assert torch.equal(graphed.idx[l], eager.idx[l]), (step, l)
            assert torch.equal(outs[l], want), (step, l)
            check_against_oracle(graphed, hist, l, q_np[l], nk_np[l], nv_np[l], outs[l], graphed.idx[l], want_suffix)
            hist.push(l, nk_np[l], nv_np[l])
        graphed.advance_host_step()
        want_suffix += 1
        n_recent, region_hi, append_pos, overflow = graphed._state.tolist()
        assert (n_recent, region_hi, append_pos, overflow) == (want_suffix, graphed._region()[1],
                                                               graphed._region()[1] + want_suffix, 0)
        assert eager.kvbuf_suffix_len == graphed.kvbuf_suffix_len and eager.generation == graphed.generation
        (torch.randn(1000, device=DEV) * 2).sum().item()    # unrelated eager work between replays
    assert rollovers >= 4
    graphed.check_status()
    # one replay too many without a rollover is not silent: the device notes the dropped token
    while not graphed.window_full():
        g.replay()
        graphed.advance_host_step()
    g.replay()
    with pytest.raises(AssertionError, match="full recent window"):
        graphed.check_status()


@pytest.mark.parametrize("key_sketch", [True, False])
def test_decode_attention_rolls_the_recent_window_over(key_sketch):
    """3 x kvbuf_suffix_maxlen decode steps: when the window is full its oldest rows join the
    retrieval region; ids and output of every step equal the oracle's on the grown history."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(71)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 1, 2, 8, 128, 64, 4, 6, 12, 700
    steps = 3 * smax
    cache = make_cache(L, b, seq + steps + 4, hkv, hq, hd, budget, p, s, smax, key_sketch=key_sketch)
    scale = np.exp(rng.standard_normal((1, 1, hkv, hd))).astype(np.float32)
    K = [orc.f32_to_bf16(rng.standard_normal((b, seq, hkv, hd)).astype(np.float32) * scale) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    for l in range(L):
        cache.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    hist = History(K, V)
    want_suffix, region0, rollovers = s, cache.retrieval_region_len, 0
    for step in range(steps):
        if want_suffix == smax:             # what the cache is expected to do at the start of this step
            want_suffix, rollovers = s, rollovers + 1
        for l in range(L):
            q = rand_bf16(rng, b, hq, hd)
            # some tokens far outside the range the sketch scales were fitted to, aligned with a query
            big = 25.0 if step % 7 == 3 else 1.0
            nk, nv = rand_bf16(rng, b, 1, hkv, hd, scale=big), rand_bf16(rng, b, 1, hkv, hd)
            out = cache.decode_attention(l, dev_bf16(q), dev_bf16(nk), dev_bf16(nv), order=_hip.ORDER_BEST)
            torch.cuda.synchronize()
            assert cache.generation == rollovers
            check_against_oracle(cache, hist, l, q, nk, nv, out, cache.idx[l], want_suffix)
            hist.push(l, nk, nv)
        want_suffix += 1
        assert cache.kvbuf_suffix_len == want_suffix == int(cache.step_state.item())
        assert cache.retrieval_region_len == region0 + rollovers * (smax - s)
        assert cache.seq_len(0) == seq + step + 1
    assert rollovers >= 5


def test_hook_route_rolls_over_with_tokens_kept_in_the_assembled_buffer():
    """The reference-shaped hooks: the harness's attention call writes each new token into
    kbuf / vbuf (as flash_attn_with_kvcache does), not into the store.  At rollover those rows
    move into the store and the region; the assembled buffer afterwards holds
    [retrieved best first | prefix | the rows that stayed in the window]."""
    rng = np.random.default_rng(72)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 1, 1, 2, 8, 128, 48, 4, 5, 9, 400
    cache = make_cache(L, b, seq + 40, hkv, hq, hd, budget, p, s, smax)
    K, V = [rand_bf16(rng, b, seq, hkv, hd)], [rand_bf16(rng, b, seq, hkv, hd)]
    cache.prefill_update_kv_cache(dev_bf16(K[0]), dev_bf16(V[0]), 0)
    hist = History(K, V)
    b0 = budget
    for step in range(2 * smax):
        q = rand_bf16(rng, b, 1, hq * hd)
        cache.decode_pre_query_operation(dev_bf16(q))
        cache.decode_query_kvcache(0)           # rolls over first when the window is full
        cache.decode_post_query_operation(0)
        torch.cuda.synchronize()
        s_before = cache.kvbuf_suffix_len - 1   # the hook has counted this step's token already
        lo, hi = cache._region()
        n_now = hist.k[0].shape[2]
        assert hi + s_before == n_now
        kc, vc = cache.get_kvcache(0)
        kc, vc = np_u16(kc), np_u16(vc)
        qmean = orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)
        r_len = min(budget, hi - lo)
        for h in range(hkv):
            Kh, Vh = hist.k[0][0, h], hist.v[0][0, h]
            sel = orc.topk_select(orc.scores_f32(qmean[0, h], Kh[lo:hi]), budget, orc.MODE_REF_DIST)
            rows = orc.attended_rows(sel, lo, hi, n_now)
            n_att = r_len + lo + s_before
            assert np.array_equal(kc[0, :n_att, h], Kh[rows]), (step, h)
            assert np.array_equal(vc[0, :n_att, h], Vh[rows]), (step, h)
        # the harness's attention appends the token at cache_seqlens in the assembled buffer
        nk, nv = rand_bf16(rng, b, 1, hkv, hd), rand_bf16(rng, b, 1, hkv, hd)
        slot = b0 + cache.kvbuf_prefix_len + s_before
        cache.kbuf[0][:, :, slot].copy_(dev_bf16(nk)[:, 0])
        cache.vbuf[0][:, :, slot].copy_(dev_bf16(nv)[:, 0])
        hist.push(0, nk, nv)
    assert cache.generation >= 3


def test_prefill_cache_saved_after_decode_steps_holds_the_decoded_tokens(tmp_path):
    """save_prefill_cache after two native decode steps: the suffix files hold the appended
    tokens (they live in the store, not in kbuf / vbuf), and a cache loaded from them continues
    exactly like the original."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(73)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 1, 2, 4, 64, 32, 4, 8, 16, 300
    cache = make_cache(L, b, seq + 20, hkv, hq, hd, budget, p, s, smax)
    K = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    for l in range(L):
        cache.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    hist = History(K, V)
    for step in range(2):
        for l in range(L):
            nk, nv = rand_bf16(rng, b, 1, hkv, hd), rand_bf16(rng, b, 1, hkv, hd)
            cache.decode_attention(l, dev_bf16(rand_bf16(rng, b, hq, hd)), dev_bf16(nk), dev_bf16(nv))
            hist.push(l, nk, nv)
    d = str(tmp_path / "c1")
    os.makedirs(d)
    cache.save_prefill_cache(d)
    sk = torch.load(os.path.join(d, "s_l_001", "k.pt"), weights_only=True)
    assert sk.shape[2] == s + 2
    assert np.array_equal(np_u16(sk), hist.k[1][:, :, seq - s:])
    cache2 = make_cache(L, b, seq + 20, hkv, hq, hd, budget, p, s, smax)
    cache2.load_prefill_cache(torch.zeros((b, seq + 2), dtype=torch.long), d)
    assert cache2.kvbuf_suffix_len == s + 2 == int(cache2.step_state.item())
    q = dev_bf16(rand_bf16(rng, b, hq, hd))
    nk, nv = dev_bf16(rand_bf16(rng, b, 1, hkv, hd)), dev_bf16(rand_bf16(rng, b, 1, hkv, hd))
    for l in range(L):
        a = cache.decode_attention(l, q, nk, nv, order=_hip.ORDER_BEST).clone()
        c = cache2.decode_attention(l, q, nk, nv, order=_hip.ORDER_BEST).clone()
        assert torch.equal(a, c) and torch.equal(cache.idx[l], cache2.idx[l])
