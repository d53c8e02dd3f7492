"""GPU parity of the two host classes that mirror the reference's interfaces:
``DiffCacheHIP`` (lib.rs ``DiffCacheCPU``) against the C restatement of the
exact scan, and ``DiffCache`` (kvcache/diffcache.py) against the numpy oracle."""
import os

import numpy as np
import pytest
import torch

from oracle import cpu_ref
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rand_bf16(rng, *shape, scale=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


def dev_bf16(u16):
    return torch.from_numpy(u16.view(np.int16).copy()).view(torch.bfloat16).to(DEV)


def np_u16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_close(got_f32, want_f64):
    tol = np.maximum(2e-3, np.abs(want_f64) * 2.0 ** -8)
    return bool(np.all(np.abs(got_f32 - want_f64) <= tol))


# ---------------------------------------------------------------- DiffCacheHIP

def test_data_layer_with_key_sketch_built_from_inserts_only():
    """No prefill: the first insert fits the scales, later ones only raise the residual bounds."""
    from diffcache_amd import DiffCacheHIP
    rng = np.random.default_rng(34)
    b, hkv, hd, n = 1, 2, 64, 40
    dl = DiffCacheHIP(b, 2, hkv, hd, max_ctx_len=64, key_sketch=True)
    ks = orc.f32_to_bf16(rng.integers(-9, 10, (n, b, hkv, hd)).astype(np.float32))
    vs = rand_bf16(rng, n, b, hkv, hd)
    for i in range(n):
        dl.insert(ks[i], vs[i])
    q = orc.f32_to_bf16(rng.integers(-2, 3, (b, hkv, hd)).astype(np.float32))
    out_k = torch.zeros((b, hkv, 16, hd), dtype=torch.bfloat16, device=DEV)
    out_v = torch.zeros_like(out_k)
    dl.query(out_k, out_v, q, 16)
    ck, cv, _ = cpu_ref.query(np.transpose(ks, (1, 2, 0, 3)).copy(), np.transpose(vs, (1, 2, 0, 3)).copy(), q, 16)
    assert np.array_equal(np_u16(out_k), ck) and np.array_equal(np_u16(out_v), cv)


def test_data_layer_with_key_sketch_follows_inserts():
    """key_sketch=True: same rows as the C restatement of the exact scan, also after rows far
    outside the range the sketch was fitted to have been inserted."""
    from diffcache_amd import DiffCacheHIP
    rng = np.random.default_rng(33)
    b, hkv, hd, n0 = 1, 2, 128, 600
    dl = DiffCacheHIP(b, 2, hkv, hd, max_ctx_len=1024, key_sketch=True)
    keys = orc.f32_to_bf16(rng.integers(-3, 4, (b, hkv, n0, hd)).astype(np.float32))
    vals = rand_bf16(rng, b, hkv, n0, hd)
    dl.prefill(keys, vals)
    extra_k = orc.f32_to_bf16(rng.integers(-60, 61, (8, b, hkv, hd)).astype(np.float32))
    extra_v = rand_bf16(rng, 8, b, hkv, hd)
    for i in range(8):
        dl.insert(extra_k[i], extra_v[i])
    all_k = np.concatenate([keys, np.transpose(extra_k, (1, 2, 0, 3))], axis=2)
    all_v = np.concatenate([vals, np.transpose(extra_v, (1, 2, 0, 3))], axis=2)
    q = orc.f32_to_bf16(rng.integers(-2, 3, (b, hkv, hd)).astype(np.float32))
    out_k = torch.zeros((b, hkv, 64, hd), dtype=torch.bfloat16, device=DEV)
    out_v = torch.zeros_like(out_k)
    dl.query(out_k, out_v, q, 64)
    ck, cv, _ = cpu_ref.query(all_k, all_v, q, 64)
    assert np.array_equal(np_u16(out_k), ck) and np.array_equal(np_u16(out_v), cv)


def test_data_layer_query_equals_cpu_reference_rows():
    """prefill + query with numpy u16 in/out, the calling convention of
    diffcache.py:147,218-220; integer-valued data makes every fp32 accumulation
    order exact, so rows must match the C restatement of nsw.rs:592-630 bit for bit."""
    from diffcache_amd import DiffCacheHIP, init_metrics, metrics
    init_metrics()
    rng = np.random.default_rng(1)
    b, hq, hkv, hd, n, ef = 2, 8, 2, 128, 3000, 256
    keys = orc.f32_to_bf16(rng.integers(-3, 4, (b, hkv, n, hd)).astype(np.float32))
    vals = rand_bf16(rng, b, hkv, n, hd)
    q = orc.f32_to_bf16(rng.integers(-2, 3, (b, hkv, hd)).astype(np.float32))
    dl = DiffCacheHIP(b, hq, hkv, hd, max_ctx_len=4096, name="l007", use_bruteforce=True)
    neighbours = np.zeros((b, hkv, n, 32), np.uint32)
    dl.prefill(keys, vals, neighbours)
    out_k = np.zeros((b, hkv, ef, hd), np.uint16)
    out_v = np.zeros((b, hkv, ef, hd), np.uint16)
    dl.query(out_k, out_v, q, ef)
    ck, cv, cids = cpu_ref.query(keys, vals, q, ef, n_threads=4)
    assert np.array_equal(out_k, ck) and np.array_equal(out_v, cv)
    ids = dl.query_ids(q, ef).cpu().numpy().astype(np.uint32).reshape(b, hkv, ef)
    assert np.array_equal(ids, cids)
    m = metrics()
    assert m["l007_num_searches"] == b * hkv and m["l007_total_query_latency"] > 0
    # keys come back as f32 (lib.rs:646-649)
    assert np.array_equal(dl.get_keys(), orc.bf16_to_f32(keys))


def test_data_layer_random_data_ids_follow_gpu_scores():
    from diffcache_amd import DiffCacheHIP
    rng = np.random.default_rng(2)
    b, hq, hkv, hd, n, ef = 1, 4, 4, 128, 20000, 1024
    keys, vals = rand_bf16(rng, b, hkv, n, hd), rand_bf16(rng, b, hkv, n, hd)
    q = rand_bf16(rng, b, hkv, hd)
    for key_mode, mode in (("ref_dist", orc.MODE_REF_DIST), ("ip", orc.MODE_IP)):
        dl = DiffCacheHIP(b, hq, hkv, hd, max_ctx_len=n, key_mode=key_mode)
        dl.prefill(dev_bf16(keys), dev_bf16(vals))
        ids, scores = dl.query_ids(dev_bf16(q), ef, return_scores=True)
        ids2 = dl.query_ids(dev_bf16(q), ef)                         # streaming path
        sc = scores.cpu().numpy()
        for u in range(hkv):
            want = orc.topk_select(sc[u], ef, mode)
            assert np.array_equal(ids.cpu().numpy()[u].astype(np.uint32), want)
            assert np.array_equal(ids2.cpu().numpy()[u].astype(np.uint32), want)
            ref = orc.scores_f64(q[0, u], keys[0, u])
            assert np.max(np.abs(sc[u] - ref)) <= 1e-5 * np.max(np.abs(ref)) + 1e-4


def test_data_layer_insert_ef_clamp_and_device_outputs():
    from diffcache_amd import DiffCacheHIP
    rng = np.random.default_rng(3)
    b, hkv, hd = 1, 2, 64
    dl = DiffCacheHIP(b, 4, hkv, hd, max_ctx_len=64)
    keys = orc.f32_to_bf16(rng.integers(-3, 4, (b, hkv, 10, hd)).astype(np.float32))
    vals = rand_bf16(rng, b, hkv, 10, hd)
    dl.prefill(keys, vals)
    extra_k = orc.f32_to_bf16(rng.integers(-3, 4, (5, b, hkv, hd)).astype(np.float32))
    extra_v = rand_bf16(rng, 5, b, hkv, hd)
    for i in range(5):
        dl.insert(extra_k[i], extra_v[i])
    assert dl.ctx_len == 15
    all_k = np.concatenate([keys, np.transpose(extra_k, (1, 2, 0, 3))], axis=2)
    all_v = np.concatenate([vals, np.transpose(extra_v, (1, 2, 0, 3))], axis=2)
    q = orc.f32_to_bf16(rng.integers(-2, 3, (b, hkv, hd)).astype(np.float32))
    out_k = torch.zeros((b, hkv, 40, hd), dtype=torch.bfloat16, device=DEV)
    out_v = torch.zeros_like(out_k)
    dl.query(out_k, out_v, q, 40)                       # ef 40 > ctx 15 -> 15 rows (lib.rs:374)
    ck, cv, _ = cpu_ref.query(all_k, all_v, q, 40)
    assert ck.shape[2] == 15
    assert np.array_equal(np_u16(out_k)[:, :, :15], ck) and np.array_equal(np_u16(out_v)[:, :, :15], cv)
    assert np.all(np_u16(out_k)[:, :, 15:] == 0)
    # raw-pointer variant (lib.rs:626-636)
    sk = torch.zeros((b, hkv, 15, hd), dtype=torch.bfloat16, device=DEV)
    sv = torch.zeros_like(sk)
    dl.query_streaming(torch.cuda.current_stream().cuda_stream, sk.data_ptr(), sv.data_ptr(), q, 15)
    torch.cuda.synchronize()
    assert np.array_equal(np_u16(sk), ck) and np.array_equal(np_u16(sv), cv)
    with pytest.raises(AssertionError):
        dl.update_r_sq([1.0])                           # lib.rs:652
    with pytest.raises(AssertionError):
        dl.query(out_k, out_v, np.zeros((b, hkv + 1, hd), np.uint16), 4)


def test_data_layer_save_load_roundtrip(tmp_path):
    from diffcache_amd import DiffCacheHIP
    rng = np.random.default_rng(4)
    b, hkv, hd, n = 1, 2, 64, 500
    keys, vals = rand_bf16(rng, b, hkv, n, hd), rand_bf16(rng, b, hkv, n, hd)
    dl = DiffCacheHIP(b, 2, hkv, hd, max_ctx_len=512, r_sq=[2.5, 3.5])
    dl.prefill(keys, vals)
    prefix = str(tmp_path / "d_l_000")                  # files land beside it: d_l_000b000_h000.idx
    dl.save(prefix)
    assert os.path.exists(prefix + "b000_h001.idx")
    dl2 = DiffCacheHIP(b, 2, hkv, hd, max_ctx_len=512)
    dl2.load(prefix, 100000)                            # the reference passes the full prompt length
    assert dl2.ctx_len == n and dl2.r_sq == [2.5, 3.5]
    assert np.array_equal(np_u16(dl2.keys[:, :, :n]), keys) and np.array_equal(np_u16(dl2.vals[:, :, :n]), vals)


# ---------------------------------------------------------------- DiffCache

def make_cache(num_layers, b, max_len, hkv, hq, hd, budget, p, s, smax, key_mode="ref_dist",
               key_sketch=True, **extra):
    from diffcache_amd import DiffCache
    if extra:
        kw = dict(num_layers=num_layers, batch_size=b, max_length=max_len, num_kv_heads=hkv,
                  num_q_heads=hq, head_dim=hd, retrieval_budget=budget, nsw_m=16, nsw_ef_cons=200,
                  kvbuf_prefix_len=p, kvbuf_suffix_len=s, kvbuf_suffix_maxlen=smax,
                  attn_mass_threshold=0.9, k_check_seq=[1048576],
                  r_sq=[[4.0] * hkv for _ in range(num_layers)], key_mode=key_mode, key_sketch=key_sketch)
        kw.update(extra)
        return DiffCache(**kw)
    return DiffCache(key_sketch=key_sketch, num_layers=num_layers, batch_size=b, max_length=max_len, num_kv_heads=hkv,
                     num_q_heads=hq, head_dim=hd, retrieval_budget=budget, nsw_m=16, nsw_ef_cons=200,
                     kvbuf_prefix_len=p, kvbuf_suffix_len=s, kvbuf_suffix_maxlen=smax,
                     attn_mass_threshold=0.9, k_check_seq=[1048576],
                     r_sq=[[4.0] * hkv for _ in range(num_layers)], key_mode=key_mode)


@pytest.mark.parametrize("seq", [3000, 150])
def test_diffcache_hooks_assemble_the_reference_buffer(seq):
    """The reference call order (base.py:150-155) through the kept hooks; the
    assembled kbuf/vbuf view must hold [retrieved best-first | prefix | suffix]."""
    rng = np.random.default_rng(10 + seq)
    L, b, hkv, hq, hd, budget, p, s, smax = 2, 2, 2, 8, 128, 256, 16, 32, 64
    g = hq // hkv
    cache = make_cache(L, b, seq + 40, hkv, hq, hd, budget, p, s, smax)
    ks = [orc.f32_to_bf16(rng.integers(-3, 4, (b, seq, hkv, hd)).astype(np.float32)) for _ in range(L)]
    vs = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    for l in range(L):
        k_dev, v_dev = dev_bf16(ks[l]), dev_bf16(vs[l])
        rk, rv = cache.prefill_update_kv_cache(k_dev, v_dev, l)
        assert rk is k_dev and rv is v_dev
    p_len, s_len, lo, hi = orc.region_split(seq, p, s)
    assert (cache.kvbuf_prefix_len, cache.kvbuf_suffix_len, cache.retrieval_region_len) == (p_len, s_len, hi - lo)
    assert cache.seq_len(0) == seq and cache.seq_len_gpu(0) == p_len + s_len + min(budget, hi - lo)
    r_len = min(budget, hi - lo)
    for l in range(L):
        q = orc.f32_to_bf16((rng.integers(-2, 3, (b, 1, hq * hd))).astype(np.float32))
        cache.decode_pre_query_operation(dev_bf16(q))
        cache.decode_query_kvcache(l)
        cache.decode_post_query_operation(l)
        kc, vc = cache.get_kvcache(l)                       # (b, S, hkv, hd) views
        assert kc.shape[1] == r_len + p_len + smax
        kc, vc = np_u16(kc), np_u16(vc)
        qmean = orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)
        assert np.array_equal(np_u16(cache.qbuf), qmean)
        for bi in range(b):
            for h in range(hkv):
                K, V = ks[l][bi, :, h], vs[l][bi, :, h]
                sel = orc.topk_select(orc.scores_f32(qmean[bi, h], K[lo:hi]), budget, orc.MODE_REF_DIST)
                rows = orc.attended_rows(sel, p_len, hi, seq)
                n_att = r_len + p_len + s_len
                assert np.array_equal(kc[bi, :n_att, h], K[rows])
                assert np.array_equal(vc[bi, :n_att, h], V[rows])
    assert cache.kvbuf_suffix_len == s_len + 1               # grows once per step (diffcache.py:222-223)


@pytest.mark.parametrize("key_sketch", [True, False])
def test_diffcache_hooks_in_any_order_hold_the_same_rows(key_sketch):
    """hook_order=ORDER_ANY: the retrieved part of the buffer is a permutation of the reference's
    best-first list (K and V rows permuted alike); prefix and suffix are unchanged."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(12)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 1, 1, 2, 8, 128, 300, 16, 32, 64, 4000
    cache = make_cache(L, b, seq + 40, hkv, hq, hd, budget, p, s, smax, key_sketch=key_sketch,
                       hook_order=_hip.ORDER_ANY)
    ks, vs = rand_bf16(rng, b, seq, hkv, hd), rand_bf16(rng, b, seq, hkv, hd)
    cache.prefill_update_kv_cache(dev_bf16(ks), dev_bf16(vs), 0)
    p_len, s_len, lo, hi = orc.region_split(seq, p, s)
    q = rand_bf16(rng, b, 1, hq * hd)
    cache.decode_pre_query_operation(dev_bf16(q))
    cache.decode_query_kvcache(0)
    cache.decode_post_query_operation(0)
    kc, vc = cache.get_kvcache(0)
    kc, vc = np_u16(kc), np_u16(vc)
    qmean = orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)
    ids = cache.idx[0].cpu().numpy()[:, :budget].astype(np.int64)
    for h in range(hkv):
        K, V = ks[0, :, h], vs[0, :, h]
        sel = orc.topk_select(orc.scores_f32(qmean[0, h], K[lo:hi]), budget, orc.MODE_REF_DIST)
        assert np.array_equal(np.sort(ids[h]), np.sort(sel))
        assert np.array_equal(kc[0, :budget, h], K[ids[h] + lo]) and np.array_equal(vc[0, :budget, h], V[ids[h] + lo])
        rest = orc.attended_rows(sel, p_len, hi, seq)[budget:]
        assert np.array_equal(kc[0, budget:budget + p_len + s_len, h], K[rest])


@pytest.mark.parametrize("key_mode", ["ref_dist", "ip"])
def test_diffcache_decode_attention_matches_oracle_over_steps(key_mode):
    rng = np.random.default_rng(20)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 2, 2, 8, 128, 128, 4, 16, 32, 2000
    mode = orc.MODE_REF_DIST if key_mode == "ref_dist" else orc.MODE_IP
    cache = make_cache(L, b, seq + 64, hkv, hq, hd, budget, p, s, smax, key_mode)
    K = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    for l in range(L):
        cache.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    hist_k = [np.transpose(K[l], (0, 2, 1, 3)).copy() for l in range(L)]      # (b, hkv, n, hd)
    hist_v = [np.transpose(V[l], (0, 2, 1, 3)).copy() for l in range(L)]
    p_len, s_len, lo, hi = orc.region_split(seq, p, s)
    from diffcache_amd import _hip
    for step in range(3):
        for l in range(L):
            q = rand_bf16(rng, b, 1, hq * hd)
            nk, nv = rand_bf16(rng, b, 1, hkv, hd), rand_bf16(rng, b, 1, hkv, hd)
            out = cache.decode_attention(l, dev_bf16(q), dev_bf16(nk), dev_bf16(nv), order=_hip.ORDER_BEST)
            torch.cuda.synchronize()
            got = orc.bf16_to_f32(np_u16(out))
            ids = cache.idx[l].cpu().numpy().astype(np.uint32)
            # dense scores of the same arithmetic decide which ids are expected
            qmean = orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)
            sc = _hip.score(cache.kstore[l], dev_bf16(qmean), lo, hi - lo,
                            _hip.MODE_REF_DIST if key_mode == "ref_dist" else _hip.MODE_IP).cpu().numpy()
            for bi in range(b):
                # history = prompt + tokens of earlier steps; the oracle's region split sees
                # the same fixed region when told the suffix is s_len + step rows long
                res = orc.decode_layer(q.reshape(b, hq, hd)[bi], hist_k[l][bi], hist_v[l][bi], hkv, budget,
                                       p, s_len + step, mode, nk[bi, 0], nv[bi, 0],
                                       scores_override=sc[bi * hkv:(bi + 1) * hkv])
                for h in range(hkv):
                    assert np.array_equal(ids[bi * hkv + h, :budget], res["sel"][h])
                assert bf16_close(got[bi], res["out"])
            # the token becomes part of the history (suffix) for later steps
            hist_k[l] = np.concatenate([hist_k[l], np.transpose(nk, (0, 2, 1, 3))], axis=2)
            hist_v[l] = np.concatenate([hist_v[l], np.transpose(nv, (0, 2, 1, 3))], axis=2)
        assert cache.kvbuf_suffix_len == s_len + step + 1


def test_diffcache_sketch_and_plain_scan_agree():
    """The same prompt and decode steps through a cache that scans the 8-bit sketch and one
    that scans the bf16 keys: identical ids, identical attention output."""
    rng = np.random.default_rng(21)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 1, 4, 16, 128, 256, 4, 8, 16, 9000
    caches = [make_cache(L, b, seq + 32, hkv, hq, hd, budget, p, s, smax, key_sketch=ks) for ks in (True, False)]
    scale = np.exp(rng.standard_normal((1, 1, hkv, hd))).astype(np.float32)
    for l in range(L):
        K = orc.f32_to_bf16(rng.standard_normal((b, seq, hkv, hd)).astype(np.float32) * scale)
        V = rand_bf16(rng, b, seq, hkv, hd)
        for c in caches:
            c.prefill_update_kv_cache(dev_bf16(K), dev_bf16(V), l)
    from diffcache_amd import _hip
    for step in range(3):
        for l in range(L):
            q = dev_bf16(rand_bf16(rng, b, 1, hq * hd))
            nk, nv = dev_bf16(rand_bf16(rng, b, 1, hkv, hd)), dev_bf16(rand_bf16(rng, b, 1, hkv, hd))
            outs = [c.decode_attention(l, q, nk, nv, order=_hip.ORDER_BEST).clone() for c in caches]
            assert torch.equal(caches[0].idx[l], caches[1].idx[l])
            assert torch.equal(outs[0], outs[1])
    # the reference-shaped hooks take the same two routes
    for c in caches:
        c.decode_pre_query_operation(q)
        c.decode_query_kvcache(0)
    assert torch.equal(caches[0].idx[0], caches[1].idx[0])


def test_diffcache_decode_attention_with_k_check():
    """use_k_check: every unit attends to the leading rows the check of nsw.rs:198-296 finds
    sufficient.  One kv-head sees keys whose scores fall off fast (few rows suffice), the other
    near-uniform scores (the whole budget is kept)."""
    rng = np.random.default_rng(44)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 1, 1, 2, 4, 128, 512, 4, 8, 16, 6000
    kseq, thr = [16, 32, 64, 128, 256], 0.9
    cache = make_cache(L, b, seq + 32, hkv, hq, hd, budget, p, s, smax, use_k_check=True,
                       k_check_seq=kseq, attn_mass_threshold=thr)
    q = rand_bf16(rng, b, 1, hq * hd)
    qf = orc.bf16_to_f32(q).reshape(b, hq, hd)
    qmean = orc.bf16_to_f32(orc.group_mean_bf16(q.reshape(b, hq, hd), hkv))          # (b, hkv, hd)
    K = orc.bf16_to_f32(rand_bf16(rng, b, seq, hkv, hd, scale=0.2))
    # head 0: 300 keys aligned with the mean query, with strengths that decay like a power law
    u0 = qmean[0, 0] / np.linalg.norm(qmean[0, 0])
    pos = rng.choice(np.arange(p, seq - s), 300, replace=False)
    strength = 200.0 - 30.0 * np.log(np.arange(1, 301))
    K[0, pos, 0, :] += (strength[:, None] / np.linalg.norm(qmean[0, 0])) * u0[None, :]
    K = orc.f32_to_bf16(K)
    V = rand_bf16(rng, b, seq, hkv, hd)
    cache.prefill_update_kv_cache(dev_bf16(K), dev_bf16(V), 0)
    nk, nv = rand_bf16(rng, b, 1, hkv, hd), rand_bf16(rng, b, 1, hkv, hd)
    out = cache.decode_attention(0, dev_bf16(q), dev_bf16(nk), dev_bf16(nv))
    torch.cuda.synchronize()
    got = orc.bf16_to_f32(np_u16(out))
    from diffcache_amd import _hip
    p_len, s_len, lo, hi = orc.region_split(seq, p, s)
    ids = cache.idx[0].cpu().numpy().astype(np.uint32)
    n_eff = cache.n_eff[0].cpu().numpy()
    kk = np.transpose(K, (0, 2, 1, 3))[0]                                             # (hkv, n, hd)
    vv = np.transpose(V, (0, 2, 1, 3))[0]
    sc = _hip.score(cache.kstore[0], dev_bf16(orc.group_mean_bf16(q.reshape(b, hq, hd), hkv)), lo, hi - lo,
                    _hip.MODE_REF_DIST).cpu().numpy()
    g = hq // hkv
    for h in range(hkv):
        want_ids = orc.topk_select(sc[h], budget, orc.MODE_REF_DIST)
        assert np.array_equal(ids[h, :budget], want_ids)
        d = orc.ref_dist(sc[h][want_ids])
        want_eff = orc.k_check_budget(d, hd, kseq, thr)
        assert int(n_eff[h]) == want_eff, (h, n_eff[h], want_eff)
        rows = orc.attended_rows(want_ids[:want_eff], lo, hi, seq)
        want, _ = orc.sparse_attention(q.reshape(b, hq, hd)[0, h * g:(h + 1) * g], kk[h][rows], vv[h][rows],
                                       nk[0, 0, h], nv[0, 0, h])
        assert bf16_close(got[0, h * g:(h + 1) * g], want)
    assert n_eff[0] < budget and n_eff[1] == budget


def test_diffcache_hooks_under_graph_capture():
    """decode_pre/post are called inside captured graphs in the reference
    (base.py:121-125,132-133): capture them, replay with fresh inputs between
    eager work, compare every replay with the eager result."""
    rng = np.random.default_rng(30)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 1, 1, 2, 8, 128, 64, 4, 8, 32, 1500
    cache = make_cache(L, b, seq + 40, hkv, hq, hd, budget, p, s, smax)
    K, V = rand_bf16(rng, b, seq, hkv, hd), rand_bf16(rng, b, seq, hkv, hd)
    cache.prefill_update_kv_cache(dev_bf16(K), dev_bf16(V), 0)
    q_static = torch.zeros((b, 1, hq * hd), dtype=torch.bfloat16, device=DEV)
    # warm up on a side stream as torch requires before capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        cache.decode_pre_query_operation(q_static)
        cache.decode_query_kvcache(0)
        cache.decode_post_query_operation(0)
    torch.cuda.current_stream().wait_stream(side)
    cache.kvbuf_suffix_len -= 1
    g_pre, g_post = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(g_pre):
        cache.decode_pre_query_operation(q_static)
    with torch.cuda.graph(g_post):
        cache.decode_post_query_operation(0)
    for it in range(3):
        q = rand_bf16(rng, b, 1, hq * hd)
        q_static.copy_(dev_bf16(q))
        g_pre.replay()
        cache.decode_query_kvcache(0)
        g_post.replay()
        torch.cuda.synchronize()
        kc_graph = np_u16(cache.get_kvcache(0)[0]).copy()
        cache.kvbuf_suffix_len -= 1
        cache.decode_pre_query_operation(q_static)
        cache.decode_query_kvcache(0)
        cache.decode_post_query_operation(0)
        torch.cuda.synchronize()
        cache.kvbuf_suffix_len -= 1
        assert np.array_equal(kc_graph, np_u16(cache.get_kvcache(0)[0]))
        (torch.randn(1000, device=DEV) * 2).sum().item()    # unrelated eager work between replays


@pytest.mark.parametrize("with_sketch", [True, False])
def test_decode_layer_chain_in_a_graph(with_sketch):
    """The whole per-layer chain (scan, select, attention) captured in one HIP graph: every
    replay, with fresh queries and eager work and synchronisations in between, must equal the
    eager call."""
    from diffcache_amd import _hip
    rng = np.random.default_rng(31)
    b, hkv, hq, hd, n, budget, p, s = 1, 4, 16, 128, 20000, 512, 4, 32
    k, v = dev_bf16(rand_bf16(rng, b, hkv, n, hd)), dev_bf16(rand_bf16(rng, b, hkv, n, hd))
    lo, hi = p, n - s
    sk = _hip.Sketch(k).build(k, lo, hi - lo) if with_sketch else None
    ws = _hip.alloc_workspace(_hip.layer_workspace_bytes(b * hkv, hi - lo, budget, hq // hkv, hd,
                                                        budget + p + s + 1), DEV)
    q_static = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
    nk, nv = dev_bf16(rand_bf16(rng, b, hkv, hd)), dev_bf16(rand_bf16(rng, b, hkv, hd))
    idx_g = torch.zeros((b * hkv, budget), dtype=torch.int32, device=DEV)
    out_g = torch.zeros((b, hq, hd), dtype=torch.bfloat16, device=DEV)
    idx_e, out_e = torch.zeros_like(idx_g), torch.zeros_like(out_g)

    def call(idx, out, ready):
        _hip.decode_layer(q_static, k, v, lo, hi, s, budget, None, idx, out, ws, nk, nv,
                          order=_hip.ORDER_INDEX, select_state_ready=ready, sketch=sk)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(idx_e, out_e, False)          # warm-up; leaves the select state ready
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(idx_g, out_g, True)
    for it in range(4):
        q_static.copy_(dev_bf16(rand_bf16(rng, b, hq, hd)))
        g.replay()
        torch.cuda.synchronize()
        call(idx_e, out_e, True)
        torch.cuda.synchronize()
        assert torch.equal(idx_g, idx_e) and torch.equal(out_g, out_e), it
        (torch.randn(1000, device=DEV) * 2).sum().item()    # unrelated eager work between replays


def test_diffcache_prefill_cache_roundtrip(tmp_path):
    rng = np.random.default_rng(40)
    L, b, hkv, hq, hd, budget, p, s, smax, seq = 2, 1, 2, 4, 64, 32, 4, 8, 16, 300
    cache = make_cache(L, b, seq + 20, hkv, hq, hd, budget, p, s, smax)
    K = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    V = [rand_bf16(rng, b, seq, hkv, hd) for _ in range(L)]
    for l in range(L):
        cache.prefill_update_kv_cache(dev_bf16(K[l]), dev_bf16(V[l]), l)
    d = str(tmp_path / "c0")
    os.makedirs(d)
    cache.save_prefill_cache(d)
    for name in ("metadata.txt", "p_l_000/k.pt", "s_l_001/v.pt", "d_l_000b000_h001.idx"):
        assert os.path.exists(os.path.join(d, name)), name
    cache2 = make_cache(L, b, seq + 20, hkv, hq, hd, budget, p, s, smax)
    cache2.load_prefill_cache(torch.zeros((b, seq), dtype=torch.long), d)
    assert cache2.retrieval_region_len == cache.retrieval_region_len
    q = rand_bf16(rng, b, 1, hq * hd)
    outs = []
    for c in (cache, cache2):
        c.decode_pre_query_operation(dev_bf16(q))
        c.decode_query_kvcache(1)
        c.decode_post_query_operation(1)
        torch.cuda.synchronize()
        n_att = c.seq_len_gpu(1) - 0
        outs.append(np_u16(c.get_kvcache(1)[0])[:, :budget + p + s])
    assert np.array_equal(outs[0], outs[1])


# ---------------------------------------------------------------- the C handle of the data layer

@pytest.mark.parametrize("use_sketch", [False, True])
def test_c_data_layer_matches_python_data_layer(use_sketch):
    """dc_data_layer_* (the C++ host mirror of lib.rs:189-404) driven through ctypes: prefill,
    a few inserts and queries give the rows DiffCacheHIP gives, which the other tests check
    against the oracle; ef larger than the context is clamped (lib.rs:374)."""
    import ctypes
    from diffcache_amd import DiffCacheHIP, _hip
    lib = _hip.lib
    rng = np.random.default_rng(31)
    b, hq, hkv, hd, n_max, n0, max_ef = 2, 8, 2, 128, 700, 600, 96
    keys, vals = rand_bf16(rng, b, hkv, n0, hd), rand_bf16(rng, b, hkv, n0, hd)
    ref = DiffCacheHIP(b, hq, hkv, hd, max_ctx_len=n_max, key_sketch=use_sketch)
    ref.prefill(keys, vals)

    h = ctypes.c_void_p()
    assert lib.dc_data_layer_create(ctypes.byref(h), b, hkv, hd, n_max, _hip.MODE_REF_DIST, int(use_sketch)) == 0
    try:
        sz = [ctypes.c_size_t() for _ in range(5)]
        assert lib.dc_data_layer_sizes(h, max_ef, *[ctypes.byref(x) for x in sz]) == 0
        store_b, codes_b, scale_b, idx_b, ws_b = [x.value for x in sz]
        kst = torch.zeros(store_b // 2, dtype=torch.bfloat16, device=DEV)
        vst = torch.zeros(store_b // 2, dtype=torch.bfloat16, device=DEV)
        codes = torch.zeros(max(codes_b, 16), dtype=torch.uint8, device=DEV)
        scale = torch.zeros(max(scale_b // 4, 4), dtype=torch.float32, device=DEV)
        resid = torch.zeros(max(scale_b // 4, 4), dtype=torch.float32, device=DEV)
        idx = torch.zeros(idx_b // 4, dtype=torch.int32, device=DEV)
        ws = _hip.alloc_workspace(ws_b, DEV)
        sk = (codes.data_ptr(), scale.data_ptr(), resid.data_ptr()) if use_sketch else (None, None, None)
        assert lib.dc_data_layer_bind(h, kst.data_ptr(), vst.data_ptr(), *sk, idx.data_ptr(), ws.data_ptr(),
                                      ws.numel() * ws.element_size(), max_ef) == 0
        stream = torch.cuda.current_stream().cuda_stream
        # prefill from host memory, as the pyo3 class takes it
        kh, vh = np.ascontiguousarray(keys), np.ascontiguousarray(vals)
        assert lib.dc_data_layer_prefill(h, kh.ctypes.data, vh.ctypes.data, n0, stream) == 0, lib.dc_last_error()
        torch.cuda.synchronize()
        assert lib.dc_data_layer_ctx_len(h) == n0

        def query(ef):
            q = rand_bf16(rng, b, hkv, hd)
            want_k = torch.zeros((b, hkv, max_ef, hd), dtype=torch.bfloat16, device=DEV)
            want_v = torch.zeros_like(want_k)
            ref.query(want_k, want_v, q, ef)
            got_k, got_v = torch.zeros_like(want_k), torch.zeros_like(want_k)
            qd = dev_bf16(q)
            n_out = ctypes.c_int(-1)
            rc = lib.dc_data_layer_query(h, got_k.data_ptr(), got_v.data_ptr(), max_ef, qd.data_ptr(), ef,
                                         ctypes.byref(n_out), stream)
            assert rc == 0, lib.dc_last_error()
            torch.cuda.synchronize()
            assert n_out.value == min(ef, ref.ctx_len)
            assert torch.equal(got_k.view(torch.int16), want_k.view(torch.int16))
            assert torch.equal(got_v.view(torch.int16), want_v.view(torch.int16))

        query(64)
        for _ in range(5):       # rows outside the fitted range of the sketch included
            nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)
            nk[0, 0, :4] = orc.f32_to_bf16(np.array([40.0, -35.0, 20.0, 9.0], dtype=np.float32))
            ref.insert(nk, nv)
            assert lib.dc_data_layer_insert(h, dev_bf16(nk).data_ptr(), dev_bf16(nv).data_ptr(), stream) == 0
            torch.cuda.synchronize()
        assert lib.dc_data_layer_ctx_len(h) == n0 + 5
        query(96)
        query(1)
        # a tiny context: ef is clamped to it
        assert lib.dc_data_layer_prefill(h, kh.ctypes.data, vh.ctypes.data, 0, stream) == 0
        ref.ctx_len = 0
        for _ in range(3):
            nk, nv = rand_bf16(rng, b, hkv, hd), rand_bf16(rng, b, hkv, hd)
            ref.insert(nk, nv)
            assert lib.dc_data_layer_insert(h, dev_bf16(nk).data_ptr(), dev_bf16(nv).data_ptr(), stream) == 0
            torch.cuda.synchronize()
        query(64)
        assert lib.dc_data_layer_query(h, kst.data_ptr(), vst.data_ptr(), max_ef, kst.data_ptr(), max_ef + 1,
                                       None, stream) == -22
    finally:
        lib.dc_data_layer_destroy(h)


# ---------------------------------------------------------------- PQ baseline

def test_pq_index_search_matches_oracle_pipeline():
    """PQIndex.search = ADC scan -> candidates -> exact rerank; codes and tables are
    checked against the numpy oracle, ids against the oracle's pipeline run on the
    GPU's own ADC and exact scores."""
    from diffcache_amd import _hip
    from diffcache_amd.pq import PQIndex, encode, train_codebooks
    rng = np.random.default_rng(50)
    b, h, n, hd, m = 1, 2, 30000, 128, 32
    keys = rand_bf16(rng, b, h, n, hd)
    store = dev_bf16(keys)
    index = PQIndex.build(store, m=m, sample=8192, iters=3, seed=1, n_cand=1024, topk=128)
    books = index.books.cpu().numpy()
    codes = index.codes.cpu().numpy()
    for u in range(h):
        want = orc.pq_encode(orc.bf16_to_f32(keys[0, u]), books[u])
        # the nearest centroid may tie within fp32 rounding of the distance: allow a handful
        assert np.mean(codes[u] != want) < 1e-3
    q = rand_bf16(rng, h, hd)
    ids = index.search(dev_bf16(q)).cpu().numpy()
    lut = _hip.pq_build_lut(dev_bf16(q), index.books, b).cpu().numpy()
    adc = _hip.pq_adc_scan(index.codes, torch.from_numpy(lut).to(DEV)).cpu().numpy()
    for u in range(h):
        assert np.allclose(lut[u], orc.pq_build_lut(q[u], books[u]), rtol=1e-5, atol=1e-5)
        assert np.allclose(adc[u], orc.pq_adc_scores(codes[u], lut[u].astype(np.float64)), rtol=1e-5, atol=1e-4)
        cand = np.sort(orc.topk_select(adc[u], 1024, orc.MODE_IP))
        exact = _hip.score_gathered(store, dev_bf16(q), torch.from_numpy(
            np.stack([cand, cand]).astype(np.int32)).to(DEV)).cpu().numpy()[u]
        order = orc.topk_select(exact, 128, orc.MODE_IP)
        assert np.array_equal(ids[u], cand[order])
        true = set(orc.topk_select(orc.scores_f32(q[u], keys[0, u]), 128, orc.MODE_IP).tolist())
        assert len(true & set(ids[u].tolist())) >= 40      # recall of ADC with 1024 candidates


@pytest.mark.parametrize("b,h,n,hd,m,n_cand,topk", [
    (1, 2, 30000, 128, 32, 1024, 128),
    (2, 3, 5000, 64, 16, 700, 100),      # 16 subspaces, ragged sizes
    (1, 1, 300, 128, 32, 4096, 1024),    # fewer keys than candidates: everything is reranked
    (1, 2, 70000, 256, 32, 9000, 5000),  # candidate list beyond the LDS staging of the finish kernel
    (1, 1, 1, 128, 32, 4, 4),
    (1, 8, 1 << 20, 128, 32, 4096, 1024),   # benchmark configuration 4 at full size
])
def test_pq_search_fused_matches_stepwise(b, h, n, hd, m, n_cand, topk):
    """dc_pq_search_bf16 (no dense ADC array) returns the ids of the entry-point chain
    dc_pq_adc_scan -> dc_topk_select -> dc_score_gathered_bf16 -> dc_topk_select -> dc_compose_idx,
    twice in a row on one workspace."""
    from diffcache_amd.pq import PQIndex
    rng = np.random.default_rng(n + m)
    g = torch.Generator(device=DEV).manual_seed(5)
    store = torch.randn((b, h, n, hd), generator=g, device=DEV).to(torch.bfloat16)
    books = torch.randn((h, m, 256, hd // m), generator=g, device=DEV)
    codes = torch.randint(0, 256, (b * h, n, m), generator=g, device=DEV, dtype=torch.uint8)
    index = PQIndex(store, books, codes, n_cand=n_cand, topk=topk)
    for rep in range(2):
        q = dev_bf16(rand_bf16(rng, b * h, hd))
        want = index.search_stepwise(q).cpu().numpy()
        got = index.search(q).cpu().numpy()
        assert got.shape == want.shape == (b * h, min(topk, n))
        assert np.array_equal(got, want), (rep, np.argwhere(got != want)[:4])


def test_pq_search_fused_ties():
    """Few distinct code rows and repeated key rows: ADC scores and exact scores tie in
    large groups, and both stages must break ties to the lower id."""
    from diffcache_amd.pq import PQIndex
    rng = np.random.default_rng(77)
    b, h, n, hd, m = 1, 2, 20000, 128, 32
    base = rand_bf16(rng, 1, h, 7, hd)
    pick = rng.integers(0, 7, n)
    keys = np.ascontiguousarray(base[:, :, pick])
    store = dev_bf16(keys)
    g = torch.Generator(device=DEV).manual_seed(6)
    books = torch.randn((h, m, 256, hd // m), generator=g, device=DEV)
    rows = torch.randint(0, 256, (b * h, 5, m), generator=g, device=DEV, dtype=torch.uint8)
    sel = torch.from_numpy(rng.integers(0, 5, n)).to(DEV)
    codes = rows[:, sel].contiguous()
    index = PQIndex(store, books, codes, n_cand=3000, topk=500)
    q = dev_bf16(rand_bf16(rng, b * h, hd))
    want = index.search_stepwise(q).cpu().numpy()
    got = index.search(q).cpu().numpy()
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- decode harness

def test_harness_decode_step_matches_dense_attention():
    """SyntheticLlama.decode_step around DiffCache.decode_attention: with a budget that covers
    the whole retrieval region the sparse path is full attention, so the step must equal the
    same layer stack computed with torch's own attention over the full key/value history."""
    from diffcache_amd.harness import SyntheticLlama, synthetic_prompt_cache
    from diffcache_amd import DiffCache
    torch.manual_seed(0)
    L, b, hq, hkv, hd, hidden, inter, ctx = 2, 2, 8, 2, 64, 256, 512, 300
    model = SyntheticLlama(L, hidden, hq, hkv, hd, inter, device=DEV)
    cache = DiffCache(num_layers=L, batch_size=b, max_length=ctx + 16, num_kv_heads=hkv, num_q_heads=hq,
                      head_dim=hd, retrieval_budget=512, nsw_m=16, nsw_ef_cons=200, kvbuf_prefix_len=4,
                      kvbuf_suffix_len=8, kvbuf_suffix_maxlen=24, attn_mass_threshold=0.9,
                      k_check_seq=[1 << 30], r_sq=[[4.0] * hkv for _ in range(L)])
    synthetic_prompt_cache(cache, ctx)
    hist_k = [cache.kstore[l][:, :, :ctx].clone() for l in range(L)]       # (b, hkv, n, hd)
    hist_v = [cache.vstore[l][:, :, :ctx].clone() for l in range(L)]
    from diffcache_amd.harness import GraphedDecoder
    x = torch.randn((b, hidden), device=DEV, dtype=torch.bfloat16)
    g = hq // hkv
    graphed = GraphedDecoder(model, cache, b)
    for step in range(4):
        pos = cache.seq_len(0)
        assert pos == ctx + step
        # eager on even steps, through the captured pre/post graphs on odd ones
        got = (graphed.decode_step(x) if step % 2 else model.decode_step(cache, x)).clone()
        # reference: the same stack with dense attention in fp32
        xr = x
        for l in range(L):
            q, k, v = model.qkv(l, xr, pos)
            hist_k[l] = torch.cat([hist_k[l], k.unsqueeze(2)], dim=2)
            hist_v[l] = torch.cat([hist_v[l], v.unsqueeze(2)], dim=2)
            kk = hist_k[l].float().repeat_interleave(g, dim=1)              # (b, hq, n, hd)
            vv = hist_v[l].float().repeat_interleave(g, dim=1)
            w = torch.softmax(torch.einsum("bhd,bhnd->bhn", q.float(), kk) / hd ** 0.5, dim=-1)
            attn = torch.einsum("bhn,bhnd->bhd", w, vv).to(torch.bfloat16)
            xr = model.post_attention(l, xr, attn)
        err = (got.float() - xr.float()).abs().max().item()
        scale = xr.float().abs().max().item()
        assert err <= 0.03 * scale + 0.03, (step, err, scale)
        x = got
