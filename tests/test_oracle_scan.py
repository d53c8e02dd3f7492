"""Pins the oracle's scoring / ordering-key / exact top-k functions.

The reference has no tests or vectors for nsw.rs / lib.rs, so each function
is pinned by what the mathematics fixes: hand-computed bit patterns, library
routines (torch bf16 casts, torch.mean, fp32 matmul), brute force on small
inputs, and cases built so that a dropped term, a wrong sign, a transposed
operand or a wrong tie rule fails.
"""
import numpy as np
import pytest
import torch

from oracle import cpu_ref
from oracle import oracle as orc


def rand_bf16(rng, *shape, scale=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


# ---------------- bf16 casts ----------------

def test_bf16_known_bit_patterns():
    assert orc.f32_to_bf16(np.float32([1.0]))[0] == 0x3F80
    assert orc.bf16_to_f32(np.uint16([0x3F80]))[0] == 1.0
    assert orc.bf16_to_f32(np.uint16([0xC000]))[0] == -2.0
    # ties to even: 0x3F808000 is halfway between 0x3F80 and 0x3F81
    half = np.array([0x3F808000, 0x3F818000, 0x3F808001], dtype=np.uint32).view(np.float32)
    assert orc.f32_to_bf16(half).tolist() == [0x3F80, 0x3F82, 0x3F81]


def test_bf16_cast_matches_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * np.exp(rng.standard_normal(20000) * 4)).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.f32_to_bf16(x), want)
    back = torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(orc.bf16_to_f32(want), back)


# ---------------- A1 group mean ----------------

@pytest.mark.parametrize("hq,hkv", [(32, 8), (28, 4), (8, 8), (6, 2)])
def test_group_mean_matches_torch_mean(hq, hkv):
    rng = np.random.default_rng(hq * 100 + hkv)
    b, hd = 3, 128
    q = rand_bf16(rng, b, hq, hd, scale=3.0)
    tq = torch.from_numpy(q.view(np.int16)).view(torch.bfloat16)
    want = tq.view(b, hkv, hq // hkv, hd).mean(dim=2)      # diffcache.py:193
    want = want.view(torch.int16).numpy().view(np.uint16)
    got = orc.group_mean_bf16(q, hkv)
    assert np.array_equal(got, want)
    got_c = cpu_ref.group_mean(q.reshape(b * hkv, hq // hkv, hd), hq // hkv).reshape(b, hkv, hd)
    assert np.array_equal(got_c, want)


def test_group_mean_closed_form():
    # group of 4 holding (1, 2, 3, 6) in every channel -> mean 3 exactly
    q = orc.f32_to_bf16(np.tile(np.float32([1, 2, 3, 6])[None, :, None], (1, 1, 8)))
    assert np.all(orc.bf16_to_f32(orc.group_mean_bf16(q, 1)) == 3.0)


# ---------------- A2 scores ----------------

def test_scores_one_hot_query_reads_a_column():
    rng = np.random.default_rng(2)
    k = rand_bf16(rng, 50, 128)
    for col in (0, 5, 127):
        q = np.zeros(128, np.float32)
        q[col] = 1.0
        s = orc.scores_f64(orc.f32_to_bf16(q), k)
        assert np.array_equal(s, orc.bf16_to_f32(k)[:, col].astype(np.float64))
        assert abs(cpu_ref.dot_bf16(orc.f32_to_bf16(q), k[7]) - s[7]) == 0.0


def test_scores_against_fp32_matmul_and_c_dot():
    rng = np.random.default_rng(3)
    q = rand_bf16(rng, 128)
    k = rand_bf16(rng, 1000, 128, scale=2.0)
    s64 = orc.scores_f64(q, k)
    lib = (torch.from_numpy(orc.bf16_to_f32(k)).double() @ torch.from_numpy(orc.bf16_to_f32(q)).double()).numpy()
    assert np.allclose(s64, lib, rtol=1e-13, atol=1e-12)
    bound = 1e-5 * (np.abs(orc.bf16_to_f32(k).astype(np.float64)) @ np.abs(orc.bf16_to_f32(q).astype(np.float64)))
    c = np.array([cpu_ref.dot_bf16(q, k[i]) for i in range(200)])
    assert np.all(np.abs(c - s64[:200]) <= bound[:200])


def test_scores_not_symmetric_bug_guard():
    # q = e0 + 2 e1, k = 3 e0 + 5 e1 -> 13 (a transposed or squared operand gives another value)
    q = orc.f32_to_bf16(np.float32([1, 2] + [0] * 126))
    k = orc.f32_to_bf16(np.float32([[3, 5] + [0] * 126]))
    assert orc.scores_f64(q, k)[0] == 13.0
    assert cpu_ref.dot_bf16(q, k[0]) == 13.0


# ---------------- ordering key ----------------

def test_ref_dist_known_values_and_quantisation():
    d = orc.ref_dist(np.float32([1.0, 0.0, -1.0, 0.001, 0.0015, 0.002]))
    assert d[0] == np.float32(65535.0) and d[1] == np.float32(65536.0) and d[2] == np.float32(65537.0)
    assert d.view(np.uint32)[0] == 0x477FFF00
    # ulp below 65536 is 2^-8: 0.001 and 0.0015 are under half an ulp and vanish,
    # 0.002 rounds to one ulp
    assert d[3] == np.float32(65536.0) and d[4] == np.float32(65536.0)
    assert d[5] == np.float32(65536.0 - 2.0 ** -8)


def test_pack_neighbour_bits():
    assert int(orc.pack_neighbour(np.float32([1.0]), np.uint32([5]))[0]) == 0x3F80000000000005
    assert cpu_ref.pack(1.0, 5) == 0x3F80000000000005
    assert cpu_ref.pack(65535.0, 0xFFFFFFFF) == 0x477FFF00FFFFFFFF


def test_key32_orders():
    s = np.float32([5.0, -5.0, 0.0, -0.0, 1e-30, 3.0, 65000.0])
    for mode in (orc.MODE_IP, orc.MODE_REF_DIST):
        key = orc.key32(s, mode)
        # larger score never has a larger key
        for i in range(len(s)):
            for j in range(len(s)):
                if s[i] > s[j]:
                    assert key[i] <= key[j]
    kip = orc.key32(s, orc.MODE_IP)
    assert kip[2] == kip[3]                       # +0 and -0 tie
    assert kip[4] < kip[2]                        # IP mode resolves 1e-30 above 0
    kref = orc.key32(s, orc.MODE_REF_DIST)
    assert kref[4] == kref[2]                     # the reference key does not
    # for positive distances the key orders like the raw bits the reference packs
    d = orc.ref_dist(s)
    raw = d.view(np.uint32)
    assert np.array_equal(np.argsort(raw, kind="stable"), np.argsort(kref, kind="stable"))


# ---------------- A3 exact top-k ----------------

def brute(scores, k, mode):
    key = orc.key32(scores, mode)
    order = sorted(range(len(scores)), key=lambda i: (int(key[i]), i))
    return np.array(order[:k], dtype=np.uint32)


@pytest.mark.parametrize("n,k", [(1, 1), (7, 3), (64, 64), (100, 200), (513, 17), (2000, 256)])
def test_topk_equals_brute_force_and_reference_loop(n, k):
    rng = np.random.default_rng(n * 7 + k)
    # coarse scores so that ties are common
    s = (np.round(rng.standard_normal(n) * 4) / 4).astype(np.float32)
    for mode in (orc.MODE_IP, orc.MODE_REF_DIST):
        assert np.array_equal(orc.topk_select(s, k, mode), brute(s, k, mode))
    assert np.array_equal(orc.search_bruteforce(s, k), brute(s, k, orc.MODE_REF_DIST))
    dummy = np.zeros((n, 8), np.uint16)
    _, _, ids, _ = cpu_ref.search_bruteforce(dummy, dummy, np.zeros(8, np.uint16), k, pre_scores=s)
    assert np.array_equal(ids, brute(s, k, orc.MODE_REF_DIST))


def test_zero_query_keeps_lowest_indices():
    rng = np.random.default_rng(5)
    k_rows = rand_bf16(rng, 300, 128)
    q = np.zeros(128, np.uint16)
    s = orc.scores_f32(q, k_rows)
    assert np.all(s == 0)
    for mode in (orc.MODE_IP, orc.MODE_REF_DIST):
        assert orc.topk_select(s, 40, mode).tolist() == list(range(40))
    _, _, ids, _ = cpu_ref.search_bruteforce(k_rows, k_rows, q, 40)
    assert ids.tolist() == list(range(40))


def test_quantised_ties_differ_between_modes():
    # scores 0.0015 (index 0) and 0.001 (index 1) then a clear loser
    s = np.float32([0.001, 0.0015, -3.0])
    assert orc.topk_select(s, 1, orc.MODE_IP).tolist() == [1]
    assert orc.topk_select(s, 1, orc.MODE_REF_DIST).tolist() == [0]   # tie -> lower index
    assert orc.search_bruteforce(s, 1).tolist() == [0]


def test_duplicate_rows_tie_to_lower_index():
    rng = np.random.default_rng(6)
    base = rand_bf16(rng, 20, 128)
    keys = np.concatenate([base, base, base], axis=0)       # every row three times
    q = rand_bf16(rng, 128)
    s = orc.scores_f32(q, keys)
    sel = orc.topk_select(s, 30, orc.MODE_REF_DIST)
    best10 = np.argsort(-s[:20], kind="stable")[:10]
    want = np.concatenate([[i, i + 20, i + 40] for i in best10])
    assert sel.tolist() == want.tolist()
    ok, ov, ids, _ = cpu_ref.search_bruteforce(keys, keys, q, 30)
    # the C path uses fp32 accumulation; duplicates still score identically
    assert sorted(ids.tolist()) == sorted(want.tolist())
    assert np.array_equal(ok, keys[ids])


def test_planted_keys_fill_the_top(tmp_path):
    # benchmark configuration 1: N 8192, 16 planted keys = 3 q + 0.1 noise, k 256
    rng = np.random.default_rng(1000)
    n, hd, k = 8192, 128, 256
    qf = rng.standard_normal(hd).astype(np.float32)
    kf = rng.standard_normal((n, hd)).astype(np.float32)
    planted = rng.choice(n, 16, replace=False)
    kf[planted] = 3 * qf + 0.1 * rng.standard_normal((16, hd)).astype(np.float32)
    q, keys = orc.f32_to_bf16(qf), orc.f32_to_bf16(kf)
    vals = rand_bf16(rng, n, hd)
    s = orc.scores_f32(q, keys)
    sel = orc.topk_select(s, k, orc.MODE_REF_DIST)
    assert set(sel[:16].tolist()) == set(planted.tolist())
    ok, ov, ids, sc = cpu_ref.search_bruteforce(keys, vals, q, k)
    assert set(ids[:16].tolist()) == set(planted.tolist())
    assert np.array_equal(ov, vals[ids])
    # invariants of any correct selection
    kept = np.zeros(n, bool)
    kept[sel] = True
    assert kept.sum() == k
    assert s[kept].min() >= s[~kept].max()


def test_data_layer_query_matches_c_fanout():
    rng = np.random.default_rng(8)
    b, h, ctx, n_max, hd, ef = 2, 3, 500, 640, 64, 32
    # integer-valued bf16 -> every fp32 accumulation order is exact -> ids must agree bit for bit
    keys = orc.f32_to_bf16(rng.integers(-4, 5, (b, h, n_max, hd)).astype(np.float32))
    vals = rand_bf16(rng, b, h, n_max, hd)
    q = orc.f32_to_bf16(rng.integers(-4, 5, (b, h, hd)).astype(np.float32))
    ok, ov, ids = orc.data_layer_query(keys[:, :, :ctx], vals[:, :, :ctx], q, ef)
    ck, cv, cids = cpu_ref.query(keys, vals, q, ef, ctx_len=ctx, n_threads=3)
    assert np.array_equal(ids, cids)
    assert np.array_equal(ok, ck) and np.array_equal(ov, cv)
    # ef larger than the context is clamped (lib.rs:374)
    ck2, _, cids2 = cpu_ref.query(keys, vals, q, 10_000, ctx_len=ctx, n_threads=2)
    assert cids2.shape == (b, h, ctx)
    assert sorted(cids2[0, 0].tolist()) == list(range(ctx))


# ---------------- A6 regions ----------------

def test_region_split_known_cases():
    assert orc.region_split(1000, 128, 128) == (128, 128, 128, 872)
    assert orc.region_split(100, 128, 128) == (100, 0, 100, 100)
    assert orc.region_split(200, 128, 128) == (128, 72, 128, 128)
    assert orc.region_split(32768, 4, 64) == (4, 64, 4, 32704)
    rows = orc.attended_rows(np.uint32([5, 0]), 4, 32704, 32768)
    assert rows[:2].tolist() == [9, 4] and rows[2:6].tolist() == [0, 1, 2, 3]
    assert rows[6:].tolist() == list(range(32704, 32768))
    assert len(set(rows.tolist())) == len(rows)
