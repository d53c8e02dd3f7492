"""Pins the oracle's sparse-attention and whole-layer functions by identities
and by torch's scaled_dot_product_attention (a library routine on CPU).  The
reference calls flash-attn here (src/diffcache/base.py:134-142), which is not
in its tree and has no vectors, so nothing stronger exists."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cpu_ref
from oracle import oracle as orc


def rand_bf16(rng, *shape, scale=1.0):
    return orc.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


def bf16_close(got_f32, want_f64):
    """The bar for a bf16 attention output: 2e-3 absolute, widened to half a
    bf16 ulp (2^-8 relative) where the value itself is too large for bf16 to
    hold it to 2e-3."""
    tol = np.maximum(2e-3, np.abs(want_f64) * 2.0 ** -8)
    return bool(np.all(np.abs(got_f32 - want_f64) <= tol))


def test_attention_matches_sdpa():
    rng = np.random.default_rng(11)
    g, s, hd = 4, 333, 128
    q, k, v = rand_bf16(rng, g, hd), rand_bf16(rng, s, hd), rand_bf16(rng, s, hd)
    out, lse = orc.sparse_attention(q, k, v)
    tq = torch.from_numpy(orc.bf16_to_f32(q)).double()[None]          # (1, g, hd)
    tk = torch.from_numpy(orc.bf16_to_f32(k)).double()[None]
    tv = torch.from_numpy(orc.bf16_to_f32(v)).double()[None]
    want = F.scaled_dot_product_attention(tq, tk, tv)[0].numpy()      # default scale 1/sqrt(hd)
    assert np.allclose(out, want, rtol=1e-10, atol=1e-12)
    logits = (tq[0] @ tk[0].T) / np.sqrt(hd)
    assert np.allclose(lse, torch.logsumexp(logits, dim=1).numpy(), rtol=1e-12)


def test_attention_new_token_is_one_more_row():
    rng = np.random.default_rng(12)
    g, s, hd = 2, 40, 64
    q, k, v = rand_bf16(rng, g, hd), rand_bf16(rng, s, hd), rand_bf16(rng, s, hd)
    a, _ = orc.sparse_attention(q, k[:-1], v[:-1], k[-1], v[-1])
    b, _ = orc.sparse_attention(q, k, v)
    assert np.allclose(a, b, rtol=1e-13, atol=1e-14)


def test_attention_identities():
    rng = np.random.default_rng(13)
    g, s, hd = 4, 100, 128
    q, k = rand_bf16(rng, g, hd), rand_bf16(rng, s, hd)
    row = rand_bf16(rng, hd)
    v_same = np.tile(row[None], (s, 1))
    out, _ = orc.sparse_attention(q, k, v_same)                 # weights sum to one
    assert np.allclose(out, np.tile(orc.bf16_to_f32(row)[None], (g, 1)), rtol=1e-12)
    v = rand_bf16(rng, s, hd)
    perm = rng.permutation(s)
    a, la = orc.sparse_attention(q, k, v)
    b, lb = orc.sparse_attention(q, k[perm], v[perm])           # order of the set is irrelevant
    assert np.allclose(a, b, rtol=1e-12, atol=1e-13) and np.allclose(la, lb, rtol=1e-13)
    # two chunks merged through their log-sum-exp equal one chunk
    o1, l1 = orc.sparse_attention(q, k[:37], v[:37])
    o2, l2 = orc.sparse_attention(q, k[37:], v[37:])
    m = np.maximum(l1, l2)
    w1, w2 = np.exp(l1 - m), np.exp(l2 - m)
    merged = (o1 * w1[:, None] + o2 * w2[:, None]) / (w1 + w2)[:, None]
    assert np.allclose(merged, a, rtol=1e-12, atol=1e-13)
    # a dominating key makes the output that key's value row
    k_dom = k.copy()
    k_dom[5] = orc.f32_to_bf16(orc.bf16_to_f32(q[0]) * 50)
    o, _ = orc.sparse_attention(q[:1], k_dom, v)
    assert np.allclose(o[0], orc.bf16_to_f32(v[5]), atol=1e-6)


def test_c_attention_within_bf16_tolerance():
    rng = np.random.default_rng(14)
    g, s, hd = 4, 1093, 128
    q, k, v = rand_bf16(rng, g, hd), rand_bf16(rng, s, hd), rand_bf16(rng, s, hd)
    want, _ = orc.sparse_attention(q, k, v)
    got = orc.bf16_to_f32(cpu_ref.sparse_attention(q, k, v, 1.0 / np.sqrt(hd)))
    assert np.max(np.abs(got - want)) <= 2e-3
    assert bf16_close(got, want)


def test_decode_layer_budget_covers_region_equals_dense():
    rng = np.random.default_rng(15)
    hq, hkv, n, hd = 8, 2, 300, 64
    q = rand_bf16(rng, hq, hd)
    k, v = rand_bf16(rng, hkv, n, hd), rand_bf16(rng, hkv, n, hd)
    res = orc.decode_layer(q, k, v, hkv, budget=10_000, prefix_len=4, suffix_len=16)
    g = hq // hkv
    for h in range(hkv):
        dense, _ = orc.sparse_attention(q[h * g:(h + 1) * g], k[h], v[h])
        assert np.allclose(res["out"][h * g:(h + 1) * g], dense, rtol=1e-11, atol=1e-12)
        assert sorted(res["sel"][h].tolist()) == list(range(n - 20))


@pytest.mark.parametrize("new_tok", [False, True])
def test_decode_layer_python_vs_c(new_tok):
    rng = np.random.default_rng(16)
    b, hq, hkv, n, n_max, hd = 2, 8, 2, 700, 768, 128
    g = hq // hkv
    budget, p, s = 64, 4, 16
    # small-integer keys and queries: scores are exact in any fp32 order
    k = orc.f32_to_bf16(rng.integers(-3, 4, (b, hkv, n_max, hd)).astype(np.float32))
    q = orc.f32_to_bf16((rng.integers(-2, 3, (b, hq, hd)) * 4).astype(np.float32))
    v = rand_bf16(rng, b, hkv, n_max, hd)
    nk = rand_bf16(rng, b, hkv, hd) if new_tok else None
    nv = rand_bf16(rng, b, hkv, hd) if new_tok else None
    out_c, ids_c = cpu_ref.decode_layer(
        q.reshape(b * hkv, g, hd), k.reshape(b * hkv, n_max, hd), v.reshape(b * hkv, n_max, hd),
        budget, p, s, n_ctx=n, new_k_u16=None if nk is None else nk.reshape(b * hkv, hd),
        new_v_u16=None if nv is None else nv.reshape(b * hkv, hd), n_threads=4)
    for bi in range(b):
        res = orc.decode_layer(q[bi], k[bi, :, :n], v[bi, :, :n], hkv, budget, p, s,
                               new_k_u16=None if nk is None else nk[bi],
                               new_v_u16=None if nv is None else nv[bi])
        for h in range(hkv):
            assert np.array_equal(res["sel"][h], ids_c[bi * hkv + h])
        got = orc.bf16_to_f32(out_c[bi * hkv:(bi + 1) * hkv]).reshape(hq, hd)
        assert bf16_close(got, res["out"])
