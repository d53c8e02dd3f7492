"""Pins the oracle's PQ asymmetric-distance functions.  The PQ baseline has no
source in the reference (evaluation/impl/pqcache is an empty directory), so
parity with it is unpinned; these closed forms are what pins the oracle."""
import numpy as np

from oracle import oracle as orc


def test_adc_equals_dot_with_reconstructed_key():
    rng = np.random.default_rng(21)
    n, hd, m, nc = 500, 128, 32, 256
    keys = rng.standard_normal((n, hd)).astype(np.float32)
    books = orc.pq_train(keys, m, nc, iters=2, seed=7)
    codes = orc.pq_encode(keys, books)
    q = orc.f32_to_bf16(rng.standard_normal(hd).astype(np.float32))
    lut = orc.pq_build_lut(q, books)
    adc = orc.pq_adc_scores(codes, lut)
    recon = orc.pq_reconstruct(codes, books).astype(np.float64)
    assert np.allclose(adc, recon @ orc.bf16_to_f32(q).astype(np.float64), rtol=1e-12, atol=1e-12)


def test_one_point_per_cell_is_exact():
    rng = np.random.default_rng(22)
    n, hd, m = 64, 32, 8
    keys = orc.bf16_to_f32(orc.f32_to_bf16(rng.standard_normal((n, hd)).astype(np.float32)))
    books = np.stack([keys[:, j * 4:(j + 1) * 4] for j in range(m)])     # centroid i == key i
    codes = orc.pq_encode(keys, books)
    assert np.array_equal(codes, np.tile(np.arange(n, dtype=np.uint8)[:, None], (1, m)))
    q = orc.f32_to_bf16(rng.standard_normal(hd).astype(np.float32))
    adc = orc.pq_adc_scores(codes, orc.pq_build_lut(q, books))
    assert np.allclose(adc, orc.scores_f64(q, orc.f32_to_bf16(keys)), rtol=1e-12, atol=1e-12)


def test_lut_is_a_small_gemv_and_encode_is_nearest():
    rng = np.random.default_rng(23)
    m, nc, ds = 4, 16, 4
    books = rng.standard_normal((m, nc, ds)).astype(np.float32)
    q = orc.f32_to_bf16(rng.standard_normal(m * ds).astype(np.float32))
    lut = orc.pq_build_lut(q, books)
    qf = orc.bf16_to_f32(q).astype(np.float64)
    for j in range(m):
        assert np.allclose(lut[j], books[j].astype(np.float64) @ qf[j * ds:(j + 1) * ds])
    keys = rng.standard_normal((50, m * ds)).astype(np.float32)
    codes = orc.pq_encode(keys, books)
    for i in range(50):
        for j in range(m):
            d = ((books[j].astype(np.float64) - keys[i, j * ds:(j + 1) * ds]) ** 2).sum(1)
            assert codes[i, j] == d.argmin()


def test_pq_search_rerank_is_exact_topk_of_candidates():
    rng = np.random.default_rng(24)
    n, hd, m, nc = 4000, 128, 32, 64
    keys_f = rng.standard_normal((n, hd)).astype(np.float32)
    keys = orc.f32_to_bf16(keys_f)
    books = orc.pq_train(keys_f, m, nc, iters=3, seed=1)
    codes = orc.pq_encode(orc.bf16_to_f32(keys), books)
    q = orc.f32_to_bf16(rng.standard_normal(hd).astype(np.float32))
    lut = orc.pq_build_lut(q, books).astype(np.float32)
    cand, top = orc.pq_search(q, keys, codes, lut, n_cand=400, k=50)
    assert len(cand) == 400 and len(set(cand.tolist())) == 400 and len(top) == 50
    s = orc.scores_f32(q, keys)
    best = sorted(cand.tolist(), key=lambda i: (-s[i], i))[:50]
    assert top.tolist() == best
    # recall of the true top-50 inside 400 ADC candidates is high on Gaussian data
    true = set(orc.topk_select(s, 50, orc.MODE_IP).tolist())
    assert len(true & set(top.tolist())) >= 35


def test_pq_adc_fp32_order_agrees_with_float64_sum():
    """The fp32 restatement (cyclic order of additions) stays within fp32 rounding of the
    float64 sum, and is that sum exactly when the table holds small integers."""
    rng = np.random.default_rng(3)
    n, m = 3000, 32
    codes = rng.integers(0, 256, (n, m), dtype=np.uint8)
    lut = rng.standard_normal((m, 256)).astype(np.float32)
    want = orc.pq_adc_scores(codes, lut.astype(np.float64))
    got = orc.pq_adc_scores_f32(codes, lut)
    assert got.dtype == np.float32
    assert np.max(np.abs(got - want)) <= 32 * 2.0 ** -23 * np.abs(lut).max() * m
    lut_i = rng.integers(-1000, 1000, (m, 256)).astype(np.float32)
    assert np.array_equal(orc.pq_adc_scores_f32(codes, lut_i),
                          orc.pq_adc_scores(codes, lut_i.astype(np.float64)).astype(np.float32))
    # 16 subspaces, key i starts from subspace i mod 16: one key, spelled out
    lut16 = rng.standard_normal((16, 256)).astype(np.float32)
    c16 = rng.integers(0, 256, (40, 16), dtype=np.uint8)
    i = 37
    acc = np.float32(0)
    for j in range(16):
        sub = (i + j) % 16
        acc = np.float32(acc + lut16[sub, c16[i, sub]])
    assert orc.pq_adc_scores_f32(c16, lut16)[i] == acc
