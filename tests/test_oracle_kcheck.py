"""Pins the oracle's restatement of the reference's k-check (nsw.rs:198-296).  The
reference has no tests or vectors for it, so the pins are closed forms: an exact power
law, numpy's least-squares routine, hand-computed masses and the guard clauses."""
import numpy as np
import pytest

from oracle import oracle as orc


def test_fit_alpha_recovers_an_exact_power_law():
    # z_r = c - alpha * ln(r)  =>  slope = -alpha for any window of ranks
    for alpha, c, h in [(1.7, 3.0, 100), (0.4, -2.0, 37), (2.5, 10.0, 6)]:
        r = np.arange(1, h + 1, dtype=np.float64)
        z = (c - alpha * np.log(r)).astype(np.float32)
        got = orc.fit_alpha_from_logits(z, 5)
        assert got is not None and got.dtype == np.float32
        assert abs(float(got) - alpha) < 2e-5 * max(1.0, abs(c))


def test_fit_alpha_equals_numpy_polyfit_on_noisy_data_and_ignores_the_first_ranks():
    rng = np.random.default_rng(0)
    h = 300
    z = (5 - 1.3 * np.log(np.arange(1, h + 1)) + 0.2 * rng.standard_normal(h)).astype(np.float32)
    want = -np.polyfit(np.log(np.arange(5, h + 1, dtype=np.float64)), z[4:].astype(np.float64), 1)[0]
    got = orc.fit_alpha_from_logits(z, 5)
    assert abs(float(got) - want) < 1e-6
    z2 = z.copy()
    z2[:4] += 100.0                      # ranks 1..4 are outside the fit
    assert orc.fit_alpha_from_logits(z2, 5) == got


def test_fit_alpha_guards():
    z = np.zeros(10, np.float32)
    assert orc.fit_alpha_from_logits(np.zeros(0, np.float32), 5) is None       # h == 0
    assert orc.fit_alpha_from_logits(z, 0) is None                             # min_rank == 0
    assert orc.fit_alpha_from_logits(z[:5], 5) is None                         # min_rank >= h
    assert orc.fit_alpha_from_logits(z[:6], 5) is not None                     # n == 2 is enough
    assert float(orc.fit_alpha_from_logits(z, 5)) == 0.0                       # flat logits
    # nsw.rs:15,207-210: the ln(rank) table holds MAX_EF = 16384 entries; a longer list is never fitted
    r = np.arange(1, 16386, dtype=np.float64)
    zl = (10.0 - 2.0 * np.log(r)).astype(np.float32)
    assert orc.MAX_EF == 16384
    assert abs(float(orc.fit_alpha_from_logits(zl[:16384], 5)) - 2.0) < 1e-4
    assert orc.fit_alpha_from_logits(zl[:16385], 5) is None


def test_budget_never_stops_at_a_size_beyond_max_ef():
    # a steep power law passes at every size up to 16384 and can never pass beyond it
    sq = np.sqrt(np.float32(128))
    r = np.arange(1, 20001, dtype=np.float64)
    s = ((12.0 - 3.0 * np.log(r)) * sq).astype(np.float32)
    d = orc.ref_dist(s)
    assert orc.k_check_budget(d, 128, [16384, 18000], 0.5) == 16384
    assert orc.k_check_budget(d, 128, [16385, 18000], 0.5) == 20000


def test_mass_hand_values():
    # two equal logits, alpha 3: head = 2, tail = 1 * 2 / 2 = 1  ->  2/3
    m = orc.estimate_top_h_mass(np.float32([0.5, 0.5]), 2, np.float32(3.0))
    assert abs(float(m) - 2.0 / 3.0) < 1e-7
    # logits ln4, ln2, ln1 (max ln4): head = 1 + 1/2 + 1/4, v_h = 1/4, h = 3, alpha 2 -> tail 3/4
    z = np.log(np.float64([4, 2, 1])).astype(np.float32)
    m = orc.estimate_top_h_mass(z, 3, np.float32(2.0))
    assert abs(float(m) - 1.75 / 2.5) < 1e-6
    # shift invariance (the max is subtracted) and only the first h logits matter
    m2 = orc.estimate_top_h_mass(np.concatenate([z + np.float32(40.0), np.float32([-1e9])]), 3, np.float32(2.0))
    assert abs(float(m2) - float(m)) < 1e-6
    # a steeper tail leaves more mass in the head
    assert orc.estimate_top_h_mass(z, 3, np.float32(5.0)) > m


def test_mass_guards():
    z = np.float32([1.0, 0.5])
    assert orc.estimate_top_h_mass(z, 0, np.float32(2.0)) is None
    assert orc.estimate_top_h_mass(z, 3, np.float32(2.0)) is None
    assert orc.estimate_top_h_mass(z, 2, np.float32(1.0)) is None              # alpha <= 1
    assert orc.estimate_top_h_mass(z, 2, np.float32(0.3)) is None


def test_logits_follow_the_reference_distance():
    # dist = f32(65536 - s): logits are the quantised scores over sqrt(dim)
    s = np.float32([10.0, 3.5, -2.25])
    d = orc.ref_dist(s)
    assert np.allclose(orc.k_check_logits(d, 64), s / 8.0, atol=1e-6)


def test_early_stop_and_budget_on_a_power_law():
    dim = 128
    sq = np.sqrt(np.float32(dim))
    r = np.arange(1, 2001, dtype=np.float64)

    def dists(alpha, c=20.0):
        z = c - alpha * np.log(r)
        return orc.ref_dist((z * sq).astype(np.float32))

    # alpha 3: after H rows the modelled tail is v_H * H / 2; the head dominates early
    d = dists(3.0)
    assert orc.k_check_early_stoppable(d[:100], dim, 0.9)
    assert orc.k_check_budget(d, dim, [100, 200, 400], 0.9) == 100
    # alpha 1.05: a heavy tail never reaches 0.99 within the checked sizes -> full budget
    d = dists(1.05)
    assert not orc.k_check_early_stoppable(d[:100], dim, 0.99)
    assert orc.k_check_budget(d, dim, [100, 200, 400, 800, 1600], 0.99) == 2000
    # flat scores: alpha = 0 <= 1 -> never stoppable; sizes >= ef are not checked
    flat = orc.ref_dist(np.full(50, 3.0, np.float32))
    assert orc.k_check_budget(flat, dim, [10, 20, 50, 100], 0.5) == 50
    # a threshold between the masses of two sizes picks the later one
    d = dists(1.6)
    masses = []
    for h in (100, 200, 400, 800):
        lg = orc.k_check_logits(d[:h], dim)
        masses.append(float(orc.estimate_top_h_mass(lg, h, orc.fit_alpha_from_logits(lg, 5))))
    assert masses == sorted(masses)
    thr = 0.5 * (masses[1] + masses[2])
    assert orc.k_check_budget(d, dim, [100, 200, 400, 800], thr) == 400
