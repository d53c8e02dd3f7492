"""Pins the oracle's bounded top-k container against the reference's own unit
tests (diffcache_cpu/src/dualheap.rs:109-359): same input sequences, same
seeded LCG, same sort-and-truncate expected values, invariants checked after
every push."""
import json
import os

import pytest

from oracle import cpu_ref
from oracle import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "dualheap_vectors.json")) as f:
    GOLD = json.load(f)


def baseline_kept(all_items, cap):
    return sorted(all_items)[:cap]


def check(h, all_items, d, cap):
    kept = baseline_kept(all_items, cap)
    assert h.into_sorted_vec() == kept
    assert len(h) == len(kept)
    assert h.dth_min() == (kept[d - 1] if len(kept) >= d else None)
    assert h.kept_max() == (kept[-1] if kept else None)


class Lcg:
    def __init__(self, seed, mul, add):
        self.s, self.mul, self.add = seed, mul, add

    def next_u32(self):
        self.s = (self.s * self.mul + self.add) & 0xFFFFFFFFFFFFFFFF
        return self.s >> 32

    def next_range(self, lo, hi):
        return lo + (self.next_u32() % (hi - lo + 1))


IMPLS = [("numpy", orc.DualHeap), ("c", cpu_ref.DualHeap)]


@pytest.mark.parametrize("impl", IMPLS, ids=[i[0] for i in IMPLS])
@pytest.mark.parametrize("case", GOLD["cases"], ids=[c["name"] for c in GOLD["cases"]])
def test_fixed_sequences(impl, case):
    h = impl[1](case["d"], case["cap"])
    seen = []
    for x in case["seq"]:
        h.push(x)
        seen.append(x)
        check(h, seen, case["d"], case["cap"])


@pytest.mark.parametrize("impl", IMPLS, ids=[i[0] for i in IMPLS])
def test_known_answers_from_reference_comments(impl):
    # dualheap.rs:207-236: after 10,9,8,7,6 then 100 (discarded) then 1
    h = impl[1](5, 5)
    for x in [10, 9, 8, 7, 6, 100, 1]:
        h.push(x)
    assert h.into_sorted_vec() == [1, 6, 7, 8, 9]
    # dualheap.rs:341-357: kept_max == running max while not full
    h = impl[1](4, 10)
    run = []
    for x in [3, 1, 4, 1, 5]:
        h.push(x)
        run.append(x)
        assert h.kept_max() == max(run)
    # dualheap.rs:191-205: fewer than d items -> no d-th minimum
    h = impl[1](5, 10)
    for x in [7, 3, 9, 1]:
        h.push(x)
        assert h.dth_min() is None


@pytest.mark.parametrize("impl", IMPLS, ids=[i[0] for i in IMPLS])
def test_random_regression(impl):
    rr = GOLD["random_regression"]
    rng = Lcg(rr["seed"], rr["lcg_mul"], rr["lcg_add"])
    for d, cap in rr["configs"]:
        h = impl[1](d, cap)
        seen = []
        for _ in range(rr["pushes"]):
            x = rng.next_range(rr["lo"], rr["hi"])
            h.push(x)
            seen.append(x)
            check(h, seen, d, cap)


def test_lcg_first_values():
    # The generator itself: x1 = seed*mul+1 mod 2^64, output = high 32 bits.
    rr = GOLD["random_regression"]
    rng = Lcg(rr["seed"], rr["lcg_mul"], rr["lcg_add"])
    x1 = (rr["seed"] * rr["lcg_mul"] + 1) % (1 << 64)
    assert rng.next_u32() == x1 >> 32


def test_constructor_asserts():
    with pytest.raises(AssertionError):
        orc.DualHeap(0, 1)
    with pytest.raises(AssertionError):
        orc.DualHeap(3, 2)
    with pytest.raises(AssertionError):
        cpu_ref.DualHeap(3, 2)
