"""sharding_round: the C oracle (oracle/sharding_round.c) and the product's native routine
(hapmi_sharding_round) against hand-derived known answers, invariants and an exact-arithmetic
largest-deficit simulation.  Reference rule: /root/reference/hap.rs:3536-3559."""
from fractions import Fraction

import pytest
from hypothesis import given, settings, strategies as st

import hap_amd
from oracle import ops as ref

# derived by hand from the rule (floor, then +1 at the largest deficit, ties to the LAST index)
KNOWN = [
    (8, [.375, .375, .125, .125], [3, 3, 1, 1]),
    (2048, [.375, .375, .125, .125], [768, 768, 256, 256]),
    (4096, [.375, .375, .125, .125], [1536, 1536, 512, 512]),
    (32, [.375, .375, .125, .125], [12, 12, 4, 4]),
    (128, [.375, .375, .125, .125], [48, 48, 16, 16]),
    (197, [.375, .375, .125, .125], [74, 74, 24, 25]),
    (30522, [.375, .375, .125, .125], [11446, 11446, 3815, 3815]),
    (33280, [.375, .375, .125, .125], [12480, 12480, 4160, 4160]),
    (1, [.375, .375, .125, .125], [1, 1, 1, 1]),
    (16, [.3125, .3125, .1875, .1875], [5, 5, 3, 3]),
    (10, [.25, .25, .25, .25], [2, 2, 3, 3]),     # floor 2,2,2,2; equal deficits: last index first, then index 2
    (3, [.5, .5], [1, 2]),                         # one unit left, tie -> last
    (0, [.5, .5], [0, 0]),
]

IMPLS = [("oracle", ref.sharding_round), ("product", hap_amd.sharding_lengths)]


@pytest.mark.parametrize("name,fn", IMPLS)
@pytest.mark.parametrize("n,ratios,want", KNOWN)
def test_known_answers(name, fn, n, ratios, want):
    assert fn(n, ratios) == want


def test_in_place_form_matches_reference_export():
    """hap.sharding_round(n, list) overwrites the list (hap.rs:211-218)."""
    r = [.375, .375, .125, .125]
    assert hap_amd.sharding_round(197, r) is None
    assert r == [74, 74, 24, 25]


def _exact(n, ratios):
    """Same rule in exact rational arithmetic; valid for dyadic ratios, where float64 is exact too."""
    if n == 1:
        return [1] * len(ratios)
    fr = [Fraction(r) for r in ratios]
    out = [int(r * n) for r in fr]
    while sum(out) < n:
        best, key = 0, None
        for i, r in enumerate(fr):
            k = r - Fraction(out[i], n)
            if key is None or k >= key:
                best, key = i, k
        out[best] += 1
    return out


dyadic = st.lists(st.integers(1, 64), min_size=1, max_size=8).map(
    lambda ws: [w / 256 for w in ws]).filter(lambda r: sum(r) <= 1.0)


@settings(max_examples=300, deadline=None)
@given(n=st.integers(0, 100000), ratios=dyadic)
def test_against_exact_simulation_and_invariants(n, ratios):
    total = sum(ratios)
    got_o, got_p = ref.sharding_round(n, ratios), hap_amd.sharding_lengths(n, ratios)
    assert got_o == got_p
    if n == 1:
        assert got_o == [1] * len(ratios)
        return
    if total == 1.0:
        assert got_o == _exact(n, ratios)
        assert sum(got_o) == n
        for r, l in zip(ratios, got_o):
            assert int(r * n) <= l <= int(r * n) + len(ratios)


@settings(max_examples=200, deadline=None)
@given(n=st.integers(2, 50000), raw=st.lists(st.floats(0.01, 1.0), min_size=2, max_size=8))
def test_oracle_equals_product_on_arbitrary_ratios(n, raw):
    s = sum(raw)
    ratios = [x / s * 0.999999 for x in raw]        # sums just below 1: truncation can never overshoot
    assert ref.sharding_round(n, ratios) == hap_amd.sharding_lengths(n, ratios)
    assert sum(ref.sharding_round(n, ratios)) == n


def test_overshoot_is_an_error():
    with pytest.raises(Exception):
        hap_amd.sharding_lengths(10, [0.8, 0.8])
    with pytest.raises(AssertionError):
        ref.sharding_round(10, [0.8, 0.8])
