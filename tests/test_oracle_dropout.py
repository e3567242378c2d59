"""Pins oracle.ops.dropout_keep, the CPU restatement of the product's counter-based dropout decisions, by what a
dropout mask must be: Bernoulli(1 - p) per element within the binomial bound, uncorrelated between neighbouring
elements (also the two that share one 32-bit hash), between steps, between streams and between seeds, identical
for identical arguments, and the exact edge cases p = 0 (all kept) and p = 1 (none kept)."""
import math

import pytest
import torch

from oracle import ops as ref

N = 1 << 20


@pytest.mark.parametrize("p", [0.1, 0.5, 0.03])
def test_keep_rate_within_the_binomial_bound(p):
    for seed, step, sid in ((0, 1, 7), (39, 12345, 203), (2 ** 40 + 5, 2 ** 33, 2 ** 35 + 1)):
        keep = ref.dropout_keep(seed, step, sid, p, N).double()
        sigma = math.sqrt(p * (1 - p) / N)
        assert abs(keep.mean().item() - (1 - p)) < 4.5 * sigma + 2.0 ** -16, (seed, step, sid)


def test_edge_probabilities_and_determinism():
    assert ref.dropout_keep(3, 1, 2, 0.0, 1001).all()
    assert not ref.dropout_keep(3, 1, 2, 1.0, 1001).any()
    a, b = ref.dropout_keep(3, 1, 2, 0.3, 1001), ref.dropout_keep(3, 1, 2, 0.3, 1001)
    assert torch.equal(a, b)
    assert torch.equal(ref.dropout_keep(3, 1, 2, 0.3, 500), a[:500])          # a prefix is a prefix


def _corr(a, b):
    a, b = a.double() - a.double().mean(), b.double() - b.double().mean()
    return (a * b).mean().item() / math.sqrt((a * a).mean().item() * (b * b).mean().item())


def test_no_correlation_between_neighbours_steps_streams_and_seeds():
    p, bound = 0.25, 4.5 / math.sqrt(N)
    base = ref.dropout_keep(11, 5, 9, p, N)
    assert abs(_corr(base[:-1], base[1:])) < bound                             # lag 1 (includes the pairs of one hash)
    assert abs(_corr(base[0::2], base[1::2])) < bound * math.sqrt(2)           # exactly the two halves of one hash
    assert abs(_corr(base[:-2], base[2:])) < bound
    assert abs(_corr(base[:-1024], base[1024:])) < bound                       # one row of a 1024-wide tensor apart
    for other in (ref.dropout_keep(11, 6, 9, p, N), ref.dropout_keep(11, 5, 10, p, N), ref.dropout_keep(12, 5, 9, p, N),
                  ref.dropout_keep(11, 5 + 2 ** 32, 9, p, N), ref.dropout_keep(11, 5, 9 + 2 ** 32, p, N)):
        assert abs(_corr(base, other)) < bound
        assert 0.3 < (base != other).double().mean().item() < 0.45            # 2 p (1 - p) = 0.375
