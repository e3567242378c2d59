"""Pins the oracle's in-memory world (oracle/ops.py JointWorld) with the expectations the reference keeps
next to its own 4-GPU smoke test (/root/reference/collectives.py:195-323) and round-trip identities."""
import torch

from oracle.ops import JointWorld

L = [1, 2, 3, 4]
W = 4


def _params(make):
    return [make(r).clone().requires_grad_(True) for r in range(W)]


def test_all_gather_ones():            # collectives.py:195-204: losses equal (12.5), grads are 1
    world = JointWorld(W)
    ps = _params(lambda r: torch.ones(5, r + 1))
    outs = world.all_gather("t", ps, 1, L)
    losses = [o.sum() / 4 for o in outs]
    sum(losses).backward()
    for r in range(W):
        assert outs[r].shape == (5, 10) and torch.equal(outs[r], torch.ones(5, 10))
        assert losses[r].item() == 12.5
        assert torch.equal(ps[r].grad, torch.ones(5, r + 1))


def test_all_reduce():                 # collectives.py:225-234: every element 6, loss 30, grads 1
    world = JointWorld(W)
    ps = _params(lambda r: torch.ones(5, 4) * r)
    outs = world.all_reduce("t", ps)
    losses = [o.sum() / 4 for o in outs]
    sum(losses).backward()
    for r in range(W):
        assert torch.equal(outs[r], torch.full((5, 4), 6.0)) and losses[r].item() == 30.0
        assert torch.equal(ps[r].grad, torch.ones(5, 4))


def test_reduce_scatter_ones():        # collectives.py:240-249: out = 4*ones(5, r+1), loss 20*(r+1), grads ones
    world = JointWorld(W)
    ps = _params(lambda r: torch.ones(5, 10))
    outs = world.reduce_scatter("t", ps, 1, L)
    sum(o.sum() for o in outs).backward()
    for r in range(W):
        assert torch.equal(outs[r], 4 * torch.ones(5, r + 1)) and outs[r].sum().item() == 20.0 * (r + 1)
        assert torch.equal(ps[r].grad, torch.ones(5, 10))


def test_dynamic_slice():              # collectives.py:270-279: loss 5*(r+1), grad 1 on own columns only
    for r in range(W):
        p = torch.ones(5, 10, requires_grad=True)
        out = JointWorld.dynamic_slice(p, 1, L, r)
        out.sum().backward()
        assert out.sum().item() == 5.0 * (r + 1)
        want = torch.zeros(5, 10)
        want[:, sum(L[:r]):sum(L[:r + 1])] = 1
        assert torch.equal(p.grad, want)


def test_all_to_all():                 # collectives.py:285-294: out [split[r], 10], loss 40,30,20,10, grads 1
    world = JointWorld(W)
    ps = _params(lambda r: torch.ones(10, r + 1))
    split = [4, 3, 2, 1]
    outs = world.all_to_all("t", ps, 0, 1, split, L)
    sum(o.sum() for o in outs).backward()
    for r in range(W):
        assert outs[r].shape == (split[r], 10) and outs[r].sum().item() == 10.0 * split[r]
        assert torch.equal(ps[r].grad, torch.ones(10, r + 1))


def test_all_to_all_zero_lengths():    # collectives.py:297-309
    world = JointWorld(W)
    cat = [0, 2, 0, 8]
    ps = [torch.ones(10, cat[r]) for r in range(W)]
    outs = world.all_to_all("t", ps, 0, 1, [5, 0, 5, 0], cat)
    assert [tuple(o.shape) for o in outs] == [(5, 10), (0, 10), (5, 10), (0, 10)]


def test_replicate():                  # collectives.py:314-323: loss 6.25, grads 1
    world = JointWorld(W)
    ps = _params(lambda r: torch.ones(5, 5))
    outs = world.replicate("t", ps)
    losses = [o.sum() / 4 for o in outs]
    sum(losses).backward()
    for r in range(W):
        assert losses[r].item() == 6.25 and torch.equal(ps[r].grad, torch.ones(5, 5))


def test_round_trips_and_pad_is_never_read():
    g = torch.Generator().manual_seed(0)
    world = JointWorld(W)
    full = torch.randn(6, 10, 3, generator=g)
    shards = list(torch.split(full, L, dim=1))
    outs = world.all_gather("a", shards, 1, L)
    for o in outs:
        assert torch.equal(o, full)                       # NaN pad tails never leak
    same = [full.clone() for _ in range(W)]
    red = world.reduce_scatter("b", same, 1, L)
    for r in range(W):
        torch.testing.assert_close(red[r], W * shards[r])
    # the wire log holds padded messages with the pad still poisoned
    msg = world.log[("a", "fwd")][0][1]
    assert msg.shape == (6, 4, 3) and torch.isnan(msg[:, 1:, :]).all()
