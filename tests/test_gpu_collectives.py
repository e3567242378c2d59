"""hap_amd.collectives (the drop-in functions) on the GPU, one rank at a time with the peers' messages replayed
from the CPU world: the reference's own ones-tensor expectations (/root/reference/collectives.py:195-323)."""
import pytest
import torch

import hap_amd
from hap_amd import collectives as C
from oracle.ops import JointWorld

pytestmark = pytest.mark.gpu
L = [1, 2, 3, 4]
W = 4


def _world_log(kind, make, call):
    world = JointWorld(W)
    ps = [make(r).clone().requires_grad_(True) for r in range(W)]
    outs = call(world, ps)
    return world, ps, outs


def _run_rank(cuda, r, log_key_map, world, make, fn, loss_of):
    wire = hap_amd.ReplayWire({(log_key_map, d): world.log[("t", d)] for d in ("fwd", "bwd") if ("t", d) in world.log}, r)
    wire.world_size, wire.rank = W, r
    C.set_wire(wire)
    p = make(r).to(cuda).requires_grad_(True)
    out = fn(p, r)
    loss = loss_of(out)
    loss.backward()
    return out.detach().cpu(), loss.item(), p.grad.cpu()


def test_all_gather(cuda):
    make = lambda r: torch.ones(5, r + 1)
    world, ps, outs = _world_log("ag", make, lambda w, ps: w.all_gather("t", ps, 1, L))
    sum(o.sum() / 4 for o in outs).backward()
    for r in range(W):
        out, loss, grad = _run_rank(cuda, r, "all_gather#0", world, make, lambda p, r: C.all_gather(p, 1, L, r),
                                    lambda o: o.sum() / 4)
        assert torch.equal(out, torch.ones(5, 10)) and loss == 12.5 and torch.equal(grad, torch.ones(5, r + 1))


def test_reduce_scatter(cuda):
    make = lambda r: torch.ones(5, 10)
    world, ps, outs = _world_log("rs", make, lambda w, ps: w.reduce_scatter("t", ps, 1, L))
    sum(o.sum() for o in outs).backward()
    for r in range(W):
        out, loss, grad = _run_rank(cuda, r, "reduce_scatter#0", world, make,
                                    lambda p, r: C.reduce_scatter(p, 1, L, r), lambda o: o.sum())
        assert torch.equal(out, 4 * torch.ones(5, r + 1)) and loss == 20.0 * (r + 1)
        assert torch.equal(grad, torch.ones(5, 10))


def test_all_reduce_and_replicate(cuda):
    make = lambda r: torch.ones(5, 4) * r
    world, ps, outs = _world_log("ar", make, lambda w, ps: w.all_reduce("t", ps))
    sum(o.sum() / 4 for o in outs).backward()
    for r in range(W):
        out, loss, grad = _run_rank(cuda, r, "all_reduce#0", world, make, lambda p, r: C.all_reduce(p),
                                    lambda o: o.sum() / 4)
        assert torch.equal(out, torch.full((5, 4), 6.0)) and loss == 30.0 and torch.equal(grad, torch.ones(5, 4))
    make = lambda r: torch.ones(5, 5)
    world, ps, outs = _world_log("rp", make, lambda w, ps: w.replicate("t", ps))
    sum(o.sum() / 4 for o in outs).backward()
    for r in range(W):
        out, loss, grad = _run_rank(cuda, r, "replicate#0", world, make, lambda p, r: C.replicate(p),
                                    lambda o: o.sum() / 4)
        assert loss == 6.25 and torch.equal(grad, torch.ones(5, 5))


def test_dynamic_slice(cuda):
    C.set_wire(hap_amd.SilentWire())
    for r in range(W):
        p = torch.ones(5, 10, device=cuda, requires_grad=True)
        out = C.dynamic_slice(p, 1, L, r)
        out.sum().backward()
        want = torch.zeros(5, 10)
        want[:, sum(L[:r]):sum(L[:r + 1])] = 1
        assert out.sum().item() == 5.0 * (r + 1) and torch.equal(p.grad.cpu(), want)


def test_all_to_all_and_zero_lengths(cuda):
    make = lambda r: torch.ones(10, r + 1)
    split = [4, 3, 2, 1]
    world, ps, outs = _world_log("aa", make, lambda w, ps: w.all_to_all("t", ps, 0, 1, split, L))
    sum(o.sum() for o in outs).backward()
    for r in range(W):
        out, loss, grad = _run_rank(cuda, r, "all_to_all#0", world, make,
                                    lambda p, r: C.all_to_all(p, 0, 1, split, L, r), lambda o: o.sum())
        assert out.shape == (split[r], 10) and loss == 10.0 * split[r] and torch.equal(grad, torch.ones(10, r + 1))
    cat = [0, 2, 0, 8]
    make = lambda r: torch.ones(10, cat[r])
    world, ps, outs = _world_log("az", make, lambda w, ps: w.all_to_all("t", ps, 0, 1, [5, 0, 5, 0], cat))
    shapes = []
    for r in range(W):
        wire = hap_amd.ReplayWire({("all_to_all#0", "fwd"): world.log[("t", "fwd")]}, r)
        C.set_wire(wire)
        shapes.append(tuple(C.all_to_all(make(r).to(cuda), 0, 1, [5, 0, 5, 0], cat, r).shape))
    assert shapes == [(5, 10), (0, 10), (5, 10), (0, 10)]
