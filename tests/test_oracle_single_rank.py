"""Pins oracle.cpu_executor.SingleRankCPURun (and PeerlessCPURun, its silent-wire case), the checker of the
full-size GPU tests, on the CPU:

* fed the messages recorded from a joint run of all W ranks (JointCPURun, itself pinned against the single-device
  models), every rank's loss, parameter gradients and (after an optimizer step) parameters equal the joint
  run's, for every plan form (column-sharded FFN with its all_gather / all_to_all, pure data parallel, expert
  parallel with reduce_scatter, ZeRO-gathered parameters, head-parallel attention).  The recorded messages keep
  the NaN pads of the joint world, so any read of a pad shows;
* with zeros recorded for the peers it equals the silent-wire run (all_gather / all_to_all receive zeros,
  reductions nothing);
* with one rank (W = 1) it equals the single-device model built from stock torch.nn;
* with a SyntheticWire it receives the same seeded tensors the product's executor asks its wire for (same tags,
  directions and shapes), checked through the wire's own record of the requests.
"""
import copy

import pytest
import torch

import hap_amd
from helpers import (RATIOS4, RATIOS_E, lm_batch, make_lm, make_moe, make_vit, rank_programs, rel_err, vit_batch)
from oracle import single_device
from oracle.cpu_executor import JointCPURun, PeerlessCPURun, SingleRankCPURun

CASES = {
    "lm-column": (lambda: make_lm(), RATIOS4, 8, lambda: lm_batch(8, 16, 97), dict(ffn="column")),
    "lm-batch": (lambda: make_lm(), RATIOS4, 8, lambda: lm_batch(8, 16, 97), dict(ffn="batch")),
    "lm-column-zero": (lambda: make_lm(), RATIOS4, 8, lambda: lm_batch(8, 16, 97), dict(ffn="column", zero=True)),
    "lm-heads": (lambda: make_lm(H=8), RATIOS4, 8, lambda: lm_batch(8, 16, 97), dict(ffn="column", attn="heads")),
    "lm-sequence": (lambda: make_lm(S=19), RATIOS4, 6, lambda: lm_batch(6, 19, 97), dict(ffn="batch", shard_dim="sequence")),
    "lm-feature-embedding": (lambda: make_lm(d=40, H=4), RATIOS4, 8, lambda: lm_batch(8, 16, 97),
                             dict(ffn="column", embedding="features")),
    "lm-vocabulary-decoder": (lambda: make_lm(), RATIOS4, 8, lambda: lm_batch(8, 16, 97), dict(ffn="column", decoder="vocabulary")),
    "vit": (lambda: make_vit(), RATIOS4, 8, lambda: vit_batch(8, 16, 10), dict(ffn="batch")),
    "vit-weight-split-patches": (lambda: make_vit(), RATIOS4, 8, lambda: vit_batch(8, 16, 10),
                                 dict(ffn="batch", patch_embed="features", decoder="vocabulary")),
    "moe": (lambda: make_moe(), RATIOS_E, 16, lambda: lm_batch(16, 16, 61), dict(ffn="batch")),
    "moe-capacity": (lambda: make_moe(C=10), RATIOS_E, 16, lambda: lm_batch(16, 16, 61), dict(ffn="batch", moe="capacity")),
    "moe-hidden": (lambda: make_moe(C=10), RATIOS_E, 16, lambda: lm_batch(16, 16, 61), dict(ffn="batch", moe="hidden")),
    "moe-model": (lambda: make_moe(C=10), RATIOS_E, 16, lambda: lm_batch(16, 16, 61), dict(ffn="batch", moe="model")),
    "moe-sequence": (lambda: make_moe(C=10), RATIOS_E, 16, lambda: lm_batch(16, 16, 61), dict(ffn="batch", moe="sequence")),
    "moe-replicated-batch": (lambda: make_moe(), RATIOS_E, 4, lambda: lm_batch(4, 16, 61),
                             dict(ffn="batch", batch_sharded=False)),
}


def _grads(program):
    return {n: p.grad.clone() for n, p in program.named_parameters() if p.grad is not None}


@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_replayed_rank_equals_joint_run(case, dtype):
    make, ratios, B, batch, kw = CASES[case]
    model = make()
    x, y = batch()
    joint = JointCPURun(rank_programs(model, ratios, B, **kw), dtype)
    opts = [torch.optim.Adam(p.parameters(), lr=5e-4) for p in joint.programs]
    start = [copy.deepcopy(p.state_dict()) for p in joint.programs]
    losses = joint.step(x, y, optimizers=opts, clip_grad_norm=0.5)
    W = len(ratios)
    for r in range(W):
        prog = rank_programs(model, ratios, B, **kw)[r]
        prog.load_state_dict(start[r])
        run = SingleRankCPURun(prog, r, W, hap_amd.ReplayWire(joint.world.log, r), dtype)
        opt = torch.optim.Adam(prog.parameters(), lr=5e-4)
        loss = run.step(x, y, optimizers=[opt], clip_grad_norm=0.5)[0]
        torch.testing.assert_close(loss.float(), losses[r].float(), rtol=0, atol=0)
        want = _grads(joint.programs[r])
        got = _grads(prog)
        assert set(got) == set(want)
        for n in want:
            assert not torch.isnan(got[n]).any(), n
            torch.testing.assert_close(got[n], want[n], rtol=0, atol=0, msg=lambda m, n=n: f"{n}: {m}")
        for (n, p), (_, q) in zip(prog.named_parameters(), joint.programs[r].named_parameters()):
            torch.testing.assert_close(p, q, rtol=0, atol=0, msg=lambda m, n=n: f"{n}: {m}")


def _zero_peer_log(log, rank):
    """The recorded messages with everything the peers sent replaced by zeros."""
    out = {}
    for key, table in log.items():
        out[key] = [[torch.zeros_like(table[src][dst]) if src != rank else table[src][dst]
                     for dst in range(len(table[src]))] for src in range(len(table))]
    return out


@pytest.mark.parametrize("case", ["lm-column", "moe", "lm-column-zero"])
def test_silent_peers_equal_zero_messages(case):
    make, ratios, B, batch, kw = CASES[case]
    model = make()
    x, y = batch()
    joint = JointCPURun(rank_programs(model, ratios, B, **kw))
    joint.step(x, y)
    W, r = len(ratios), 0
    a = rank_programs(model, ratios, B, **kw)[r]
    b = rank_programs(model, ratios, B, **kw)[r]
    replay = SingleRankCPURun(a, r, W, hap_amd.ReplayWire(_zero_peer_log(joint.world.log, r), r))
    silent = PeerlessCPURun(b, r)
    assert silent.world_size == W
    la = replay.step(x, y)[0]
    lb = silent.step(x, y)[0]
    torch.testing.assert_close(la, lb, rtol=0, atol=0)
    ga, gb = _grads(a), _grads(b)
    assert set(ga) == set(gb)
    for n in ga:
        torch.testing.assert_close(ga[n], gb[n], rtol=0, atol=0, msg=lambda m, n=n: f"{n}: {m}")


def test_world_of_one_equals_single_device():
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    prog = rank_programs(model, [1.0], 8)[0]
    run = SingleRankCPURun(prog, 0, 1, hap_amd.SilentWire())
    loss = run.step(x, y)[0]
    ref = copy.deepcopy(model)
    ref.train()
    want = single_device.forward(ref, x, y)
    want.backward()
    torch.testing.assert_close(loss, want.detach(), rtol=1e-5, atol=1e-5)
    for n, p in ref.named_parameters():
        if p.grad is None:
            continue
        held = dict(prog.named_parameters()).get(n)
        if held is None or held.grad is None:
            assert ".norm" in n, n             # LayerNorm affine parameters are never read by the program
            continue
        got = held.grad
        assert rel_err(got, p.grad) < 2e-5, n


class _RecordingWire(hap_amd.SyntheticWire):
    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.requests = []

    def recv(self, tag, direction, src, shape, dtype, device, reduction=False, into=None):
        self.requests.append((tag, direction, src, tuple(shape), bool(reduction)))
        return super().recv(tag, direction, src, shape, dtype, device, reduction=reduction, into=into)


def test_seeded_peers_are_a_function_of_tag_direction_and_sender_only():
    """The seeded messages do not depend on who asks, in which order, on which device or in which element type they
    are first made (bf16 messages are the rounded float32 ones), so the CPU run and the GPU run, which ask in
    different orders, receive the same tensors."""
    a, b = hap_amd.SyntheticWire(seed=5), hap_amd.SyntheticWire(seed=5)
    cpu = torch.device("cpu")
    t1 = a.recv("all_gather_3", "fwd", 2, (4, 8), torch.float32, cpu)
    a.recv("all_to_all_1", "bwd", 1, (2, 8), torch.float32, cpu)
    b.recv("all_to_all_1", "bwd", 1, (2, 8), torch.float32, cpu)
    t2 = b.recv("all_gather_3", "fwd", 2, (4, 8), torch.bfloat16, cpu)
    torch.testing.assert_close(t1.to(torch.bfloat16), t2, rtol=0, atol=0)
    assert not torch.equal(t1, a.recv("all_gather_3", "fwd", 1, (4, 8), torch.float32, cpu))
    # forward messages are N(0, scale), backward messages N(0, grad_scale)
    big = a.recv("x", "fwd", 1, (256, 256), torch.float32, cpu)
    small = a.recv("x", "bwd", 1, (256, 256), torch.float32, cpu)
    assert abs(big.std().item() - 1.0) < 0.02 and abs(small.std().item() - 1e-3) < 2e-5


def test_single_rank_run_asks_for_every_peer_message_once_per_direction():
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    prog = rank_programs(model, RATIOS4, 8)[0]
    wire = _RecordingWire(seed=3)
    run = SingleRankCPURun(prog, 0, 4, wire)
    run.step(x, y)
    tags = [n.name for n in prog.graph.nodes if n.op == "call_function"
            and n.target in (hap_amd.collectives.all_gather, hap_amd.collectives.all_to_all)]
    assert len(tags) == 4                                   # two layers: all_gather + all_to_all each
    for tag in tags:
        for direction in ("fwd", "bwd"):
            got = sorted(src for t, d, src, _, _ in wire.requests if t == tag and d == direction)
            assert got == [1, 2, 3], (tag, direction, got)
    # shapes: the all_gather of [3, 16, 32] shards receives shards padded to the longest length
    shapes = {(t, d): s for t, d, src, s, _ in wire.requests if src == 2}
    ag = [t for t in tags if "gather" in t][0]
    aa = [t for t in tags if "all_to_all" in t][0]
    assert shapes[(ag, "fwd")] == (3, 16, 32) and shapes[(ag, "bwd")] == (3, 16, 32)
    L_F = hap_amd.sharding_lengths(64, RATIOS4)
    assert shapes[(aa, "fwd")] == (3, 16, L_F[2])           # rank 2's columns of this rank's samples
    assert shapes[(aa, "bwd")] == (1, 16, L_F[0])           # this rank's columns of rank 2's samples


def _own_decisions(run, prog):
    """The discrete decisions a finished run took itself: relu masks and expert choices, by node name."""
    import torch.nn.functional as F
    out = {}
    for node in prog.graph.nodes:
        if node.op != "call_function":
            continue
        if node.target is F.relu:
            out[node.name] = run.env[0][node.args[0].name].detach() > 0
        elif node.target is hap_amd.models.top_2_gating:
            x, wg = run.env[0][node.args[0].name], run.env[0][node.args[3].name]
            out[node.name] = torch.softmax(x.float() @ wg.float(), dim=2).topk(2, dim=2).indices
    return out


@pytest.mark.parametrize("case", ["lm-column", "moe"])
def test_a_run_given_its_own_decisions_reproduces_itself(case):
    """SingleRankCPURun(decisions=...): relu as a multiplication with a given mask and gating with given expert
    choices are the same functions as the run's own when the decisions are its own."""
    make, ratios, B, batch, kw = CASES[case]
    model = make()
    x, y = batch()
    W = len(ratios)
    a = rank_programs(model, ratios, B, **kw)[0]
    free = SingleRankCPURun(a, 0, W, hap_amd.SyntheticWire(seed=3))
    la = free.step(x, y)[0]
    decisions = _own_decisions(free, a)
    assert any(v.dtype == torch.bool for v in decisions.values())
    if case == "moe":
        assert any(v.dtype == torch.int64 for v in decisions.values())
    b = rank_programs(model, ratios, B, **kw)[0]
    lb = SingleRankCPURun(b, 0, W, hap_amd.SyntheticWire(seed=3), decisions=decisions).step(x, y)[0]
    torch.testing.assert_close(la, lb, rtol=0, atol=0)
    ga, gb = _grads(a), _grads(b)
    for n in ga:
        torch.testing.assert_close(ga[n], gb[n], rtol=1e-6, atol=1e-9, msg=lambda m, n=n: f"{n}: {m}")
    # other decisions give another result (the argument is used)
    flipped = {k: (~v if v.dtype == torch.bool else v.flip(2)) for k, v in decisions.items()}
    c = rank_programs(model, ratios, B, **kw)[0]
    SingleRankCPURun(c, 0, W, hap_amd.SyntheticWire(seed=3), decisions=flipped).step(x, y)
    gc = _grads(c)
    assert max(rel_err(gc[n], ga[n]) for n in ga if ga[n].norm() > 0) > 0.5
