"""Pins oracle.ops.top_2_gating (restatement of /root/reference/models.py:477-502) and oracle.ops.switch_gating
(models.py:452-475), each with a hand-worked routing vector, a per-token brute force and the slot invariants the
algorithm implies."""
import torch

from oracle import ops as ref
from helpers import gating_vector_logits, gating_vectors


def _logits_for_choices(choices, E):
    """Logits whose top-2 per token are exactly `choices` (first, second)."""
    B, S = len(choices), len(choices[0])
    lg = torch.full((B, S, E), -4.0)
    for b in range(B):
        for s, (k0, k1) in enumerate(choices[b]):
            lg[b, s, k0] = 2.0
            lg[b, s, k1] = 1.0
    return lg


def test_hand_worked_vector():
    # B=1, S=4, E=2, C=4; choices t0:(0,1) t1:(0,1) t2:(1,0) t3:(0,1)
    # first-choice positions: e0 {t0:1, t1:2, t3:3}, e1 {t2:1}; sums of positions: e0 = 6, e1 = 1
    # second-choice positions: e1 {t0:1+1, t1:2+1, t3:3+1 -> dropped (>= C)}, e0 {t2:1+6 -> dropped}
    v = gating_vectors()["top2"]
    lg = gating_vector_logits(v)
    assert torch.equal(lg, _logits_for_choices([[tuple(ch) for ch in v["choices"]]], 2))
    d, c = ref.top_2_gating(lg, v["E"], v["C"], torch.eye(2))   # gate_input @ gate_weight = logits via the identity
    kept = sorted([s, e, k] for _, s, e, k in d.nonzero().tolist())
    assert kept == v["kept_token_expert_slot"]
    probs = torch.softmax(lg, dim=2)
    assert torch.equal(c[0, 0, 0, 1], probs[0, 0, 0]) and torch.equal(c[0, 0, 1, 2], probs[0, 0, 1])
    assert torch.equal(c[0, 2, 1, 1], probs[0, 2, 1])
    assert d.dtype == torch.float32


def test_dense_restatement_equals_per_token_brute_force():
    g = torch.Generator().manual_seed(5)
    for (B, S, E, C) in [(2, 16, 4, 5), (3, 33, 8, 6), (1, 64, 16, 12), (2, 20, 4, 40)]:
        x = torch.randn(B, S, 12, generator=g)
        w = torch.randn(12, E, generator=g)
        d, c = ref.top_2_gating(x, E, C, w)
        idx, slot, gate = ref.top_2_gating_sparse(x @ w, C)
        d2, c2 = ref.densify(idx, slot, gate, E, C)
        assert torch.equal(d, d2)
        torch.testing.assert_close(c, c2, rtol=0, atol=0)


def test_slot_invariants():
    g = torch.Generator().manual_seed(7)
    B, S, E, C = 4, 48, 8, 10
    x, w = torch.randn(B, S, 16, generator=g), torch.randn(16, E, generator=g)
    d, c = ref.top_2_gating(x, E, C, w)
    assert torch.equal(d, (c > 0).float())
    assert d[:, :, :, 0].sum() == 0                      # slot 0 never holds a token
    assert (d.sum(dim=1) <= 1).all()                     # a slot holds at most one token
    assert (d.sum(dim=(2, 3)) <= 2).all()                # a token has at most two destinations
    idx, slot, gate = ref.top_2_gating_sparse(x @ w, C)
    for b in range(B):
        for e in range(E):
            first = [int(slot[b, s, 0]) for s in range(S) if idx[b, s, 0] == e]
            n = len(first)
            assert first == [p if p < C else 0 for p in range(1, n + 1)]     # 1..n in token order
            second = [int(slot[b, s, 1]) for s in range(S) if idx[b, s, 1] == e]
            want = [n * (n + 1) // 2 + j for j in range(1, len(second) + 1)]
            assert second == [p if p < C else 0 for p in want]


def test_gradient_flows_through_gates_only():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 8, 6, generator=g, requires_grad=True)
    w = torch.randn(6, 4, generator=g, requires_grad=True)
    d, c = ref.top_2_gating(x, 4, 6, w)
    assert not d.requires_grad and c.requires_grad
    c.sum().backward()
    assert w.grad.abs().sum() > 0


# ---- switch (top-1) gating: oracle.ops.switch_gating restates /root/reference/models.py:452-475 ----------------

def test_switch_hand_worked_vector():
    # B=1, S=6, E=3, C=3; first choices t0:0 t1:0 t2:2 t3:0 t4:2 t5:1
    # positions (1-based, per expert, in token order): e0 {t0:1, t1:2, t3:3 -> dropped (>= C)}, e2 {t2:1, t4:2}, e1 {t5:1}
    v = gating_vectors()["switch"]
    lg = gating_vector_logits(v)
    d, c = ref.switch_gating(lg, v["E"], v["C"], torch.eye(3))
    kept = sorted([s, e, k] for _, s, e, k in d.nonzero().tolist())
    assert kept == v["kept_token_expert_slot"]
    probs = torch.softmax(lg, dim=2)
    assert torch.equal(c[0, 1, 0, 2], probs[0, 1, 0]) and torch.equal(c[0, 5, 1, 1], probs[0, 5, 1])
    assert c[0, 3].sum() == 0                                            # the dropped token reaches no expert
    assert d.dtype == torch.float32 and d.shape == (1, 6, 3, 3)


def test_switch_dense_restatement_equals_per_token_brute_force():
    g = torch.Generator().manual_seed(15)
    for (B, S, E, C) in [(2, 16, 4, 5), (3, 33, 8, 6), (1, 64, 16, 12), (2, 20, 4, 40)]:
        x = torch.randn(B, S, 12, generator=g)
        w = torch.randn(12, E, generator=g)
        d, c = ref.switch_gating(x, E, C, w)
        idx, slot, gate = ref.switch_gating_sparse(x @ w, C)
        zeros = torch.zeros_like(idx)
        d2, c2 = ref.densify(torch.stack([idx, zeros], 2), torch.stack([slot, zeros], 2),
                             torch.stack([gate, torch.zeros_like(gate)], 2), E, C)
        assert torch.equal(d, d2)
        torch.testing.assert_close(c, c2, rtol=0, atol=0)


def test_switch_invariants_and_agreement_with_the_first_choices_of_top_2():
    g = torch.Generator().manual_seed(17)
    B, S, E, C = 4, 48, 8, 10
    x, w = torch.randn(B, S, 16, generator=g), torch.randn(16, E, generator=g)
    d, c = ref.switch_gating(x, E, C, w)
    assert torch.equal(d, (c > 0).float())
    assert d[:, :, :, 0].sum() == 0                      # slot 0 never holds a token
    assert (d.sum(dim=1) <= 1).all()                     # a slot holds at most one token
    assert (d.sum(dim=(2, 3)) <= 1).all()                # a token has at most one destination
    # the first choice of top-2 gating is routed by the same rule (models.py:485 vs :462)
    idx2, slot2, gate2 = ref.top_2_gating_sparse(x @ w, C)
    idx1, slot1, gate1 = ref.switch_gating_sparse(x @ w, C)
    assert torch.equal(idx1, idx2[:, :, 0]) and torch.equal(slot1, slot2[:, :, 0]) and torch.equal(gate1, gate2[:, :, 0])
