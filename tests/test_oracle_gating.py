"""Pins oracle.ops.top_2_gating (restatement of /root/reference/models.py:477-502) and oracle.ops.switch_gating
(models.py:452-475), each with a hand-worked routing vector, a per-token brute force and the slot invariants the
algorithm implies."""
import torch
import torch.nn.functional as F

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


# ---- the C restatement of the integer part (oracle/gating_slots.c) ------------------------------------------------

def test_c_slots_on_the_hand_worked_vectors():
    v = gating_vectors()["top2"]
    index = torch.tensor([[list(ch) for ch in v["choices"]]])
    slot, tos = ref.gating_slots(index, v["E"], v["C"])
    kept = sorted([s, int(index[0, s, k]), int(slot[0, s, k])] for s in range(v["S"]) for k in range(2) if slot[0, s, k] > 0)
    assert kept == v["kept_token_expert_slot"]
    assert sorted([int(tos[0, e, c]), e, c] for e in range(v["E"]) for c in range(v["C"]) if tos[0, e, c] >= 0) == kept
    assert (tos[:, :, 0] == -1).all()                                 # slot 0 never holds a token
    w = gating_vectors()["switch"]
    index1 = torch.tensor([[[ch] for ch in w["choices"]]])
    slot1, _ = ref.gating_slots(index1, w["E"], w["C"])
    kept1 = sorted([s, int(index1[0, s, 0]), int(slot1[0, s, 0])] for s in range(w["S"]) if slot1[0, s, 0] > 0)
    assert kept1 == w["kept_token_expert_slot"]


def test_c_slots_follow_the_closed_forms():
    """One row in which every token's first choice is expert 0 and second choice expert 1: first choices take
    positions 1, 2, ..., second choices n(n+1)/2 + 1, ... -- the sum of the first-choice positions OF THEIR OWN
    expert, which is 0 for expert 1 here, so they start at 1; with the choices swapped on the second half of the row
    expert 1's second choices queue behind its n(n+1)/2."""
    S, E, C = 12, 4, 1000
    index = torch.zeros(1, S, 2, dtype=torch.int64)
    index[0, :, 1] = 1
    slot, _ = ref.gating_slots(index, E, C)
    assert slot[0, :, 0].tolist() == list(range(1, S + 1))
    assert slot[0, :, 1].tolist() == list(range(1, S + 1))            # expert 1 has no first choices: offset 0
    index[0, S // 2:, 0], index[0, S // 2:, 1] = 1, 0                  # second half: first choice 1, second choice 0
    slot, _ = ref.gating_slots(index, E, C)
    n = S // 2
    off = n * (n + 1) // 2                                            # both experts have n first choices
    assert slot[0, :, 0].tolist() == list(range(1, n + 1)) * 2
    assert slot[0, :n, 1].tolist() == [off + j for j in range(1, n + 1)]          # expert 1's second choices
    assert slot[0, n:, 1].tolist() == [off + j for j in range(1, n + 1)]          # expert 0's second choices
    slot, _ = ref.gating_slots(index, E, off + 3)                     # capacity: positions >= C are dropped
    assert slot[0, :n, 1].tolist() == [off + 1, off + 2] + [0] * (n - 2)


def test_c_slots_equal_the_dense_restatement_at_the_benchmark_shape():
    """B 16, S 512, E 16 (benchmark configuration 4) with C = 80 and C = 40: the dense PyTorch restatement of the
    reference and the C index form place the same tokens in the same slots with the same gates."""
    g = torch.Generator().manual_seed(39)
    B, S, E, d = 16, 512, 16, 64
    x, w = torch.randn(B, S, d, generator=g), torch.randn(d, E, generator=g) * 0.3
    probs = torch.softmax(x @ w, dim=2)
    gate, index = probs.topk(2, dim=2)
    for C in (80, 40):
        d_ref, c_ref = ref.top_2_gating(x, E, C, w)
        slot, tos = ref.gating_slots(index, E, C)
        d2, c2 = ref.densify_vectorised(index, slot, gate, E, C)
        assert torch.equal(d_ref, d2) and torch.equal(c_ref, c2)
        # closed form of how many choices fit: an expert with n1 first and n2 second choices in a row keeps
        # min(n1, C - 1) first choices and min(n2, max(0, C - 1 - n1 (n1 + 1) / 2)) second ones (with 32 first choices
        # per expert on average, 528 >= C, nearly every second choice is dropped at either capacity: the reference
        # offsets them by the SUM of the first-choice positions, models.py:486)
        n1 = F.one_hot(index[..., 0], E).sum(dim=1)
        n2 = F.one_hot(index[..., 1], E).sum(dim=1)
        kept1 = torch.clamp(n1, max=C - 1)
        kept2 = torch.minimum(n2, torch.clamp(C - 1 - n1 * (n1 + 1) // 2, min=0))
        assert int((slot[..., 0] > 0).sum()) == int(kept1.sum())
        assert int((slot[..., 1] > 0).sum()) == int(kept2.sum())
        assert int(kept2.sum()) < B * S // 50
        # token_of_slot is the inverse map of slot
        b, s, k = (slot > 0).nonzero(as_tuple=True)
        assert torch.equal(tos[b, index[b, s, k], slot[b, s, k]], s)
        assert int((tos >= 0).sum()) == len(b)
    d_ref, c_ref = ref.switch_gating(x, E, 40, w)
    slot1, _ = ref.gating_slots(index[..., :1], E, 40)
    d2, c2 = ref.densify_vectorised(index[..., :1], slot1, gate[..., :1], E, 40)
    assert torch.equal(d_ref, d2) and torch.equal(c_ref, c2)
