"""Top-2 and switch gating and the dispatch / combine gathers on the GPU: routing (expert index, slot, dropped flags,
dense layouts) is bit-exact against the oracle on the same float32 logits; gate values and the float paths
within tolerance.  Reference: /root/reference/models.py:477-502, 452-475, 356-364."""
import pytest
import torch

from hap_amd import ops
from oracle import ops as ref
from helpers import gating_vector_logits, gating_vectors, rel_err

pytestmark = pytest.mark.gpu

SHAPES = [(1, 4, 2, 4), (2, 16, 4, 5), (3, 33, 8, 6), (2, 512, 16, 80), (2, 512, 16, 40), (1, 700, 16, 20),
          (4, 64, 64, 3)]


def _logits(B, S, E, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, S, E, generator=g)


def test_hand_worked_vector(cuda):
    v = gating_vectors()["top2"]
    r = ops.top2_gate(gating_vector_logits(v).to(cuda), v["C"])
    assert r["index"].cpu().tolist() == [v["choices"]]
    assert r["slot"].cpu().tolist() == [v["slot"]]
    assert r["token_of_slot"].cpu()[0].tolist() == v["token_of_slot"]


@pytest.mark.parametrize("B,S,E,C", SHAPES)
def test_routing_is_bit_exact(cuda, B, S, E, C):
    lg = _logits(B, S, E, S + E)
    r = ops.top2_gate(lg.to(cuda), C)
    idx, slot, gate = ref.top_2_gating_sparse(lg, C)
    assert torch.equal(r["index"].cpu().long(), idx)
    assert torch.equal(r["slot"].cpu().long(), slot)
    torch.testing.assert_close(r["gate"].cpu(), gate, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(r["probs"].cpu(), torch.softmax(lg, 2), rtol=1e-5, atol=1e-7)
    # dense layouts against the restated reference computation on the same logits
    d_ref, c_ref = ref.top_2_gating(lg, E, C, torch.eye(E))
    d, c = ops.top2_densify(r, E, C)
    assert torch.equal(d.cpu(), d_ref)
    assert torch.equal((c.cpu() > 0), (c_ref > 0))
    torch.testing.assert_close(c.cpu(), c_ref, rtol=1e-5, atol=1e-7)
    # inverse map
    tos = r["token_of_slot"].cpu()
    nz = d_ref.nonzero()
    assert (tos >= 0).sum().item() == nz.shape[0]
    for b, s, e, k in nz.tolist()[:200]:
        assert tos[b, e, k] == s


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [(2, 3, 0, 10, 0, 48), (2, 3, 4, 3, 0, 48), (0, 8, 0, 5, 0, 48), (0, 8, 7, 3, 0, 48),
                                    (0, 8, 0, 10, 0, 17), (0, 8, 0, 10, 17, 19), (0, 8, 0, 10, 36, 12), (2, 3, 4, 3, 17, 19),
                                    (0, 8, 0, 10, 20, 0)])
def test_dispatch_combine_match_dense_einsums(cuda, dtype, window):
    """The device's share of the dense [B, S, E, C] dispatch / combine tensors is a window of experts, of capacity
    slots and of positions (dynamic_slice on dim 2 / dim 3 / dim 1): whole capacity, a capacity range, a range that
    holds slot 0 (always empty) next to the whole expert range; the first, a middle and the last range of positions
    (token tensors then hold those positions only), all three windows at once, and an empty range of positions."""
    B, S, E, C, d = 2, 48, 8, 10, 32
    e_lo, E_loc, c_lo, C_loc, s_lo, S_loc = window
    g = torch.Generator().manual_seed(9)
    lg = torch.randn(B, S, E, generator=g)
    x = torch.randn(B, S, d, generator=g).to(dtype)
    r = ops.top2_gate(lg.to(cuda), C)
    dispatch, combine = ref.top_2_gating(lg, E, C, torch.eye(E))
    pos = slice(s_lo, s_lo + S_loc)
    dsl = dispatch[:, pos, e_lo:e_lo + E_loc, c_lo:c_lo + C_loc]
    csl = combine[:, pos, e_lo:e_lo + E_loc, c_lo:c_lo + C_loc]
    xs = x[:, pos].contiguous()
    ei = torch.full((E_loc, B, C_loc, d), float("nan"), dtype=dtype, device=cuda)
    ops.moe_dispatch(xs.to(cuda), r, ei, E, C, e_lo, E_loc, c_lo, C_loc, s_lo)
    want_ei = torch.einsum("bsd,bsec->becd", xs.float(), dsl)
    assert torch.equal(ei.float().cpu().permute(1, 0, 2, 3), want_ei)            # a gather: exact
    eo = torch.randn(E_loc, B, C_loc, d, generator=g).to(dtype)
    out = torch.full((B, S_loc, d), float("nan"), dtype=dtype, device=cuda)
    ops.moe_combine(eo.to(cuda), r, out, C, e_lo, E_loc, c_lo, C_loc, s_lo)
    want_out = torch.einsum("becd,bsec->bsd", eo.float().permute(1, 0, 2, 3), csl)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    if S_loc:
        assert rel_err(out, want_out) < tol
    # backward of combine and dispatch against autograd on the dense einsums
    dout = torch.randn(B, S_loc, d, generator=g).to(dtype)
    eo_a = eo.float().permute(1, 0, 2, 3).clone().requires_grad_(True)
    c_a = csl.clone().requires_grad_(True)
    torch.einsum("becd,bsec->bsd", eo_a, c_a).backward(dout.float())
    d_eo = torch.full((E_loc, B, C_loc, d), float("nan"), dtype=dtype, device=cuda)
    dgate = torch.full((B, S, 2), float("nan"), dtype=torch.float32, device=cuda)
    ops.moe_combine_bwd(dout.to(cuda), eo.to(cuda), r, d_eo, dgate, E, C, e_lo, E_loc, c_lo, C_loc, s_lo)
    if S_loc:
        assert rel_err(d_eo.float().cpu().permute(1, 0, 2, 3), eo_a.grad) < tol
    else:
        assert not d_eo.any()
    idx, slot = r["index"].cpu().long(), r["slot"].cpu().long()
    want_dgate = torch.zeros(B, S, 2)
    for b in range(B):
        for s in range(s_lo, s_lo + S_loc):
            for k in range(2):
                e = idx[b, s, k].item() - e_lo
                c = slot[b, s, k].item() - c_lo
                if slot[b, s, k] > 0 and 0 <= e < E_loc and 0 <= c < C_loc:
                    want_dgate[b, s, k] = c_a.grad[b, s - s_lo, e, c]
    if S_loc:
        assert rel_err(dgate, want_dgate) < tol
    assert torch.equal(dgate.cpu() == 0, want_dgate == 0) or dtype == torch.bfloat16     # exact zeros outside the windows
    assert not dgate.cpu()[:, :s_lo].any() and not dgate.cpu()[:, s_lo + S_loc:].any()
    d_ei = torch.randn(E_loc, B, C_loc, d, generator=g).to(dtype)
    x_a = xs.float().clone().requires_grad_(True)
    torch.einsum("bsd,bsec->becd", x_a, dsl).backward(d_ei.float().permute(1, 0, 2, 3))
    dx = torch.full((B, S_loc, d), float("nan"), dtype=dtype, device=cuda)
    ops.moe_dispatch_bwd(d_ei.to(cuda), r, dx, C, e_lo, E_loc, False, c_lo, C_loc, s_lo)
    if S_loc:
        assert rel_err(dx, x_a.grad) < tol


def test_gate_backward_matches_autograd(cuda):
    B, S, E, C, d = 2, 24, 8, 8, 16
    g = torch.Generator().manual_seed(12)
    x = torch.randn(B, S, d, generator=g)
    w = torch.randn(d, E, generator=g).requires_grad_(True)
    xr = x.clone().requires_grad_(True)
    dispatch, combine = ref.top_2_gating(xr, E, C, w)
    dc = torch.randn(B, S, E, C, generator=g)
    combine.backward(dc)
    logits = (x @ w.detach())
    r = ops.top2_gate(logits.to(cuda), C)
    idx, slot = r["index"].cpu().long(), r["slot"].cpu().long()
    dgate = torch.zeros(B, S, 2)
    for b in range(B):
        for s in range(S):
            for k in range(2):
                if slot[b, s, k] > 0:
                    dgate[b, s, k] = dc[b, s, idx[b, s, k], slot[b, s, k]]
    dlogits = torch.empty(B, S, E, device=cuda)
    ops.top2_gate_bwd(r, dgate.to(cuda), dlogits)
    want_dw = x.reshape(-1, d).t() @ dlogits.cpu().reshape(-1, E)
    assert rel_err(want_dw, w.grad) < 1e-4
    assert rel_err(dlogits.cpu().reshape(-1, E) @ w.detach().t(), xr.grad.reshape(-1, d)) < 1e-4


# ---- switch (top-1) gating, /root/reference/models.py:452-475 ---------------------------------------------------

def test_switch_hand_worked_vector(cuda):
    v = gating_vectors()["switch"]
    lg = gating_vector_logits(v)
    lg = torch.cat([lg, torch.full((1, v["S"], 1), -9.0)], 2)     # the kernel's GEMM path wants E % 4 == 0; expert 3 unused
    r = ops.switch_gate(lg.to(cuda), v["C"])
    assert r["index"].cpu()[0, :, 0].tolist() == v["choices"]
    assert r["slot"].cpu()[0].tolist() == v["slot"]
    assert r["gate"].cpu()[0, :, 1].tolist() == [0.0] * v["S"]
    assert r["token_of_slot"].cpu()[0].tolist() == v["token_of_slot"] + [[-1] * v["C"]]


@pytest.mark.parametrize("B,S,E,C", SHAPES)
def test_switch_routing_is_bit_exact(cuda, B, S, E, C):
    lg = _logits(B, S, E, 3 * S + E)
    r = ops.switch_gate(lg.to(cuda), C)
    idx, slot, gate = ref.switch_gating_sparse(lg, C)
    assert torch.equal(r["index"].cpu().long()[:, :, 0], idx)
    assert torch.equal(r["slot"].cpu().long()[:, :, 0], slot)
    assert (r["slot"].cpu()[:, :, 1] == 0).all() and (r["gate"].cpu()[:, :, 1] == 0).all()
    torch.testing.assert_close(r["gate"].cpu()[:, :, 0], gate, rtol=1e-5, atol=1e-7)
    d_ref, c_ref = ref.switch_gating(lg, E, C, torch.eye(E))
    d, c = ops.top2_densify(r, E, C)
    assert torch.equal(d.cpu(), d_ref)
    torch.testing.assert_close(c.cpu(), c_ref, rtol=1e-5, atol=1e-7)
    tos = r["token_of_slot"].cpu()
    assert (tos >= 0).sum().item() == int(d_ref.sum().item())
    for b, s, e, k in d_ref.nonzero().tolist()[:200]:
        assert tos[b, e, k] == s


def test_switch_gate_backward_is_the_softmax_backward_of_the_kept_choice(cuda):
    B, S, E, C = 2, 40, 8, 6
    lg = _logits(B, S, E, 77)
    r = ops.switch_gate(lg.to(cuda), C)
    g = torch.Generator().manual_seed(78)
    dgate = torch.randn(B, S, 2, generator=g)
    dlogits = torch.empty(B, S, E, device=cuda)
    ops.top2_gate_bwd(r, dgate.to(cuda), dlogits)
    x = lg.clone().requires_grad_(True)
    p = torch.softmax(x, 2)
    idx, slot, _ = ref.switch_gating_sparse(lg, C)
    chosen = p.gather(2, idx[:, :, None]).squeeze(2)
    (chosen * dgate[:, :, 0] * (slot > 0)).sum().backward()
    torch.testing.assert_close(dlogits.cpu(), x.grad, rtol=1e-5, atol=1e-7)
