"""Programs that hap_amd.program did not generate: hand-built torch.fx graphs in the emitted node forms
(hap.rs:991-2324), run by the executor and checked against stock PyTorch autograd on the CPU executing the same
graph (the reference's execution model, worker.py:44-76)."""
import operator

import pytest
import torch
import torch.fx
import torch.nn as nn
import torch.nn.functional as F

import hap_amd
from helpers import rel_err

pytestmark = pytest.mark.gpu


class _Holder(nn.Module):
    def __init__(self, V, d, seed=0):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        mk = lambda *shape: nn.Parameter(torch.randn(*shape, generator=g) * 0.3)
        self.emb = mk(V, d)
        for i in range(4):
            setattr(self, f"w{i}", mk(d, d))
            setattr(self, f"b{i}", mk(d))
        self.dec_w, self.dec_b = mk(V, d), mk(V)


def _finish(g, t, y, d):
    logits = g.call_function(F.linear, (t, g.get_attr("dec_w"), g.get_attr("dec_b")))
    lp = g.call_function(torch.log_softmax, (logits, 2))
    lp = g.call_function(torch.transpose, (lp, 1, 2))
    g.output(g.call_function(F.nll_loss, (lp, y), {"reduction": "sum"}))
    g.lint()


def _run_both(build, V=37, d=32, B=4, S=8):
    tokens = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(1))
    targets = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(2))
    results = []
    for device in ("cpu", "gpu"):
        holder = _Holder(V, d)
        g = torch.fx.Graph()
        x, y = g.placeholder("x"), g.placeholder("y")
        h = g.call_function(F.embedding, (x, g.get_attr("emb")))
        _finish(g, build(g, h, d), y, d)
        gm = torch.fx.GraphModule(holder, g)
        if device == "cpu":
            loss = gm(tokens, targets)
            loss.backward()
            results.append((loss.item(), {n: p.grad.clone() for n, p in gm.named_parameters() if p.grad is not None}))
        else:
            ex = hap_amd.compile_program(gm, [tokens, targets], dtype="fp32")
            loss = ex.forward(tokens, targets)
            ex.backward()
            torch.cuda.synchronize()
            assert ex.shared_gradient_copies > 0           # the case the test is about did occur
            results.append((loss.item(), {n: rec["grad"].cpu() for n, rec in ex.params.items()}))
    (want, ref), (got, grads) = results
    assert abs(got - want) <= 1e-4 * abs(want)
    assert set(grads) == set(ref)
    for n in ref:
        assert rel_err(grads[n], ref[n]) < 1e-4, n


def test_second_consumer_between_a_residual_branch_and_its_add(cuda):
    """a + f(a) followed by layer_norm hands ONE gradient buffer to both a and f(a).  Here another consumer of a
    lies between f and the add in program order, so its contribution to d(a) arrives before f's backward has read
    that buffer: it must not be added in place."""
    def build(g, h, d):
        lin = lambda x, i: g.call_function(F.linear, (x, g.get_attr(f"w{i}"), g.get_attr(f"b{i}")))
        a = lin(h, 0)
        b = lin(a, 1)                       # f(a)
        c = lin(a, 2)                       # the other consumer of a, after f
        n = g.call_function(F.layer_norm, (g.call_function(operator.add, (a, b)), (d,)))
        return g.call_function(operator.add, (n, c))
    _run_both(build)


def test_relu_output_that_shares_its_gradient_buffer(cuda):
    """relu(linear(h)) + other: the add hands one gradient buffer to both operands; the relu's backward, which
    the producing linear would apply in place, must leave the other operand's gradient alone."""
    def build(g, h, d):
        lin = lambda x, i: g.call_function(F.linear, (x, g.get_attr(f"w{i}"), g.get_attr(f"b{i}")))
        other = lin(h, 0)
        r = g.call_function(F.relu, (lin(h, 1),), {"inplace": False})
        s = g.call_function(operator.add, (r, other))
        u = lin(s, 2)                       # consumes the sum, so the add is a launch of its own
        return g.call_function(operator.add, (u, lin(h, 3)))
    _run_both(build)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_mlp_of_linear_sigmoid_new_segment_and_sum(cuda, dtype):
    """The reference's MLP model (models.py:8-24): a floating-point input split over the batch, linear -> sigmoid
    (torch.sigmoid, hap.rs:1088) -> new_segment, the program's output torch.sum (hap.rs:1133)."""
    d, B, L = 64, 16, [6, 6, 2, 2]
    g0 = torch.Generator().manual_seed(3)
    xs = torch.randn(B, d, generator=g0)
    results = []
    for device in ("cpu", "gpu"):
        holder = _Holder(11, d)
        g = torch.fx.Graph()
        x, y = g.placeholder("x"), g.placeholder("y")
        h = g.call_function(operator.getitem, (g.call_method("split", (x, L, 0)), 0))
        for i in range(3):
            h = g.call_function(F.linear, (h, g.get_attr(f"w{i}"), g.get_attr(f"b{i}")))
            h = g.call_function(torch.sigmoid, (h,))
            h = g.call_function(hap_amd.models.new_segment, (h,))
        g.output(g.call_function(torch.sum, (h,)))
        g.lint()
        gm = torch.fx.GraphModule(holder, g)
        if device == "cpu":
            loss = gm(xs, None)
            loss.backward()
            results.append((loss.item(), {n: p.grad.clone() for n, p in gm.named_parameters() if p.grad is not None}))
        else:
            ex = hap_amd.compile_program(gm, [xs, (B,)], dtype=dtype)
            loss = ex.forward(xs, None)
            ex.backward()
            torch.cuda.synchronize()
            results.append((loss.item(), {n: rec["grad"].cpu() for n, rec in ex.params.items()}))
    (want, ref), (got, grads) = results
    tol = 1e-4 if dtype == "fp32" else 2e-2
    assert abs(got - want) <= tol * abs(want)
    assert set(grads) == set(ref)
    for n in ref:
        assert rel_err(grads[n], ref[n]) < tol, n


@pytest.mark.parametrize("follow", ["linear", "other_add"])
def test_append_cls_token_without_the_position_embedding_add(cuda, follow):
    """models.append_cls_token (models.py:443-445) on its own: followed by a linear, or by an add that is not the
    [1, T + 1, d] position embedding's (a same-shape tensor), then get_cls_token and a linear head with nll_loss;
    against the same arithmetic in stock PyTorch on the CPU."""
    d, B, T, C = 32, 6, 5, 7
    g0 = torch.Generator().manual_seed(5)
    xs = torch.randn(B, T, d, generator=g0)
    ys = torch.randint(0, C, (B,), generator=g0)

    def holder():
        m = _Holder(C, d)
        m.cls = nn.Parameter(torch.randn(1, 1, d, generator=torch.Generator().manual_seed(9)) * 0.3)
        return m

    m = holder()
    h = F.linear(xs, m.w0, m.b0)
    t = torch.cat((m.cls.expand(B, -1, -1), h), dim=1)
    if follow == "linear":
        t = F.linear(t, m.w1, m.b1)
    else:
        t = torch.cat((m.cls.expand(B, -1, -1), h), dim=1) + F.linear(t, m.w1, m.b1)
    want = F.nll_loss(torch.log_softmax(F.linear(t[:, 0, :], m.dec_w, m.dec_b), 1), ys, reduction="sum")
    want.backward()
    ref = {n: p.grad.clone() for n, p in m.named_parameters() if p.grad is not None}

    g = torch.fx.Graph()
    x, y = g.placeholder("x"), g.placeholder("y")
    h = g.call_function(F.linear, (x, g.get_attr("w0"), g.get_attr("b0")))
    t = g.call_function(hap_amd.models.append_cls_token, (h, g.get_attr("cls")))
    if follow == "linear":
        t = g.call_function(F.linear, (t, g.get_attr("w1"), g.get_attr("b1")))
    else:
        u = g.call_function(F.linear, (t, g.get_attr("w1"), g.get_attr("b1")))
        t2 = g.call_function(hap_amd.models.append_cls_token, (h, g.get_attr("cls")))
        t = g.call_function(operator.add, (t2, u))
    c = g.call_function(hap_amd.models.get_cls_token, (t,))
    logits = g.call_function(F.linear, (c, g.get_attr("dec_w"), g.get_attr("dec_b")))
    lp = g.call_function(torch.log_softmax, (logits, 1))
    g.output(g.call_function(F.nll_loss, (lp, y), {"reduction": "sum"}))
    g.lint()
    ex = hap_amd.compile_program(torch.fx.GraphModule(holder(), g), [xs, ys], dtype="fp32")
    got = ex.forward(xs, ys).item()
    ex.backward()
    torch.cuda.synchronize()
    grads = {n: rec["grad"].cpu() for n, rec in ex.params.items()}
    assert abs(got - want.item()) <= 1e-4 * abs(want.item())
    assert set(grads) == set(ref)
    for n in ref:
        assert rel_err(grads[n], ref[n]) < 1e-4, n
