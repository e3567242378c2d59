"""Pins oracle.ops.head_parallel_attention (no reference counterpart) by the identity it must satisfy: the partial
outputs of any partition of the heads, plus the output bias, add up to torch's own
F.multi_head_attention_forward of the whole layer; and hap_amd.sharding.shard_heads_inplace, which cuts the
packed in-projection for it."""
import pytest
import torch
import torch.nn.functional as F

import hap_amd
from hap_amd.sharding import shard_heads_inplace
from oracle import ops as ref


def _layer(d, H, seed):
    torch.manual_seed(seed)
    m = torch.nn.MultiheadAttention(d, H, batch_first=True)
    with torch.no_grad():
        m.in_proj_bias.normal_(0, 0.5)
        m.out_proj.bias.normal_(0, 0.5)
    return m


@pytest.mark.parametrize("heads,causal", [([3, 3, 1, 1], True), ([1, 2, 5], False), ([8], True)])
def test_partial_outputs_of_a_head_partition_add_up_to_the_library_attention(heads, causal):
    d, H, b, S = 64, sum(heads), 3, 10
    hd = d // H
    m = _layer(d, H, 3)
    x = torch.randn(b, S, d)
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1) if causal else None
    xt = x.transpose(0, 1)
    want = F.multi_head_attention_forward(xt, xt, xt, d, H, m.in_proj_weight, m.in_proj_bias, None, None, False, 0.0,
                                          m.out_proj.weight, m.out_proj.bias, attn_mask=mask)[0].transpose(0, 1)
    total = torch.zeros_like(want)
    for r, n in enumerate(heads):
        part = torch.nn.Module()
        part.w = torch.nn.Parameter(m.in_proj_weight.detach().clone())
        part.b = torch.nn.Parameter(m.in_proj_bias.detach().clone())
        shard_heads_inplace(part, "w", heads, hd, r)
        shard_heads_inplace(part, "b", heads, hd, r)
        lo = sum(heads[:r]) * hd
        w_out = m.out_proj.weight[:, lo:lo + n * hd]
        assert part.w.shape == (3 * n * hd, d) and part.b.shape == (3 * n * hd,)
        # the kept rows are the q, k and v rows of heads [lo, lo + n)
        assert torch.equal(part.w[:n * hd], m.in_proj_weight[lo:lo + n * hd])
        assert torch.equal(part.w[2 * n * hd:], m.in_proj_weight[2 * d + lo:2 * d + lo + n * hd])
        total = total + ref.head_parallel_attention(x, part.w, part.b, w_out, n, mask)
    torch.testing.assert_close(total + m.out_proj.bias, want, rtol=1e-5, atol=1e-5)


def test_one_head_by_brute_force():
    """A single head on a single sample, looped over positions with math.exp."""
    import math
    torch.manual_seed(1)
    S, d, hd = 4, 6, 2
    x = torch.randn(1, S, d, dtype=torch.float64)
    w_in, b_in = torch.randn(3 * hd, d, dtype=torch.float64), torch.randn(3 * hd, dtype=torch.float64)
    w_out = torch.randn(d, hd, dtype=torch.float64)
    got = ref.head_parallel_attention(x, w_in, b_in, w_out, 1, None)[0]
    q = [[sum(w_in[j, k] * x[0, s, k] for k in range(d)) + b_in[j] for j in range(hd)] for s in range(S)]
    k_ = [[sum(w_in[hd + j, k] * x[0, s, k] for k in range(d)) + b_in[hd + j] for j in range(hd)] for s in range(S)]
    v = [[sum(w_in[2 * hd + j, k] * x[0, s, k] for k in range(d)) + b_in[2 * hd + j] for j in range(hd)] for s in range(S)]
    for s in range(S):
        e = [math.exp(float(sum(q[s][j] * k_[t][j] for j in range(hd))) / math.sqrt(hd)) for t in range(S)]
        ctx = [sum(e[t] / sum(e) * float(v[t][j]) for t in range(S)) for j in range(hd)]
        for c in range(d):
            assert abs(float(got[s, c]) - sum(float(w_out[c, j]) * ctx[j] for j in range(hd))) < 1e-6      # the restatement takes the softmax in float32


@pytest.mark.parametrize("causal", [True, False])
def test_attention_with_dropped_probabilities_is_the_library_attention_when_nothing_is_dropped(causal):
    d, H, b, S = 48, 4, 3, 9
    m = _layer(d, H, 5)
    xt = torch.randn(S, b, d)
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1) if causal else None
    want = F.multi_head_attention_forward(xt, xt, xt, d, H, m.in_proj_weight, m.in_proj_bias, None, None, False, 0.0,
                                          m.out_proj.weight, m.out_proj.bias, attn_mask=mask)[0]
    keep = torch.ones(b, H, S, S, dtype=torch.bool)
    got = ref.attention_with_dropped_probabilities(xt, m.in_proj_weight, m.in_proj_bias, m.out_proj.weight,
                                                   m.out_proj.bias, H, mask, keep, 0.0)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


def test_a_dropped_probability_removes_that_key_from_that_query():
    """Brute force on one head: with keep[n, h, l, s] = 0 the value of key s no longer enters query l's output, the
    kept probabilities are scaled by 1 / (1 - p) and NOT renormalised (torch drops after the softmax)."""
    import math
    torch.manual_seed(2)
    S, d = 5, 4
    x = torch.randn(S, 1, d, dtype=torch.float64)
    w_in, b_in = torch.randn(3 * d, d, dtype=torch.float64), torch.randn(3 * d, dtype=torch.float64)
    w_out, b_out = torch.eye(d, dtype=torch.float64), torch.zeros(d, dtype=torch.float64)
    keep = torch.ones(1, 1, S, S, dtype=torch.bool)
    keep[0, 0, 2, 1] = keep[0, 0, 2, 4] = keep[0, 0, 0, 0] = False
    p = 0.25
    got = ref.attention_with_dropped_probabilities(x, w_in, b_in, w_out, b_out, 1, None, keep, p)[:, 0]
    proj = x[:, 0] @ w_in.t() + b_in
    q, k, v = proj[:, :d], proj[:, d:2 * d], proj[:, 2 * d:]
    for l in range(S):
        e = [math.exp(float(q[l] @ k[s]) / math.sqrt(d)) for s in range(S)]
        want = sum((e[s] / sum(e)) / (1 - p) * v[s] for s in range(S) if keep[0, 0, l, s])
        torch.testing.assert_close(got[l], want, rtol=1e-5, atol=1e-6)      # the restatement takes the softmax in float32
