"""The benchmark configurations at their full per-kernel shapes (every GEMM, attention, gating, collective
copy and optimizer launch has the shape it has in the benchmark) with the depth cut to two layers, one rank with
silent peers on both sides, against the float32 CPU oracle, which is the reference's arithmetic
(stock PyTorch eager + autograd on the same generated graph).

Tolerances: the bf16 run against the float32 CPU run: 2e-2 on the loss, 3e-2 norm-wise on every gradient
that carries signal (the margin the small-size bf16 cases use as well), 8e-2 right behind a ReLU mask; the float32 run: 1e-4 on the loss, 3e-4 norm-wise on gradients (sums over 6144-16384 tokens
in a different order), 8e-4 right behind a ReLU mask, routing indices and slots bit-exact."""
import pytest
import torch

import bench
import hap_amd
from helpers import rel_err
from oracle.cpu_executor import PeerlessCPURun

pytestmark = pytest.mark.gpu


def _both(name, dtype, layers=2):
    gm_ref, x, y, meta = bench.build_workload(name, layers_override=layers)
    run = PeerlessCPURun(gm_ref, 0, "fp32")
    torch.set_num_threads(16)
    want = run.step(x, y)[0].item()
    ref_grads = {n: p.grad for n, p in gm_ref.named_parameters() if p.grad is not None}
    gm, x, y, meta = bench.build_workload(name, layers_override=layers)
    ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SilentWire(), rank=0,
                                 world_size=len(meta["ratios"]))
    loss = ex.forward(x, y)
    ex.backward()
    torch.cuda.synchronize()
    return ex, run, loss.item(), want, ref_grads


def _check_grads(ex, ref_grads, tol, tol_relu, floor=1e-4):
    """Every gradient that carries signal within ``tol`` norm-wise, except the parameters whose gradient passes
    through the ReLU mask right behind them (linear1.*, the experts' w1): the mask is a step function of the
    pre-activation, an element within rounding distance eps of zero flips it, a fraction ~eps of the elements
    does, and the norm-wise error of that gradient is ~sqrt(eps) (5e-2 for bf16, 4e-4 for float32 addends summed
    in another order): ``tol_relu``."""
    assert set(ex.params) == set(ref_grads)
    worst = {False: ("", 0.0), True: ("", 0.0)}
    scale = max(g.norm().item() for g in ref_grads.values())
    for n, rec in ex.params.items():
        ref = ref_grads[n]
        if ref.norm().item() < floor * scale:      # no signal (key bias of softmax attention): rounding noise on both sides
            continue
        err = rel_err(rec["grad"], ref)
        k = "linear1" in n or n.endswith(".w1")
        if err > worst[k][1]:
            worst[k] = (n, err)
    print("worst gradient error (plain / behind a ReLU mask):", worst[False], worst[True])
    assert worst[False][1] < tol, worst[False]
    assert worst[True][1] < tol_relu, worst[True]


def test_bert_large_shard_full_width_bf16(cuda):
    ex, run, loss, want, ref_grads = _both("bert", "bf16")
    assert abs(loss - want) <= 2e-2 * abs(want), (loss, want)
    _check_grads(ex, ref_grads, 3e-2, 8e-2)


def test_vit_large_shard_full_width_bf16(cuda):
    ex, run, loss, want, ref_grads = _both("vit", "bf16", layers=1)
    assert abs(loss - want) <= 2e-2 * abs(want), (loss, want)
    _check_grads(ex, ref_grads, 3e-2, 8e-2)


def test_moe_shard_full_width_fp32_routing_bit_exact(cuda):
    ex, run, loss, want, ref_grads = _both("moe", "fp32")
    assert abs(loss - want) <= 1e-4 * abs(want), (loss, want)
    _check_grads(ex, ref_grads, 3e-4, 8e-4)
    # dense dispatch mask and combine weights of the oracle against the GPU's routing records
    from hap_amd import models, ops
    n = 0
    for node in ex.gm.graph.nodes:
        if node.op == "call_function" and node.target is models.top_2_gating:
            dispatch, combine = run.env[0][node.name]
            B, S, E, C = dispatch.shape
            got_d, got_c = ops.top2_densify(ex.env[node].meta["r"], E, C)
            assert torch.equal(got_d.cpu().bool(), dispatch.bool())
            torch.testing.assert_close(got_c.cpu(), combine.detach().float(), rtol=1e-4, atol=1e-6)
            n += 1
    assert n == 1
