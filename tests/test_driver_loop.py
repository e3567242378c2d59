"""The reference driver's loop (worker.py:47-83): statistics on the CPU, the stepped losses on the GPU against the
CPU oracle running the same loop (Adam lr 5e-4, clip_grad_norm_ 0.5): a small float32 program with silent peers, and
two layers of the BERT-large shard at full width in bf16 with seeded peers, losses and final weights."""
import copy
import math

import numpy as np
import pytest
import torch

import hap_amd
from hap_amd import driver
from helpers import RATIOS4, lm_batch, make_lm


def test_mean_std_is_numpy_population_statistics():
    vals = [0.5, 0.25, 1.0, 0.125, 2.0]
    m, s = driver.mean_std(vals)
    assert m == pytest.approx(float(np.mean(vals))) and s == pytest.approx(float(np.std(vals)))


def test_defaults_are_the_reference_configuration():
    # config.py:48-52 and worker.py:74
    assert (driver.RUN_ITER, driver.AVG_ITER, driver.LOG_ITER, driver.LR, driver.CLIP) == (100, 50, 100, 5e-4, 0.5)


@pytest.mark.gpu
def test_loop_matches_cpu_oracle(cuda):
    from oracle.cpu_executor import PeerlessCPURun
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    B, S, iters = 8, 16, 6
    gm_ref = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), B)
    run = PeerlessCPURun(gm_ref, 0, "fp32")
    opt = torch.optim.Adam(gm_ref.parameters(), lr=5e-4)
    want = [run.step(x, y, [opt], clip_grad_norm=0.5)[0].item() for _ in range(iters)]

    gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), B)
    ex = hap_amd.compile_program(gm, [x, y], dtype="fp32", wire=hap_amd.SilentWire(), rank=0, world_size=4)
    lines = []
    out = driver.train_loop(ex, x, y, batch_size=B, seqlen=S, run_iter=iters, log_iter=2, avg_iter=3, report=lines.append)
    assert out["losses"] == pytest.approx(want, rel=2e-4)
    assert want[-1] < want[0]                                           # the loop trains
    logs = [l for l in lines if l.startswith("loss (log ppl)")]
    assert [int(l.split()[3].rstrip(":")) for l in logs] == [0, 2, 4]
    # worker.py:66-70: the running sum of loss / batch / seqlen since the last report, divided by log_iter
    second = (want[1] + want[2]) / B / S / 2
    assert float(logs[1].split()[4].rstrip(",")) == pytest.approx(second, abs=2e-3)
    assert len(out["iter_times"]) == iters and all(t > 0 for t in out["iter_times"])
    assert sum(l.startswith("avg±std") for l in lines) == iters


@pytest.mark.gpu
def test_loop_on_bert_width_bf16_shard_matches_cpu_oracle(cuda):
    """Two layers of benchmark configuration 2 at full width (d 1024, 16 heads, FFN 1536 of 4096, seq 512, 12 of 32
    samples, vocabulary 30522) in bf16 with seeded N(0, 1) peers on both sides, stepped 4 times by the driver loop:
    Adam lr 5e-4 behind clip_grad_norm_(0.5) over the rank's gradients, whose norm is far above 0.5 (the loss is a sum
    over 900 masked positions), so the clipping coefficient is at work in every step.  Every step's loss and the final
    float32 masters against the CPU oracle running the same loop, at the bf16 tolerance 2e-2."""
    import bench
    from helpers import rel_err
    from oracle.cpu_executor import SingleRankCPURun
    iters, seed, tol = 4, 11, 2e-2
    gm_ref, x, y, meta = bench.build_workload("bert", layers_override=2)
    W = len(meta["ratios"])
    torch.set_num_threads(16)
    run = SingleRankCPURun(gm_ref, 0, W, hap_amd.SyntheticWire(seed=seed), "fp32", wire_dtype=torch.bfloat16)
    start = {n: p.detach().clone() for n, p in gm_ref.named_parameters()}
    opt = torch.optim.Adam(gm_ref.parameters(), lr=5e-4)
    want, norms, clear = [], [], {}
    for _ in range(iters):
        want.append(run.step(x, y, [opt], clip_grad_norm=0.5)[0].item())
        for n, p in gm_ref.named_parameters():
            if p.grad is not None:                    # elements whose gradient is clearly non-zero in every step
                big = p.grad.abs() > 0.1 * p.grad.pow(2).mean().sqrt()
                clear[n] = big if n not in clear else clear[n] & big
        # the gradients are left clipped: their norm is the clip value when the coefficient was below 1
        norms.append(math.sqrt(sum(p.grad.double().pow(2).sum().item() for p in gm_ref.parameters() if p.grad is not None)))
    assert all(abs(n - 0.5) < 5e-3 for n in norms), norms                # clipping was active in every step

    gm, _, _, _ = bench.build_workload("bert", layers_override=2)
    ex = hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=seed), rank=0, world_size=W)
    lines = []
    out = driver.train_loop(ex, x, y, batch_size=32, seqlen=512, run_iter=iters, log_iter=1, avg_iter=2, report=lines.append)
    torch.cuda.synchronize()
    print("\n  losses", out["losses"], "oracle", want)
    assert out["losses"] == pytest.approx(want, rel=tol)
    ref = dict(gm_ref.named_parameters())
    worst, worst_u = ("", 0.0), ("", 0.0)
    for n, rec in ex.params.items():
        if ref[n].grad is None:
            continue
        got, exp = rec["master"].cpu(), ref[n].detach()
        assert torch.equal(rec["shadow"].cpu(), got.to(torch.bfloat16)), n
        # Adam's normalised step follows the sign of the gradient: where the gradient is zero up to rounding (the key
        # bias of softmax attention, embedding rows of absent tokens) both runs step along rounding noise, so weights
        # and accumulated updates are compared on the elements whose gradient was above a tenth of the tensor's root
        # mean square in every step of the oracle's run
        c = clear[n]
        if not c.any():
            continue
        err = rel_err(got[c], exp[c])
        worst = max(worst, (n, err), key=lambda t: t[1])
        assert err < tol, (n, err)
        err_u = rel_err((got - start[n])[c], (exp - start[n])[c])
        worst_u = max(worst_u, (n, err_u), key=lambda t: t[1])
        assert err_u < tol, (n, err_u)
    print("  worst weight error", worst, "worst error of the accumulated update", worst_u)
    assert sum(l.startswith("loss (log ppl)") for l in lines) == iters
