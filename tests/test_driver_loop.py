"""The reference driver's loop (worker.py:47-83): statistics on the CPU, the stepped losses on the GPU against the
CPU oracle running the same loop (Adam lr 5e-4, clip_grad_norm_ 0.5) with silent peers on both sides (two layers of
the BERT-large shard at full width in bf16 with seeded peers: tests/test_zzz_driver_loop_full_width.py)."""
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
