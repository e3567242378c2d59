"""The training loop of the reference driver (worker.py:47-83) on the compiled shard program.

One fixed batch is stepped ``run_iter`` times: forward -> backward -> clip_grad_norm_(0.5) over the rank's own
gradients (worker.py:74) -> Adam(lr 5e-4) step (worker.py:47, config.py:48), with the reference's two reports:

* every ``log_iter`` iterations the running sum of ``loss / batch_size / seqlen`` divided by ``log_iter``
  ("loss (log ppl)", worker.py:66-70; the reference reduces the partial losses of all ranks first, here the
  rank's own partial loss is what there is);
* every iteration its wall-clock duration and mean / standard deviation over the last ``avg_iter`` iterations
  (worker.py:78-83, config.py:50-52).

``report`` receives the formatted lines (default: stderr, as the reference's eprint); ``after_backward(it,
executor)``, if given, is called between backward and the optimizer step (the reference has no such hook; it lets a
caller log or record the step's gradients).
"""
from __future__ import annotations

import sys
import time
from typing import Callable, List, Optional

import torch

RUN_ITER, AVG_ITER, LOG_ITER, LR, CLIP = 100, 50, 100, 5e-4, 0.5        # config.py:48-52, worker.py:74


def _eprint(line: str) -> None:
    print(line, file=sys.stderr, flush=True)


def mean_std(values: List[float]):
    """numpy.mean / numpy.std (population standard deviation) as used by worker.py:83."""
    n = len(values)
    m = sum(values) / n
    return m, (sum((v - m) ** 2 for v in values) / n) ** 0.5


def train_loop(executor, x: torch.Tensor, y: torch.Tensor, *, batch_size: int, seqlen: int, run_iter: int = RUN_ITER,
               log_iter: int = LOG_ITER, avg_iter: int = AVG_ITER, lr: float = LR, clip_grad_norm: Optional[float] = CLIP,
               optimizer: str = "adam", report_per_iter_time: bool = True,
               report: Callable[[str], None] = _eprint,
               after_backward: Optional[Callable[[int, object], None]] = None) -> dict:
    executor.configure_optimizer(kind=optimizer, lr=lr, clip_grad_norm=clip_grad_norm)
    executor.load_inputs(x, y)
    times: List[float] = []
    losses: List[float] = []
    start = last = time.time()
    total = 0.0
    for it in range(run_iter):
        loss = executor.forward()
        value = float(loss.item())                     # the reference reads the loss on the host every iteration
        losses.append(value)
        total += value / batch_size / seqlen
        if it % log_iter == 0:
            report(f"loss (log ppl) {it}: {total / log_iter:.3f}, wall clock: {time.time() - start:.3f}")
            total = 0.0
        executor.backward()
        if after_backward is not None:                 # an observer of the step's gradients (before clipping)
            after_backward(it, executor)
        executor.step()
        if report_per_iter_time:
            torch.cuda.synchronize()
            d = time.time() - last
            times.append(d)
            last += d
            m, s = mean_std(times[-avg_iter:])
            report(f"iter time:  {d}")
            report(f"avg±std: {m} {s}")
    return dict(losses=losses, iter_times=times)
