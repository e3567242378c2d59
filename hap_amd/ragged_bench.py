"""Bandwidth of the device-local collective halves of the uneven-collective configuration: 8 virtual ragged shards
[S_i, 4096] bf16, S_i uniform in [1000, 3000] from the seed, packed in one GPU's HBM.

Algorithmic bytes (payload read + payload written; pad tails are not credited):
  pad            2 * sum(S) * 4096 * 2 B   (1 launch for the 8 shards)
  unpad+concat   2 * sum(S) * 4096 * 2 B   (1 launch)
  split+pad      2 * sum(S) * 4096 * 2 B   (1 launch)
  ragged reduce  9 * sum(S) * 4096 * 2 B   (1 launch for the 8 output shards: 8 reads + 1 write)
"""
from __future__ import annotations

import os
import time

import torch

from . import ops

WIDTH = 4096
HBM_PEAK = 8000.0


def _time(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps * 1e-3


# HBM bytes of one ragged_reduce launch on the seeded workload below, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch: 501861.1 and 125456.0), the fetch counter scaled by 2.0: the factor at which
# the plain unpad+concat copy of the same 125456 KiB payload reads its known size (it counts 62774.0 KiB).
PROFILED_S = [2201, 1374, 2567, 2270, 1333, 2391, 1194, 2352]
PROFILED_REDUCE_TRAFFIC = int((501861.1 * 2.0 + 125456.0) * 1024)


def run(steps: int = 50, warmup: int = 10, cpu_baseline: bool = True) -> dict:
    ops.init()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(39)
    S = torch.randint(1000, 3001, (8,), generator=g).tolist()
    m, total = max(S), sum(S)
    shards_cpu = [torch.randn(s, WIDTH, generator=g).bfloat16() for s in S]
    shards = [x.to(dev) for x in shards_cpu]
    padded = [torch.empty(m, WIDTH, dtype=torch.bfloat16, device=dev) for _ in S]
    full = torch.empty(total, WIDTH, dtype=torch.bfloat16, device=dev)
    fulls = [torch.randn(total, WIDTH, generator=g).bfloat16().to(dev) for _ in range(8)]
    outs = [torch.empty(s, WIDTH, dtype=torch.bfloat16, device=dev) for s in S]
    offs = [sum(S[:r]) for r in range(8)]
    payload = total * WIDTH * 2

    def pad_all():
        ops.pad_rows_multi(shards, 0, m, padded)

    def reduce_all():
        ops.ragged_reduce_multi(fulls, 0, offs, S, outs)

    t_pad = _time(pad_all, steps, warmup)
    t_cat = _time(lambda: ops.unpad_concat(padded, S, 0, full), steps, warmup)
    t_split = _time(lambda: ops.split_pad(full, S, 0, m, padded), steps, warmup)
    t_red = _time(reduce_all, steps, warmup)
    gbs = {"pad": 2 * payload / t_pad / 1e9, "unpad_concat": 2 * payload / t_cat / 1e9,
           "split_pad": 2 * payload / t_split / 1e9, "ragged_reduce": 9 * payload / t_red / 1e9}
    step_bytes = (2 + 2 + 2 + 9) * payload
    step_time = t_pad + t_cat + t_split + t_red
    result = {
        "metric": "GB/s of the device-local uneven-collective kernels (pad, unpad+concat, split+pad, ragged reduce)",
        "value": step_bytes / step_time / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": step_time * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "8 ragged shards [S_i, 4096] bf16, S_i in [1000, 3000] (seed 39)", "S": S,
                   "per_kernel_GBps": gbs},
        "roofline": {"bound": "hbm", "kernel": "ragged_reduce_kernel<bf16, 8>", "achieved": gbs["ragged_reduce"],
                     "peak": HBM_PEAK, "unit": "GB/s", "frac": gbs["ragged_reduce"] / HBM_PEAK,
                     "algorithmic_bytes": 9 * payload,
                     "traffic": PROFILED_REDUCE_TRAFFIC if S == PROFILED_S else None},
    }
    if cpu_baseline:
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        fulls_cpu = [f.cpu() for f in fulls[:8]]
        t0 = time.perf_counter()
        n = 0
        while n < 2 or time.perf_counter() - t0 < 10.0:
            pads = [torch.cat([x, torch.empty(m - x.shape[0], WIDTH, dtype=x.dtype)], 0) for x in shards_cpu]
            cat = torch.cat([p.split([s, m - s], 0)[0] for p, s in zip(pads, S)], 0)
            [torch.cat([p, torch.empty(m - p.shape[0], WIDTH, dtype=p.dtype)], 0) for p in torch.split(cat, S, 0)]
            for r in range(8):
                acc = fulls_cpu[0][offs[r]:offs[r] + S[r]].float()
                for f in fulls_cpu[1:]:
                    acc = acc + f[offs[r]:offs[r] + S[r]].float()
                acc.bfloat16()
            n += 1
        t_cpu = (time.perf_counter() - t0) / n
        result["cpu_baseline"] = {"value": step_bytes / t_cpu / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
                                  "sample": f"torch CPU cat/split/sum of the same shards, {n} passes"}
    return result
