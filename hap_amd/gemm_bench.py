"""Time of one GEMM shape under each tile configuration of the library (bf16 operands and results).

    python3 -m hap_amd.gemm_bench M N K transA transB [--configs 1,3,7] [--launches 10] [--quiet]

For every configuration: the median time of a single launch with cold caches (each launch behind a write over a
512 MB buffer) and the mean of 20 launches back to back on the same operands.  With ``--quiet --configs C`` it
only issues ``--launches`` cold launches of configuration C, which is the form to put behind
``rocprofv3 --pmc ... --`` or ``--kernel-trace``: the profiler's per-dispatch rows are then that one kernel.
"""
from __future__ import annotations

import argparse

import torch

from . import ops
from ._lib import lib

BF16_CONFIGS = tuple(range(10))


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("M", type=int)
    ap.add_argument("N", type=int)
    ap.add_argument("K", type=int)
    ap.add_argument("transA", type=int, help="1: A stored [K, M]")
    ap.add_argument("transB", type=int, help="1: B stored [N, K]")
    ap.add_argument("--configs", default=",".join(str(c) for c in BF16_CONFIGS))
    ap.add_argument("--launches", type=int, default=10)
    ap.add_argument("--quiet", action="store_true", help="launch only (for profiler runs)")
    args = ap.parse_args(argv)
    ops.init()
    dev = torch.device("cuda:0")
    M, N, K, tA, tB = args.M, args.N, args.K, bool(args.transA), bool(args.transB)
    A = torch.randn((K, M) if tA else (M, K), device=dev).bfloat16()
    B = torch.randn((N, K) if tB else (K, N), device=dev).bfloat16()
    C = torch.zeros(M, N, device=dev, dtype=torch.bfloat16)
    flush = torch.zeros(512 << 20, dtype=torch.int8, device=dev)

    def launch():
        ops.gemm(A, B, C, M, N, K, transA=tA, transB=tB)

    def cold(n):
        ts = []
        for _ in range(n):
            flush.add_(1)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            launch()
            e1.record()
            e1.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e3)
        return sorted(ts)[n // 2]

    def warm(n=20):
        for _ in range(3):
            launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            launch()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    flop = 2.0 * M * N * K
    try:
        for cfg in (int(c) for c in args.configs.split(",")):
            lib().hapmi_gemm_tuning(cfg, 1)
            if args.quiet:
                cold(args.launches)
                continue
            c_us, w_us = cold(args.launches), warm()
            print(f"M {M} N {N} K {K} {'T' if tA else 'N'}{'T' if tB else 'N'} config {cfg}: cold {c_us:7.1f} us "
                  f"{flop / c_us / 1e6:6.0f} TFLOP/s, back to back {w_us:7.1f} us {flop / w_us / 1e6:6.0f} TFLOP/s", flush=True)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)
    torch.cuda.synchronize()


if __name__ == "__main__":
    main()
