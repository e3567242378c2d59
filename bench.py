#!/usr/bin/env python3
"""Throughput of one GPU's uneven shard: fwd + bwd + optimizer step of the generated SPMD program.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload bert|lm|vit|moe|ragged]

Default workload (N = 1): the headline configuration -- BERT-large-style encoder, bf16 compute with float32 master
weights, 24 layers, d 1024, 16 heads, FFN 4096 column-split to a local 1536 slice, seq 512, local batch 12
of 32, vocab 30522, 15 % masked-LM targets, Adam.  Inputs are synthetic (seeded), resident in HBM before the
timed region; the peers' halves of the collectives come from a seeded synthetic wire (one set of message buffers per
layer).  The line's `extra` object carries the other configurations (2-layer float32 LM, ViT-L/16, MoE, the ragged
collective kernels), each measured the same way with fewer steps.
Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

RATIOS = [.375, .375, .125, .125]
RATIOS_E = [.3125, .3125, .1875, .1875]
PEAK = {"bf16": 2500.0, "fp32": 157.3}        # dense MFMA TFLOP/s, MI355X
HBM_PEAK = 8000.0                              # GB/s

# OFFLINE constants, not measured by a bench run: counted on the default workload with the commands of
# profiles/bert_large_shard_step.counters.md: 87 852 KiB fetched (x 2.0) + 33 629 KiB written per GEMM launch; every
# operand read and every result written once: 19.3 GB per step in 207 launches.  They belong to the GEMM plan below
# (signature (M, N, K, batch, transA, transB, in, out) -> (tile configuration, K splits): the plan file that the
# profile's commands name); a run whose autotuned plan or launch count differs reports no traffic.
PROFILED_GEMM_TRAFFIC_PER_LAUNCH = (2.0 * 87852 + 33629) * 1024
PROFILED_GEMM_LAUNCHES_PER_STEP = 207
PROFILED_GEMM_ALGORITHMIC_BYTES_PER_LAUNCH = 19.3e9 / PROFILED_GEMM_LAUNCHES_PER_STEP
PROFILED_GEMM_PLAN = {
    (1024, 1024, 6144, 8, 1, 0, 1, 0): (6, 1), (1024, 4096, 6144, 8, 1, 0, 1, 0): (1, 1),
    (1536, 1024, 16384, 8, 1, 0, 1, 0): (3, 1), (3072, 1024, 6144, 8, 1, 0, 1, 0): (3, 1),
    (6144, 1024, 1024, 1, 0, 0, 1, 1): (7, 1), (6144, 1024, 1024, 1, 0, 1, 1, 1): (7, 1),
    (6144, 1024, 3072, 1, 0, 0, 1, 1): (7, 1), (6144, 1024, 4096, 1, 0, 1, 1, 1): (7, 1),
    (6144, 1024, 30522, 1, 0, 0, 1, 1): (3, 2), (6144, 3072, 1024, 1, 0, 1, 1, 1): (9, 1),
    (6144, 4096, 1024, 1, 0, 0, 1, 1): (6, 1), (6144, 30522, 1024, 1, 0, 1, 1, 1): (4, 1),
    (16384, 1024, 1536, 1, 0, 0, 1, 1): (1, 1), (16384, 1536, 1024, 1, 0, 1, 1, 1): (6, 1),
    (30522, 1024, 6144, 1, 1, 0, 1, 0): (1, 1),
}

WORKLOADS = {
    # name: (description, dtype)
    "bert": ("BERT-large uneven shard: 24L d1024 h16 FFN 1536/4096 seq512 batch 12/32 vocab30522 MLM Adam", "bf16"),
    "lm": ("2-layer post-LN LM: d512 h8 FFN 768/2048 seq128 batch 3/8 vocab33280 SGD", "fp32"),
    "vit": ("ViT-L/16: 24L d1024 h16 FFN4096 197 tokens batch 48/128 1000 classes Adam", "bf16"),
    "moe": ("MoE LM: 12L d768 h12 16 experts (5 local) top-2 C=80 seq512 batch 16 vocab33280 Adam", "bf16"),
}
# capacity slots per expert of the MoE workload: ceil(512 / 16 * 2.5) = 80 by the reference's rule (config.py:25-28
# doubles the capacity factor 1.25 for models whose name ends in `moe`); 40 if the factor is taken as it stands
MOE_CAPACITY = 80


def build_workload(name, layers_override=None, attn="batch", zero=False, dropout=0.0, capacity=None):
    import torch
    import hap_amd
    from hap_amd import models
    g = torch.Generator().manual_seed(39)
    if name == "bert":
        L = layers_override or 24
        B, S, V = 32, 512, 30522
        model = models.RTransformer(V, S, 1024, 16, 4096, 0.0, nlayers=L, causal=False)
        x = torch.randint(0, V, (B, S), generator=g)
        masked = torch.rand(B, S, generator=g) < 0.15
        y = torch.where(masked, x, torch.full_like(x, -100))
        plan = hap_amd.ShardingPlan([RATIOS], 0, ffn="column", attn=attn, zero=zero)
        meta = dict(local_batch=12, global_batch=B, seq_len=S, opt=dict(kind="adam", lr=5e-4), batch_sharded=True,
                    ratios=RATIOS)
    elif name == "lm":
        L = layers_override or 2
        B, S, V = 8, 128, 33280
        model = models.RTransformer(V, S, 512, 8, 2048, 0.0, nlayers=L, causal=True)
        ids = torch.randint(0, V, (B, S + 1), generator=g)
        x, y = ids[:, :-1].contiguous(), ids[:, 1:].contiguous()
        plan = hap_amd.ShardingPlan([RATIOS], 0, ffn="column")
        meta = dict(local_batch=3, global_batch=B, seq_len=S, opt=dict(kind="sgd", lr=1e-3), batch_sharded=True,
                    ratios=RATIOS)
    elif name == "vit":
        L = layers_override or 24
        B = 128
        model = models.VTransformer(1000, 196, 1024, 16, 4096, 0.0, nlayers=L, img_size=(224, 224), patch_size=(16, 16))
        x = torch.randn(B, 3, 224, 224, generator=g)
        y = torch.randint(0, 1000, (B,), generator=g)
        plan = hap_amd.ShardingPlan([RATIOS], 0, ffn="batch")
        meta = dict(local_batch=48, global_batch=B, seq_len=197, opt=dict(kind="adam", lr=5e-4), batch_sharded=True,
                    ratios=RATIOS)
    elif name == "moe":
        L = layers_override or 12
        B, S, V = 16, 512, 33280
        model = models.RMoE(V, S, 768, 12, 3072, 0.0, 16, capacity or MOE_CAPACITY, L, causal=True)
        ids = torch.randint(0, V, (B, S + 1), generator=g)
        x, y = ids[:, :-1].contiguous(), ids[:, 1:].contiguous()
        plan = hap_amd.ShardingPlan([RATIOS_E], 0, ffn="batch")
        meta = dict(local_batch=16, global_batch=B, seq_len=S, opt=dict(kind="adam", lr=5e-4), batch_sharded=False,
                    ratios=RATIOS_E)
    else:
        raise SystemExit(f"unknown workload {name}")
    models.init_normal_(model, 0.02, 39)
    model.dropout_p = float(dropout)
    gm = hap_amd.build_program(model, plan, meta["global_batch"], batch_sharded=meta["batch_sharded"])
    return gm, x, y, meta


def cpu_baseline(name, meta, budget_s=25.0):
    """The CPU oracle (stock PyTorch eager + autograd + torch.optim on the same generated graph, float32 as in
    the reference) timed on this host for a bounded sample.  The same shard is timed at two small depths first (they
    also warm the thread pool up); when their linear extrapolation says that one step of the whole workload fits the
    budget, that whole step is run and timed (its first step: the optimizer's state is allocated inside it), otherwise
    the extrapolated figure is reported."""
    import torch
    from oracle.cpu_executor import PeerlessCPURun
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    torch.set_num_threads(cores)
    full_layers = {"bert": 24, "lm": 2, "vit": 24, "moe": 12}[name]
    sample_layers = [2] if name in ("lm",) else ([2, 4] if name == "moe" else [1, 2])
    o = meta["opt"]

    def timed_steps(layers, warm, most, seconds):
        gm, x, y, _ = build_workload(name, layers_override=layers)
        run = PeerlessCPURun(gm, 0, "fp32")
        opt = (torch.optim.Adam if o["kind"] == "adam" else torch.optim.SGD)(gm.parameters(), lr=o["lr"])
        for _ in range(warm):
            run.step(x, y, [opt])
        t0 = time.perf_counter()
        n = 0
        while n < 1 or (n < most and time.perf_counter() - t0 < seconds):
            run.step(x, y, [opt])
            n += 1
        return (time.perf_counter() - t0) / n

    times = {L: timed_steps(L, 1, 3, budget_s / 8) for L in sample_layers}
    if len(times) == 2:
        a, b = sample_layers
        per_layer = (times[b] - times[a]) / (b - a)
        t_extra = times[a] + per_layer * (full_layers - a)
        small = (f"the same shard at {a} and {b} layers takes {times[a]:.2f}s and {times[b]:.2f}s per step, which "
                 f"extrapolates linearly to {t_extra:.2f}s at {full_layers} layers")
        if t_extra <= budget_s:
            t_full = timed_steps(full_layers, 0, 1, 0.0)
            sample = f"fp32 CPU oracle, the whole workload ({full_layers} layers), one step: {t_full:.2f}s; {small}"
        else:
            t_full = t_extra
            sample = f"fp32 CPU oracle, {small} (one whole step does not fit the {budget_s:.0f}s budget)"
    else:
        t_full = times[sample_layers[0]]
        sample = f"fp32 CPU oracle, full workload, {t_full:.3f}s per step"
    return dict(value=meta["local_batch"] / t_full, unit="samples/s", cores=cores, kind="port", sample=sample)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="bert", choices=list(WORKLOADS) + ["ragged"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="headline workload only: skip the `extra` object (the other configurations, measured briefly)")
    ap.add_argument("--shared-peer-buffers", action="store_true",
                    help="one set of peer message buffers per message shape (all layers read the same 50 MB, which can "
                         "stay in the memory-side cache) instead of one per layer, as real receives are")
    ap.add_argument("--eager", action="store_true",
                    help="launch every kernel of the timed steps from the host instead of replaying a captured HIP graph")
    ap.add_argument("--no-autotune", action="store_true",
                    help="keep the built-in cost model instead of timing tile configurations per GEMM shape first")
    ap.add_argument("--overlap-optimizer", action="store_true",
                    help="update every stretch of the parameters on a second stream as soon as backward is done with it "
                         "instead of one optimizer launch after backward (same step time on the headline shard)")
    ap.add_argument("--no-relu-mask-in-dgrad", action="store_true",
                    help="run the backward of a relu that a linear's epilogue applied as its own pass instead of "
                         "masking the next linear's data gradient in the GEMM epilogue (pure data-parallel FFN, ViT, "
                         "MoE dense layers: the step loses about 1 %)")
    ap.add_argument("--attn", default="batch", choices=["batch", "heads"],
                    help="bert workload only: shard attention over samples (the headline plan) or over heads (6 of 16)")
    ap.add_argument("--dropout", type=float, default=0.0,
                    help="dropout probability of the model (the reference's default is 0.1, config.py:33; the headline "
                         "configuration names none and runs with 0)")
    ap.add_argument("--moe-capacity", type=int, default=MOE_CAPACITY,
                    help="moe workload only: capacity slots per expert (80 = the reference's rule, config.py:25-28; "
                         "40 = capacity factor 1.25 taken as it stands)")
    ap.add_argument("--zero", action="store_true",
                    help="bert workload only: parameters stored as dim-0 shards and gathered at use")
    ap.add_argument("--gemm-table", default=None,
                    help="write a table of the step's distinct GEMM shapes (tile configuration, time of a cold launch) to this file")
    ap.add_argument("--gemm-plan-file", default=None,
                    help="JSON file of pinned GEMM plans: loaded instead of autotuning when it exists, written after "
                         "autotuning otherwise (a profiler run can then repeat the plan of an unprofiled run)")
    ap.add_argument("--no-receive-in-place", action="store_true",
                    help="receive the backward all_to_all's pieces into buffers of their own and concatenate them with a "
                         "copy kernel, instead of receiving them into their rows of the result")
    ap.add_argument("--no-exchange-in-pieces", action="store_true",
                    help="keep the concatenating / splitting copies around the FFN's all_to_all (they then carry relu and its "
                         "backward) instead of letting the second FFN linear read and write the exchanged pieces in place")
    ap.add_argument("--wgrad-group", type=int, default=8,
                    help="the same linear's weight gradients of this many consecutive layers share one launch "
                         "(1: one launch, with its reduction split, per weight gradient)")
    ap.add_argument("--overlap", action="store_true",
                    help="launch the weight-gradient GEMMs on a second stream (per-kernel event times then overlap)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build executes ONE device's shard; no collective crosses the device, "
                         "so only --gpus 1 is measured")
    if args.workload == "ragged":
        from hap_amd import ragged_bench
        print(json.dumps(ragged_bench.run(args.steps, args.warmup, not args.no_cpu_baseline)))
        return

    headline = measure(args.workload, args, args.steps, args.warmup, share_shapes=args.shared_peer_buffers)
    result = headline
    if not args.no_extra and args.workload == "bert" and not args.eager:
        # the other configurations of the benchmark set, each measured the same way (fewer steps), and the headline
        # workload with one set of peer buffers per layer instead of one per message shape
        extra = {}

        def also(key, fn):
            """An additional measurement never takes the headline down with it: its failure is recorded in its place."""
            try:
                extra[key] = fn()
            except Exception as exc:                   # noqa: BLE001 -- reported, not swallowed
                import traceback
                traceback.print_exc()
                extra[key] = {"error": f"{type(exc).__name__}: {exc}"}

        half = max(5, args.steps // 2)
        key = "bert_peer_buffers_per_layer" if args.shared_peer_buffers else "bert_peer_buffers_shared_by_shape"
        also(key, lambda: _brief(measure("bert", args, half, 3, share_shapes=not args.shared_peer_buffers)))
        if args.dropout == 0.0:
            # the headline workload with the reference's default dropout probability (config.py:33): F.dropout in front
            # of the residual LayerNorms and behind the FFN's relu, dropout_p on the attention probabilities
            also("bert_dropout_0.1", lambda: _brief(measure("bert", args, half, 3, share_shapes=args.shared_peer_buffers,
                                                            dropout=0.1)))
        for name in ("lm", "vit", "moe"):
            also(name, lambda name=name: _brief(measure(name, args, half, 3, share_shapes=args.shared_peer_buffers)))
        # the MoE workload with the capacity factor 1.25 taken as it stands (C = 40) instead of the reference's doubled one
        also("moe_C40", lambda: _brief(measure("moe", args, half, 3, share_shapes=args.shared_peer_buffers, capacity=40)))

        def ragged():
            from hap_amd import ragged_bench
            rg = ragged_bench.run(20, 5, False)
            return {"workload": rg["config"]["workload"], "GBps": rg["value"], "ms_per_pass": rg["ms_per_step"],
                    "per_kernel_GBps": rg["config"]["per_kernel_GBps"],
                    "per_kernel_frac_of_hbm_peak": {k: v / HBM_PEAK for k, v in rg["config"]["per_kernel_GBps"].items()},
                    "ragged_reduce_traffic_bytes": rg["roofline"]["traffic"],
                    "ragged_reduce_algorithmic_bytes": rg["roofline"]["algorithmic_bytes"]}
        also("ragged", ragged)
        result["extra"] = extra
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.workload, headline.pop("_meta"))
    result.pop("_meta", None)
    print(json.dumps(result))


def _brief(r):
    return {"workload": r["config"]["workload"], "samples_per_s": r["value"], "ms_per_step": r["ms_per_step"],
            "dtype": r["dtype"], "gemm_TFLOPs": r["roofline"]["achieved"], "gemm_frac_of_peak": r["roofline"]["frac"],
            "gemm_ms_per_step": r["roofline"]["gemm_ms_per_step"], "final_loss": r["config"]["final_loss"]}


def _write_gemm_table(path, report, desc):
    """One row per distinct GEMM signature of the step: the tile configuration that autotuning picked and the time of
    one launch on the program's own operands with cold caches (the median of three launches, each behind a write
    over a buffer larger than the caches)."""
    rows, total_us, total_flop = [], 0.0, 0.0
    for key, cfg, splits, us, launches, problems in report:
        M, N, K, batch, tA, tB, in_dt, out_dt, segA, segB, segC, a_relu, b_relu = key
        flop = 2.0 * M * N * K * batch
        total_us += us * launches
        total_flop += flop * launches
        kind = "".join(c for c, on in (("A", segA), ("B", segB), ("C", segC)) if on)
        rows.append((us * launches, f"{us * launches / 1e3:6.2f} ms/step  x{launches:3d}  M{M:6d} N{N:6d} K{K:6d} batch{batch:4d} "
                     f"{'T' if tA else 'N'}{'T' if tB else 'N'} {'bf16' if in_dt == 1 else 'f32'}->{'bf16' if out_dt == 1 else 'f32'}"
                     f"  cfg{cfg:2d} split{splits:2d}  {us:7.1f} us {flop / us / 1e6:5.0f} TFLOP/s"
                     f"{'  pieces ' + kind if kind else ''}{'  relu on A' if a_relu else ''}{'  relu on B' if b_relu else ''}"))
    with open(path, "w") as f:
        f.write(f"{desc}\n")
        for _, line in sorted(rows, reverse=True):
            f.write(line + "\n")
        f.write(f"sum over the step's launches: {total_us / 1e3:.2f} ms, {total_flop / 1e12:.2f} TFLOP, "
                f"{total_flop / total_us / 1e6:.0f} TFLOP/s (cold single launches)\n")


def measure(workload, args, steps, warmup, share_shapes=True, dropout=None, capacity=None):
    """One workload: compile, autotune the GEMM plans (untimed), warm up, time `steps` steps, bracket the GEMMs.
    ``dropout``: the model's dropout probability (default: the command line's); ``capacity``: slots per expert of the
    MoE workload (default: --moe-capacity)."""
    import ctypes
    import gc

    import torch
    import hap_amd
    from hap_amd import ops, planner
    from hap_amd._lib import lib

    desc, dtype = WORKLOADS[workload]
    bert = workload == "bert"
    if workload == "moe":
        capacity = capacity or args.moe_capacity
        desc = desc.replace(f"C={MOE_CAPACITY}", f"C={capacity}")
    gm, x, y, meta = build_workload(workload, attn=args.attn if bert else "batch", zero=args.zero and bert,
                                    dropout=args.dropout if dropout is None else dropout, capacity=capacity)
    wire = hap_amd.SyntheticWire(seed=39, scale=1.0, grad_scale=1e-3, share_shapes=share_shapes)
    ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=wire, rank=0, world_size=len(meta["ratios"]),
                                 overlap_wgrad=args.overlap, relu_mask_in_dgrad=not args.no_relu_mask_in_dgrad,
                                 overlap_optimizer=args.overlap_optimizer, wgrad_group=args.wgrad_group,
                                 receive_in_place=not args.no_receive_in_place,
                                 exchange_in_pieces=not args.no_exchange_in_pieces)
    ex.configure_optimizer(**meta["opt"])
    ex.load_inputs(x, y)                              # inputs resident in HBM before the timed region
    torch.cuda.synchronize()

    def one_step():
        ex.train_step()

    plan_source = "cost model"
    if args.gemm_plan_file and os.path.exists(args.gemm_plan_file):
        ops.load_gemm_plans(args.gemm_plan_file)      # untimed set-up: the plan of an earlier tuning run
        plan_source = "autotuned (loaded)"
    elif not args.no_autotune:
        report = ex.autotune_gemms()                  # untimed set-up: pins a tile configuration per GEMM shape
        plan_source = "autotuned"
        if args.gemm_plan_file:
            ops.save_gemm_plans(args.gemm_plan_file)
        if args.gemm_table and workload == args.workload:
            _write_gemm_table(args.gemm_table, report, desc)

    graph = None
    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    if not args.eager:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            one_step()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                one_step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()

    lib().hapmi_prof_gemm_enable(0 if graph is not None else 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        if graph is not None:
            graph.replay()
        else:
            one_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    loss = float(ex.loss[0].item())

    ms, n_launch, flops, empty = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double(), ctypes.c_double()
    if graph is None:
        lib().hapmi_prof_gemm_collect(ctypes.byref(ms), ctypes.byref(n_launch), ctypes.byref(flops), ctypes.byref(empty))
        lib().hapmi_prof_gemm_enable(0)
    else:
        # HIP events cannot bracket a kernel inside a replayed graph: the same launches are issued eagerly for
        # three more steps right after the timed region and their per-launch durations are what `roofline` reports
        lib().hapmi_prof_gemm_enable(1)
        for _ in range(3):
            one_step()
        torch.cuda.synchronize()
        lib().hapmi_prof_gemm_collect(ctypes.byref(ms), ctypes.byref(n_launch), ctypes.byref(flops), ctypes.byref(empty))
        lib().hapmi_prof_gemm_enable(0)
    # a bracket holds the kernel(s) of the call plus what its two event records cost; the empty bracket recorded right
    # behind every call measures the latter under the same conditions, and is taken off (the dispatch latency of the
    # kernel itself stays in, so the figure still errs on the long side of the profiler's kernel durations)
    gemm_ms = ms.value - empty.value
    achieved = flops.value / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0
    peak = PEAK[dtype]
    ms_per_step = dt / steps * 1e3
    result = {
        "metric": "samples/sec of one GPU's uneven shard (fwd+bwd+step)",
        "value": meta["local_batch"] * steps / dt,
        "unit": "samples/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": desc, "local_batch": meta["local_batch"], "global_batch": meta["global_batch"],
                   "seq_len": meta["seq_len"], "launch": "hip-graph" if graph is not None else "eager",
                   "wgrad_stream": "side" if args.overlap else "main",
                   "optimizer": "one launch after backward" if ex._opt_chunks is None else "per stretch, overlapped with backward",
                   "gemm_plan": plan_source, "weight_gradient_group": ex.wgrad_group,
                   "exchange_pieces_received_in_place": ex.receive_in_place,
                   "exchange_read_and_written_in_pieces": ex.exchange_in_pieces,
                   "peer_buffers": "one set per message shape" if share_shapes else "one set per layer",
                   "attention_sharding": args.attn if bert else "batch",
                   "zero_sharded_parameters": bool(args.zero and bert), "dropout": args.dropout if dropout is None else dropout,
                   "final_loss": loss},
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel (all GEMM launches of the step)",
                     "achieved": achieved, "peak": peak, "unit": "TFLOP/s", "frac": achieved / peak,
                     "measured_over": "the timed steps" if graph is None else "3 eager steps after the timed graph replays",
                     "launches_per_step": n_launch.value / max(1, steps if graph is None else 3),
                     "gemm_ms_per_step": gemm_ms / max(1, steps if graph is None else 3),
                     "event_brackets_ms_per_step": ms.value / max(1, steps if graph is None else 3),
                     "empty_brackets_ms_per_step": empty.value / max(1, steps if graph is None else 3), "traffic": None},
    }
    default_bert = (bert and args.attn == "batch" and not args.zero and (args.dropout if dropout is None else dropout) == 0.0
                    and not args.no_exchange_in_pieces and not args.no_receive_in_place and args.wgrad_group == 8)
    if default_bert:
        # bytes per GEMM launch between the L2 caches and the memory fabric, counted OFFLINE with rocprofv3 --pmc
        # (FETCH_SIZE scaled by the factor a copy of known size gives, plus WRITE_SIZE; mean over the step's launches):
        # a property of the tile plan that was profiled, so it is reported only for a run that uses that plan
        r = result["roofline"]
        plan_now = ops.pinned_gemm_plans()
        same_plan = all(plan_now.get(k) == v for k, v in PROFILED_GEMM_PLAN.items())
        same_launches = round(r["launches_per_step"]) == PROFILED_GEMM_LAUNCHES_PER_STEP
        r["traffic"] = PROFILED_GEMM_TRAFFIC_PER_LAUNCH if same_plan and same_launches else None
        r["traffic_source"] = ("offline profile, not measured in this run: rocprofv3 --pmc FETCH_SIZE x 2.0 + WRITE_SIZE per "
                               "launch, mean over the step's GEMM launches (profiles/bert_large_shard_step.counters.md); "
                               "reported only when this run's GEMM plan and launch count are the profiled ones")
        r["traffic_plan_is_the_profiled_one"] = bool(same_plan and same_launches)
        r["traffic_unit"] = "bytes per launch"
        r["algorithmic_bytes"] = PROFILED_GEMM_ALGORITHMIC_BYTES_PER_LAUNCH if same_launches else None
    # the reference calibrates its planner with hap.stat / (seconds of one training step) (profiler.py:33-39)
    shard_stat = planner.stat(gm, {"input_shape": {"x": tuple(x.shape), "y": tuple(y.shape)}})
    result["config"]["hap_stat_flops_of_shard"] = shard_stat
    result["config"]["device_flops"] = math.floor(shard_stat / (ms_per_step * 1e-3))
    result["_meta"] = meta
    del graph, ex, wire, gm
    gc.collect()
    torch.cuda.empty_cache()
    return result


if __name__ == "__main__":
    main()
