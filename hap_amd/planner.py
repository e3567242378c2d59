"""Shape rules, FLOP count and plan selection for the generated programs.

The reference's synthesizer prices a program with three ingredients, all of
which live in its Rust extension:

* a per-op FLOP formula attached to every parsed node (``Op.flops``,
  /root/reference/hap.rs:1038-1044 linear, 1330-1337 attention, 2277-2291
  einsum, and one closure per handler in hap.rs:995-2300);
* ``hap.stat(graph_module, {"input_shape": ...})`` = 3 x the sum of those
  formulas over the single-device graph (hap.rs:190-209: one forward plus two
  for the backward);
* a cost per device of ``flops / device_flops[i]`` plus the collectives'
  element counts over their measured bandwidths, maximised over the devices
  (hap.rs:365-395; the element counts are hap.rs:2549-2551, 2572-2574,
  2648-2650, 2688-2689, 2707-2708, 2737-2738).

``device_flops`` is calibrated by timing one training step and dividing
``hap.stat`` by it (/root/reference/profiler.py:17-39).

This module restates the three on the programs ``hap_amd.program`` emits:
``infer_shapes`` / ``flops`` / ``stat`` work on any rank's program (local
shapes; for a one-device plan that is the reference's single-device count),
``calibrate_device_flops`` is the timing half, and ``choose_plan`` ranks the
legal plan forms of the fixed model families by the cost above.  The search,
the Hoare-triple derivation and the LP of the reference are not rebuilt: the
forms are the fixed ones of ``hap_amd.program`` and the ratios are
proportional to the devices' flops (the LP's optimum when computation
dominates) or uniform.
"""
from __future__ import annotations

import math
import operator
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Sequence, Tuple

import torch
import torch.fx
import torch.nn.functional as F

from . import collectives, models
from .sharding import ShardingPlan

Shape = Tuple[int, ...]


def _prod(shape) -> int:
    return int(math.prod(int(v) for v in shape))


def _with(shape, dim, n) -> Shape:
    dim = dim % len(shape)
    return tuple(shape[:dim]) + (int(n),) + tuple(shape[dim + 1:])


def _attr(gm, target: str):
    obj = gm
    for atom in target.split("."):
        obj = getattr(obj, atom)
    return obj


def _broadcast(a: Shape, b: Shape) -> Shape:
    n = max(len(a), len(b))
    a = (1,) * (n - len(a)) + tuple(a)
    b = (1,) * (n - len(b)) + tuple(b)
    out = []
    for x, y in zip(a, b):
        if x != y and 1 not in (x, y):
            raise ValueError(f"shapes {a} and {b} do not broadcast")
        out.append(max(x, y))
    return tuple(out)


_EINSUM_OUT = {
    # code -> output shape from (x, y)                                   hap.rs:2240-2262
    "bsd,bsec->becd": lambda x, y: (x[0], y[2], y[3], x[2]),
    "edh,becd->bech": lambda x, y: (y[0], y[1], y[2], x[2]),
    "ehd,bech->becd": lambda x, y: (y[0], y[1], y[2], x[2]),
    "becd,bsec->bsd": lambda x, y: (x[0], y[1], x[3]),
}

_EINSUM_FLOPS = {
    # hap.rs:2283-2286
    "bsd,bsec->becd": lambda x, y: 3 * x[0] * x[1] * x[2] * y[2] * y[3],
    "edh,becd->bech": lambda x, y: 3 * x[0] * x[1] * x[2] * y[0] * y[2],
    "ehd,bech->becd": lambda x, y: 3 * x[0] * x[1] * x[2] * y[0] * y[2],
    "becd,bsec->bsd": lambda x, y: 3 * x[0] * x[1] * x[2] * x[3] * y[1],
}


def infer_shapes(gm: torch.fx.GraphModule, input_shape: Dict[str, Sequence[int]]) -> Dict[str, object]:
    """Shape of every node of a program, from the placeholder shapes (the
    global, unsharded ones, as ``config.input_shape()`` gives them to the
    reference, hap.rs:191-194) and the attributes' actual (already sliced)
    shapes.  Tuple-valued nodes map to a list of shapes."""
    env: Dict[str, object] = {}

    def sh(a):
        return env[a.name] if isinstance(a, torch.fx.Node) else None

    for node in gm.graph.nodes:
        if node.op == "placeholder":
            env[node.name] = tuple(int(v) for v in input_shape[node.name])
        elif node.op == "get_attr":
            env[node.name] = tuple(_attr(gm, node.target).shape)
        elif node.op == "call_method":
            if node.target != "split":
                raise ValueError(f"method {node.target!r} has no shape rule")
            x, lengths, dim = node.args
            env[node.name] = [_with(sh(x), dim, n) for n in lengths]
        elif node.op == "output":
            env[node.name] = sh(node.args[0])
        elif node.op == "call_function":
            env[node.name] = _call_shape(node, sh)
        else:
            raise ValueError(node.op)
    return env


def _call_shape(node, sh):
    t, a, kw = node.target, node.args, node.kwargs
    if t is operator.getitem:
        return sh(a[0])[a[1]]
    if t in (collectives.replicate, collectives.all_reduce, models.new_segment,
             F.relu, F.gelu, F.dropout, F.layer_norm, torch.sigmoid):
        return sh(a[0])
    if t is collectives.all_gather:
        x, dim, L, _rank = a
        return _with(sh(x), dim, sum(L))
    if t in (collectives.reduce_scatter, collectives.dynamic_slice):
        x, dim, L, rank = a
        return _with(sh(x), dim, L[rank])
    if t is collectives.all_to_all:
        x, split_dim, cat_dim, split_L, cat_L, rank = a
        return _with(_with(sh(x), split_dim, split_L[rank]), cat_dim, sum(cat_L))
    if t is F.linear:
        return tuple(sh(a[0])[:-1]) + (sh(a[1])[0],)
    if t is F.embedding:
        return tuple(sh(a[0])) + (sh(a[1])[1],)
    if t is operator.mul:
        return sh(a[0]) if not isinstance(a[1], torch.fx.Node) else _broadcast(sh(a[0]), sh(a[1]))
    if t is operator.add:
        return _broadcast(sh(a[0]), sh(a[1]))
    if t is torch.transpose:
        s = list(sh(a[0]))
        s[a[1]], s[a[2]] = s[a[2]], s[a[1]]
        return tuple(s)
    if t is F.multi_head_attention_forward:
        L, N, E = sh(kw["query"])
        S = sh(kw["key"])[0]
        return [(L, N, E), (N, L, S)]
    if t is models.head_parallel_attention:
        return tuple(sh(a[0])[:2]) + (sh(a[3])[0],)
    if t is F.conv2d:
        n, _c, h, w = sh(a[0])
        o, _ci, kh, kw_ = sh(a[1])
        stride, padding = a[3], a[4]
        return (n, o, (h + 2 * padding[0] - kh) // stride[0] + 1, (w + 2 * padding[1] - kw_) // stride[1] + 1)
    if t is torch.flatten:
        s = sh(a[0])
        start, end = a[1] % len(s), a[2] % len(s)
        return tuple(s[:start]) + (_prod(s[start:end + 1]),) + tuple(s[end + 1:])
    if t is torch.log_softmax:
        return sh(a[0])
    if t in (F.nll_loss, torch.sum):
        return ()
    if t is models.append_cls_token:
        b, s, d = sh(a[0])
        return (b, s + 1, d)
    if t is models.get_cls_token:
        b, _s, d = sh(a[0])
        return (b, d)
    if t in (models.top_2_gating, models.switch_gating):
        b, s, _d = sh(a[0])
        return [(b, s, a[1], a[2]), (b, s, a[1], a[2])]
    if t is torch.einsum:
        return tuple(_EINSUM_OUT[a[0]](sh(a[1]), sh(a[2])))
    raise ValueError(f"{t} has no shape rule")


def _node_flops(node, sh) -> int:
    """The reference's ``Op.flops`` closure of the node's handler, on the
    node's input shapes.  Collectives, ``getitem``, ``new_segment`` and
    attribute reads are not ``Op`` nodes there and count nothing."""
    t, a, kw = node.target, node.args, node.kwargs
    if t is F.linear:                                            # hap.rs:1038-1044
        return 3 * _prod(sh(a[0])) * sh(a[1])[0]
    if t in (torch.sigmoid, F.relu, F.dropout):                  # hap.rs:1090, 1420, 1467
        return 3 * _prod(sh(a[0]))
    if t is F.gelu:                                              # no handler in the reference: priced like relu
        return 3 * _prod(sh(a[0]))
    if t in (torch.transpose, operator.add, operator.mul, torch.flatten, F.nll_loss, torch.sum):
        return _prod(sh(a[0]))                                   # hap.rs:1216, 1518, 1566/1609, 1782, 1884, 1136
    if t is F.multi_head_attention_forward:                      # hap.rs:1330-1337
        L, N, E = sh(kw["query"])
        S = sh(kw["key"])[0]
        return 3 * L * N * E * S + 5 * L * S * N + 3 * L * N * E * S
    if t is models.head_parallel_attention:                      # hap.rs:1330-1337 with E = the local heads' width
        N, L, _d = sh(a[0])
        Ea = sh(a[1])[0] // 3
        return 3 * L * N * Ea * L + 5 * L * L * N + 3 * L * N * Ea * L
    if t is F.layer_norm:                                        # hap.rs:1656
        return 10 * _prod(sh(a[0]))
    if t is F.conv2d:                                            # hap.rs:1727
        return 3 * sh(a[1])[0] * _prod(sh(a[0]))
    if t is torch.log_softmax:                                   # hap.rs:1832
        return 15 * _prod(sh(a[0]))
    if t is F.embedding:                                         # hap.rs:2044
        return _prod(sh(a[0]))
    if t in (models.append_cls_token, models.get_cls_token):     # hap.rs:2096, 2144
        s = sh(a[0])
        return s[0] * s[2]
    if t in (models.top_2_gating, models.switch_gating):         # hap.rs:2206 (switch: no handler there, same price)
        return 10 * _prod(sh(a[0]))
    if t is torch.einsum:                                        # hap.rs:2283-2286
        return _EINSUM_FLOPS[a[0]](sh(a[1]), sh(a[2]))
    return 0


def flops(gm: torch.fx.GraphModule, input_shape: Dict[str, Sequence[int]]) -> int:
    """Forward FLOPs of the program by the reference's per-op formulas."""
    env = infer_shapes(gm, input_shape)

    def sh(a):
        return env[a.name]

    return sum(_node_flops(n, sh) for n in gm.graph.nodes if n.op == "call_function")


def stat(gm: torch.fx.GraphModule, config: Dict[str, Dict[str, Sequence[int]]]) -> float:
    """``hap.stat`` (hap.rs:190-209): ``config["input_shape"]`` names the
    placeholder shapes; the result is 3 x the forward FLOPs, as a float."""
    return float(flops(gm, config["input_shape"])) * 3.0


def calibrate_device_flops(step: Callable[[], object], total_flops: float, synchronize: Callable[[], None],
                           warmup: int = 11) -> int:
    """FlopsProfiler (profiler.py:17-39): ``warmup`` untimed training steps, one
    timed step bracketed by device synchronisation, ``floor(flops / seconds)``."""
    for _ in range(warmup):
        step()
    synchronize()
    t0 = time.time()
    step()
    synchronize()
    duration = time.time() - t0
    return math.floor(total_flops / duration)


# ---------------------------------------------------------------------------------------------------------
# Cost of a plan

@dataclass
class ClusterInfo:
    """The measured quantities the reference's cost divides by (hap.rs:373-379);
    bandwidths in elements per second as BandwidthProfiler reports them
    (profiler.py:41-60)."""
    device_flops: List[float]
    all_gather_bandwidth: float
    all_reduce_bandwidth: float
    reduce_scatter_bandwidth: float
    all_to_all_bandwidth: float

    @property
    def n_devices(self) -> int:
        return len(self.device_flops)


@dataclass
class Traffic:
    """Element counts per collective kind, forward plus backward (hap.rs:452-471)."""
    all_gather: int = 0
    all_reduce: int = 0
    reduce_scatter: int = 0
    all_to_all: int = 0


def communication(gm: torch.fx.GraphModule, input_shape: Dict[str, Sequence[int]], n_devices: int) -> Traffic:
    """What the reference's profile closures add up for one device's program:
    gathers, scatters and exchanges count the local shard x n_devices in both
    directions with the mirrored kind; an all_reduce counts the full tensor
    twice; a replicated parameter counts one all_reduce of its gradient."""
    env = infer_shapes(gm, input_shape)
    tr = Traffic()
    for node in gm.graph.nodes:
        if node.op != "call_function":
            continue
        t = node.target
        if t is collectives.all_gather:                          # hap.rs:2648-2650
            n = _prod(env[node.args[0].name]) * n_devices
            tr.all_gather += n
            tr.reduce_scatter += n
        elif t is collectives.reduce_scatter:                    # hap.rs:2688-2689
            n = _prod(env[node.name]) * n_devices
            tr.reduce_scatter += n
            tr.all_gather += n
        elif t is collectives.all_to_all:                        # hap.rs:2737-2738
            n = _prod(env[node.args[0].name]) * n_devices
            tr.all_to_all += 2 * n
        elif t is collectives.all_reduce:                        # hap.rs:2707-2708
            tr.all_reduce += 2 * _prod(env[node.name])
        elif t is collectives.replicate:                         # hap.rs:2572-2574
            tr.all_reduce += _prod(env[node.name])
    return tr


def device_cost(gm, input_shape, cluster: ClusterInfo, device: int) -> Tuple[float, float]:
    """(computation seconds, communication seconds) of one device (hap.rs:365-383)."""
    comp = stat(gm, {"input_shape": input_shape}) / cluster.device_flops[device]
    tr = communication(gm, input_shape, cluster.n_devices)
    comm = (tr.all_gather / cluster.all_gather_bandwidth + tr.all_reduce / cluster.all_reduce_bandwidth
            + tr.reduce_scatter / cluster.reduce_scatter_bandwidth + tr.all_to_all / cluster.all_to_all_bandwidth)
    return comp, comm


@dataclass
class PlanCost:
    ffn: str
    ratios: List[float]
    computation: float
    communication: float
    per_device: List[Tuple[float, float]] = field(default_factory=list)

    @property
    def total(self) -> float:
        return self.computation + self.communication


def plan_cost(model_factory: Callable[[], torch.nn.Module], global_batch: int, input_shape, cluster: ClusterInfo,
              ffn: str, ratios: Sequence[float], activation: str = "relu") -> PlanCost:
    """max over devices of the computation time + max over devices of the
    communication time (hap.rs:385-394).  ``model_factory`` builds a fresh
    model (on the ``meta`` device is enough: only shapes are read)."""
    from .program import build_program
    per = []
    for r in range(cluster.n_devices):
        plan = ShardingPlan([list(ratios)], r, ffn=ffn)
        gm = build_program(model_factory(), plan, global_batch, activation=activation)
        per.append(device_cost(gm, input_shape, cluster, r))
    return PlanCost(ffn, list(ratios), max(c for c, _ in per), max(m for _, m in per), per)


def choose_plan(model_factory, global_batch: int, input_shape, cluster: ClusterInfo,
                forms: Sequence[str] = ("batch", "column"), activation: str = "relu") -> List[PlanCost]:
    """Candidates = plan forms x {ratios proportional to device_flops, uniform},
    cheapest first."""
    n = cluster.n_devices
    total = float(sum(cluster.device_flops))
    candidates = [[f / total for f in cluster.device_flops]]
    if any(abs(c - 1.0 / n) > 1e-12 for c in candidates[0]):
        candidates.append([1.0 / n] * n)
    out = [plan_cost(model_factory, global_batch, input_shape, cluster, ffn, ratios, activation)
           for ffn in forms for ratios in candidates]
    return sorted(out, key=lambda c: c.total)
