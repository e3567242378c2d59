"""Stock-PyTorch CPU execution of the generated shard programs.
TEST INFRASTRUCTURE ONLY -- this is the checker, never the product path.

The reference runs its emitted graph with PyTorch eager + autograd
(/root/reference/worker.py:44-76): ``GraphModule(x, y)``, ``loss.backward()``,
``optimizer.step()``.  This module does the same on the CPU for all W ranks of
the SPMD program at once: the W graphs are walked in lock step, ordinary nodes
call their stock PyTorch target per rank, and ``collectives.*`` nodes are
replaced by the in-memory world of oracle/ops.py, which follows
/root/reference/collectives.py and records every message that crosses ranks.

bf16 mode (the reference is fp32 only, so these rules are this build's own
definition): parameters are cast to bfloat16 at their ``get_attr`` (gradients
return to the float32 masters), activations are bfloat16, log-softmax + NLL
and the gating run in float32, and the routing einsums contract in float32
before rounding the result to bfloat16.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.fx
import torch.nn.functional as F

import hap_amd.collectives as product_collectives
import hap_amd.models as product_models

from . import ops as ref


class JointCPURun:
    def __init__(self, programs: List[torch.fx.GraphModule], dtype: str = "fp32"):
        assert dtype in ("fp32", "bf16")
        self.programs = programs
        self.W = len(programs)
        self.dtype = dtype
        self.world = ref.JointWorld(self.W)
        self.env: List[Dict[str, object]] = [dict() for _ in range(self.W)]

    # ------------------------------------------------------------------
    def _lookup(self, r, a):
        return torch.fx.node.map_arg(a, lambda n: self.env[r][n.name])

    def _get_attr(self, r, target):
        obj = self.programs[r]
        for atom in target.split("."):
            obj = getattr(obj, atom)
        if self.dtype == "bf16" and obj.is_floating_point():
            obj = obj.to(torch.bfloat16)
        return obj

    def _call_local(self, r, node):
        args = self._lookup(r, node.args)
        kwargs = self._lookup(r, node.kwargs)
        t = node.target
        if t in (product_models.top_2_gating, product_models.switch_gating):
            x, n_expert, capacity, wg = args[:4]
            gating = ref.top_2_gating if t is product_models.top_2_gating else ref.switch_gating
            # float32 whatever the activations' type; a float64 run (a model cast with .double(), used to
            # calibrate tolerances) gates in float64 and needs the dispatch mask in float64 for the einsums
            hi = torch.float64 if x.dtype == torch.float64 else torch.float32
            dispatch, combine = gating(x.to(hi), n_expert, capacity, wg.to(hi))
            return dispatch.to(hi), combine
        if t is product_models.head_parallel_attention:
            return ref.head_parallel_attention(*args, **kwargs)
        if t is product_models.append_cls_token:
            x, cls = args
            return torch.cat((cls.expand(x.shape[0], -1, -1), x), dim=1)
        if t is product_models.get_cls_token:
            return args[0][:, 0, :]
        if t is product_models.new_segment:
            return args[0]
        if t is product_collectives.dynamic_slice:
            return self.world.dynamic_slice(*args)
        if self.dtype == "bf16":
            if t is F.conv2d:                           # images arrive as float32; the patch GEMM runs in bf16
                return F.conv2d(args[0].to(torch.bfloat16), *args[1:], **kwargs)
            if t is torch.log_softmax:
                return torch.log_softmax(args[0].float(), *args[1:], **kwargs)
            if t is torch.einsum and any(a.dtype == torch.float32 for a in args[1:]):
                out = torch.einsum(args[0], *[a.float() for a in args[1:]])
                return out.to(torch.bfloat16)
        return t(*args, **kwargs)

    def forward(self, x, y) -> List[torch.Tensor]:
        W = self.W
        node_lists = [list(p.graph.nodes) for p in self.programs]
        n_inputs = 0
        result = None
        for step in zip(*node_lists):
            node0 = step[0]
            name = node0.name
            if node0.op == "placeholder":
                val = (x, y)[n_inputs]
                n_inputs += 1
                for r in range(W):
                    self.env[r][step[r].name] = val
            elif node0.op == "get_attr":
                for r in range(W):
                    self.env[r][step[r].name] = self._get_attr(r, step[r].target)
            elif node0.op == "call_method":
                for r in range(W):
                    a = self._lookup(r, step[r].args)
                    self.env[r][step[r].name] = getattr(a[0], step[r].target)(*a[1:])
            elif node0.op == "call_function":
                t = node0.target
                if t in (product_collectives.all_gather, product_collectives.reduce_scatter):
                    xs = [self._lookup(r, step[r].args[0]) for r in range(W)]
                    _, dim, L, _rank = node0.args
                    fn = self.world.all_gather if t is product_collectives.all_gather else self.world.reduce_scatter
                    outs = fn(name, xs, dim, list(L))
                elif t is product_collectives.all_to_all:
                    xs = [self._lookup(r, step[r].args[0]) for r in range(W)]
                    _, sd, cd, sL, cL, _rank = node0.args
                    outs = self.world.all_to_all(name, xs, sd, cd, list(sL), list(cL))
                elif t is product_collectives.all_reduce:
                    outs = self.world.all_reduce(name, [self._lookup(r, step[r].args[0]) for r in range(W)])
                elif t is product_collectives.replicate:
                    outs = self.world.replicate(name, [self._lookup(r, step[r].args[0]) for r in range(W)])
                else:
                    outs = [self._call_local(r, step[r]) for r in range(W)]
                for r in range(W):
                    self.env[r][step[r].name] = outs[r]
            elif node0.op == "output":
                result = [self._lookup(r, step[r].args[0]) for r in range(W)]
            else:
                raise ValueError(node0.op)
        return result

    def step(self, x, y, optimizers: Optional[list] = None, clip_grad_norm: Optional[float] = None) -> List[torch.Tensor]:
        """zero_grad -> forward -> backward of the summed loss -> [clip_grad_norm_ over each rank's own
        gradients, worker.py:74] -> optimizer step (worker.py:59-76)."""
        for p in self.programs:
            p.zero_grad(set_to_none=True)
        losses = self.forward(x, y)
        total = losses[0].float()
        for l in losses[1:]:
            total = total + l.float()
        total.backward()
        if clip_grad_norm is not None:
            for p in self.programs:
                torch.nn.utils.clip_grad_norm_(p.parameters(), clip_grad_norm)
        if optimizers is not None:
            for opt in optimizers:
                opt.step()
        return [l.detach() for l in losses]


def _rank_ordered_sum(own: torch.Tensor, rank: int, peers: Dict[int, Optional[torch.Tensor]], W: int) -> torch.Tensor:
    """Sum over ranks in rank order with float32 accumulation (collectives.py:27, :77, :95); a peer that
    contributes nothing (None) is left out."""
    parts = [own if s == rank else peers.get(s) for s in range(W)]
    parts = [p for p in parts if p is not None]
    acc = parts[0].float().clone()
    for p in parts[1:]:
        acc = acc + p.float()
    return acc.to(own.dtype)


class SingleRankCPURun(JointCPURun):
    """ONE rank of the SPMD program on the CPU; what the other ranks would send comes from a wire object with
    the interface of hap_amd.wire.Wire (``recv(tag, direction, src, shape, dtype, device, reduction)``), asked
    for exactly the messages, shapes and directions that the product's executor asks its wire for:

    * all_gather (collectives.py:14-29): forward receives every peer's shard padded to the longest length and
      keeps its first L[src] entries; backward splits the gradient, keeps this rank's piece and adds the peers'
      padded pieces (first L[rank] entries) in rank order;
    * reduce_scatter (collectives.py:88-103): the two directions swapped;
    * all_to_all (collectives.py:152-166): receives from rank src a piece of this rank's split length along the
      split dimension and cat_L[src] along the concatenation dimension; backward with the roles swapped;
    * all_reduce (collectives.py:73-84) and the gradient of replicate (collectives.py:176-180): rank-ordered sum
      with the peers' tensors of the same shape.

    With a ReplayWire over the log of a JointCPURun it reproduces that rank of the joint run (this is what
    pins it: tests/test_oracle_single_rank.py); with a SyntheticWire the peers' messages are the same seeded
    tensors the GPU run receives; with a SilentWire the peers send zeros / nothing.

    ``wire_dtype``: element type the messages are made in before they are cast to this run's own type
    (a float32 CPU run that checks a bf16 GPU run receives the same bf16-rounded messages)."""

    def __init__(self, program: torch.fx.GraphModule, rank: int, world_size: int, wire, dtype: str = "fp32",
                 wire_dtype: Optional[torch.dtype] = None, decisions: Optional[Dict[str, torch.Tensor]] = None):
        """``decisions``: discrete decisions taken from another run of the same program, by node name -- for an
        ``F.relu`` node the boolean mask of the elements it lets through, for a ``top_2_gating`` node the expert
        choices [B, S, 2], for an ``F.dropout`` node the boolean keep mask of its input's shape, for an
        ``F.multi_head_attention_forward`` node with dropout_p > 0 the keep mask [N, H, L, S] of its probabilities.
        The node then applies those instead of its own (relu(z) becomes z * mask, the gates stay this run's
        probabilities of the given experts, dropout becomes x * keep / (1 - p): the GPU's random stream cannot be
        shared with torch's generator, its masks can).  A step function turns a rounding-sized difference of
        its argument into a whole-sized difference of the result; with the decisions shared, what is left between
        two runs is their continuous arithmetic, which tolerances can bound.  Whether the other run's decisions
        differ from this run's own only where the argument is within rounding distance of the step is for the
        caller to check."""
        super().__init__([program], dtype)
        self.rank, self.world_size, self.wire = rank, world_size, wire
        self.wire_dtype = wire_dtype
        self.decisions = decisions or {}

    def _call_local(self, r, node):
        forced = self.decisions.get(node.name)
        if forced is not None:
            args = self._lookup(r, node.args)
            if node.target is F.relu:
                return args[0] * forced.to(args[0].dtype)
            if node.target is F.dropout:
                x, p = args[0], float(args[1])
                scale = 1.0 / (1.0 - p) if p < 1.0 else 0.0
                return (x.to(torch.float64 if x.dtype == torch.float64 else torch.float32)
                        * (forced.to(torch.float32) * scale)).to(x.dtype)
            if node.target is F.multi_head_attention_forward:
                kw = self._lookup(r, node.kwargs)
                out = ref.attention_with_dropped_probabilities(
                    kw["query"], kw["in_proj_weight"], kw["in_proj_bias"], kw["out_proj_weight"], kw["out_proj_bias"],
                    kw["num_heads"], kw.get("attn_mask"), forced, float(kw["dropout_p"]))
                return out, None
            if node.target is product_models.top_2_gating:
                x, n_expert, capacity, wg = args[:4]
                hi = torch.float64 if x.dtype == torch.float64 else torch.float32
                dispatch, combine = ref.top_2_gating(x.to(hi), n_expert, capacity, wg.to(hi), index=forced.long())
                return dispatch.to(hi), combine
            raise ValueError(f"no shared decision is defined for {node.target}")
        return super()._call_local(r, node)

    # -- wire access -----------------------------------------------------
    def _recv(self, tag, direction, src, shape, like: torch.Tensor, reduction: bool, dtype=None):
        dt = dtype or self.wire_dtype or like.dtype
        t = self.wire.recv(tag, direction, src, tuple(shape), dt, torch.device("cpu"), reduction=reduction)
        return None if t is None else t.to(like.dtype)

    def _peers(self, tag, direction, shape, like, reduction, dtype=None):
        return {s: self._recv(tag, direction, s, shape, like, reduction, dtype)
                for s in range(self.world_size) if s != self.rank}

    # -- the two directions of all_gather / reduce_scatter ---------------
    def _gather(self, tag, direction, x, dim, L, dtype=None):
        m = max(L)
        pshape = list(x.shape)
        pshape[dim] = m
        peers = self._peers(tag, direction, pshape, x, False, dtype)
        return torch.cat([x if s == self.rank else peers[s].narrow(dim, 0, L[s]) for s in range(len(L))], dim=dim)

    def _scatter(self, tag, direction, full, dim, L, dtype=None):
        m = max(L)
        own = torch.split(full.contiguous(), list(L), dim=dim)[self.rank]
        pshape = list(full.shape)
        pshape[dim] = m
        peers = self._peers(tag, direction, pshape, full, True, dtype)
        peers = {s: (p.narrow(dim, 0, L[self.rank]) if p is not None else None) for s, p in peers.items()}
        return _rank_ordered_sum(own, self.rank, peers, len(L))

    def _exchange(self, tag, direction, x, split_dim, cat_dim, split_L, cat_L):
        own = torch.split(x.contiguous(), list(split_L), dim=split_dim)[self.rank]
        parts = []
        for s in range(len(split_L)):
            if s == self.rank:
                parts.append(own)
            else:
                shape = list(own.shape)
                shape[cat_dim] = cat_L[s]
                parts.append(self._recv(tag, direction, s, shape, x, False))
        return torch.cat(parts, dim=cat_dim)

    def _sum(self, tag, direction, x, dtype=None):
        return _rank_ordered_sum(x, self.rank, self._peers(tag, direction, x.shape, x, True, dtype), self.world_size)

    # -- collectives as autograd nodes over this rank's tensor -----------
    def _collective(self, node, args):
        run, t, tag = self, node.target, node.name
        # a gathered parameter (ZeRO form) is not an activation: its shard travels in the type it is stored in and
        # its gradient comes back in float32, whatever type the activations' messages are made in
        of_param = node.args[0].op == "get_attr"

        if t in (product_collectives.all_gather, product_collectives.reduce_scatter):
            xin, dim, L, rank = args
            assert rank == self.rank
            gather_fwd = t is product_collectives.all_gather
            fwd_dtype = xin.dtype if of_param else None
            bwd_dtype = torch.float32 if (of_param and self.wire_dtype is not None) else fwd_dtype

            class Fn(torch.autograd.Function):
                @staticmethod
                def forward(ctx, x):
                    if gather_fwd:
                        return run._gather(tag, "fwd", x, dim, list(L), fwd_dtype)
                    return run._scatter(tag, "fwd", x, dim, list(L))

                @staticmethod
                def backward(ctx, g):
                    if gather_fwd:
                        return run._scatter(tag, "bwd", g, dim, list(L), bwd_dtype)
                    return run._gather(tag, "bwd", g.contiguous(), dim, list(L))
            return Fn.apply(xin)

        if t is product_collectives.all_to_all:
            xin, sd, cd, sL, cL, rank = args
            assert rank == self.rank

            class Fn(torch.autograd.Function):
                @staticmethod
                def forward(ctx, x):
                    return run._exchange(tag, "fwd", x, sd, cd, sL, cL)

                @staticmethod
                def backward(ctx, g):
                    return run._exchange(tag, "bwd", g, cd, sd, cL, sL)
            return Fn.apply(xin)

        if t is product_collectives.all_reduce:
            class Fn(torch.autograd.Function):
                @staticmethod
                def forward(ctx, x):
                    return run._sum(tag, "fwd", x.contiguous())

                @staticmethod
                def backward(ctx, g):
                    return run._sum(tag, "bwd", g.contiguous())
            return Fn.apply(args[0])

        if t is product_collectives.replicate:
            class Fn(torch.autograd.Function):
                @staticmethod
                def forward(ctx, x):
                    return x.view_as(x)

                @staticmethod
                def backward(ctx, g):
                    return run._sum(tag, "bwd", g.contiguous(), torch.float32)
            return Fn.apply(args[0])
        raise ValueError(t)

    def forward(self, x, y):
        env = self.env[0]
        prog = self.programs[0]
        look = lambda a: torch.fx.node.map_arg(a, lambda n: env[n.name])
        wire_ops = (product_collectives.all_gather, product_collectives.reduce_scatter, product_collectives.all_to_all,
                    product_collectives.all_reduce, product_collectives.replicate)
        n_inputs = 0
        for node in prog.graph.nodes:
            if node.op == "placeholder":
                env[node.name] = (x, y)[n_inputs]
                n_inputs += 1
            elif node.op == "get_attr":
                env[node.name] = self._get_attr(0, node.target)
            elif node.op == "call_method":
                a = look(node.args)
                env[node.name] = getattr(a[0], node.target)(*a[1:])
            elif node.op == "output":
                return [look(node.args[0])]
            elif node.target in wire_ops:
                env[node.name] = self._collective(node, look(node.args))
            else:
                env[node.name] = self._call_local(0, node)
        raise RuntimeError("program has no output node")


class PeerlessCPURun(SingleRankCPURun):
    """One rank only, peers silent: every collective keeps its local half and receives zeros (all_gather /
    all_to_all) or nothing (reductions) from the other ranks.  Used to time the CPU baseline of a single
    shard at full size without executing the peers' share of the work."""

    def __init__(self, program: torch.fx.GraphModule, rank: int, dtype: str = "fp32", world_size: Optional[int] = None):
        from hap_amd.wire import SilentWire
        if world_size is None:
            world_size = 1
            for node in program.graph.nodes:
                if node.op == "call_function" and node.target in (product_collectives.all_gather,
                                                                  product_collectives.reduce_scatter):
                    world_size = max(world_size, len(node.args[2]))
                elif node.op == "call_function" and node.target is product_collectives.all_to_all:
                    world_size = max(world_size, len(node.args[3]))
        super().__init__(program, rank, world_size, SilentWire(), dtype)
