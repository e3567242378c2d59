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

import operator
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
            dispatch, combine = gating(x.float(), n_expert, capacity, wg.float())
            return dispatch, combine
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


class PeerlessCPURun(JointCPURun):
    """One rank only, peers silent: every collective keeps its local half and
    receives zeros (all_gather / all_to_all) or nothing (reductions) from the
    other ranks.  Used to time the CPU baseline of a single shard at full
    size without executing the peers' share of the work."""

    def __init__(self, program: torch.fx.GraphModule, rank: int, dtype: str = "fp32"):
        super().__init__([program], dtype)
        self.rank = rank

    def forward(self, x, y):
        env = self.env[0]
        prog = self.programs[0]
        look = lambda a: torch.fx.node.map_arg(a, lambda n: env[n.name])
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
            else:
                t = node.target
                if t is product_collectives.all_gather:
                    xin, dim, L, rank = look(node.args)
                    parts = []
                    for i, l in enumerate(L):
                        if i == rank:
                            parts.append(xin)
                        else:
                            shape = list(xin.shape)
                            shape[dim] = l
                            parts.append(torch.zeros(shape, dtype=xin.dtype))
                    env[node.name] = torch.cat(parts, dim=dim)
                elif t is product_collectives.reduce_scatter:
                    xin, dim, L, rank = look(node.args)
                    env[node.name] = torch.split(xin, list(L), dim=dim)[rank].contiguous()
                elif t is product_collectives.all_to_all:
                    xin, sd, cd, sL, cL, rank = look(node.args)
                    own = torch.split(xin, list(sL), dim=sd)[rank]
                    parts = []
                    for i, l in enumerate(cL):
                        if i == rank:
                            parts.append(own)
                        else:
                            shape = list(own.shape)
                            shape[cd] = l
                            parts.append(torch.zeros(shape, dtype=own.dtype))
                    env[node.name] = torch.cat(parts, dim=cd)
                elif t in (product_collectives.all_reduce, product_collectives.replicate):
                    env[node.name] = look(node.args[0])
                else:
                    env[node.name] = self._call_local(0, node)
        raise RuntimeError("program has no output node")
