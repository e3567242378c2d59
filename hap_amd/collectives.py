"""Drop-in for /root/reference/collectives.py: the same six callables with the
same signatures, usable directly on GPU tensors and as node targets of the
emitted program.

    all_gather(tensor, dim, sharding_lengths, rank)           collectives.py:70
    reduce_scatter(tensor, dim, sharding_lengths, rank)       collectives.py:142
    dynamic_slice(tensor, dim, sharding_lengths, rank)        collectives.py:146-148
    all_to_all(tensor, split_dim, cat_dim, split_L, cat_L, rank)   collectives.py:168
    all_reduce(tensor)                                         collectives.py:86
    replicate(tensor)                                          collectives.py:182

Each call runs its device-local half (pad / split / slice / concat / rank-ordered
sum) as HIP kernels and takes the peers' messages from the wire installed with
``set_wire`` (see ``hap_amd.wire``).  Messages are keyed by a per-function call
counter (``all_gather#0``, ...) which ``reset_tags`` rewinds.  CPU tensors are
refused.
"""
from __future__ import annotations

from collections import defaultdict
from typing import Optional

import torch

from . import ops
from .wire import SilentWire, Wire

_wire: Wire = SilentWire()
_counters = defaultdict(int)


def set_wire(wire: Wire) -> None:
    global _wire
    _wire = wire
    reset_tags()


def reset_tags() -> None:
    _counters.clear()


def _tag(kind: str) -> str:
    t = f"{kind}#{_counters[kind]}"
    _counters[kind] += 1
    return t


def _shape_with(shape, dim, n):
    return tuple(shape[:dim]) + (n,) + tuple(shape[dim + 1:])


def _gather_local(tag, direction, x, dim, L, rank):
    """pad own shard, take the peers' padded shards from the wire, cut the pads and concatenate."""
    m = max(L)
    own = ops.pad_rows(x.contiguous(), dim, m)
    slices = []
    for src in range(len(L)):
        if src == rank:
            slices.append(own)
        else:
            t = _wire.recv(tag, direction, src, own.shape, own.dtype, own.device)
            slices.append(t if t is not None else own)
    lengths = list(L)
    return ops.unpad_concat(slices, lengths, dim)


def _scatter_local(tag, direction, x, dim, L, rank):
    """split + pad the full tensor, sum own piece with the peers' pieces for this rank, cut the pad."""
    m = max(L)
    sent = ops.split_pad(x.contiguous(), list(L), dim, m)
    contribs = []
    for src in range(len(L)):
        if src == rank:
            contribs.append(sent[rank])
        else:
            t = _wire.recv(tag, direction, src, sent[rank].shape, x.dtype, x.device, reduction=True)
            if t is not None:
                contribs.append(t)
    return ops.ragged_reduce(contribs, dim, 0, L[rank])


class _AllGather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, dim, sharding_lengths, rank):
        ctx.meta = (dim, list(sharding_lengths), rank, _tag("all_gather"))
        return _gather_local(ctx.meta[3], "fwd", tensor, dim, ctx.meta[1], rank)

    @staticmethod
    def backward(ctx, grad_output):
        dim, L, rank, tag = ctx.meta
        return _scatter_local(tag, "bwd", grad_output, dim, L, rank), None, None, None


class _ReduceScatter(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, dim, sharding_lengths, rank):
        ctx.meta = (dim, list(sharding_lengths), rank, _tag("reduce_scatter"))
        return _scatter_local(ctx.meta[3], "fwd", tensor, dim, ctx.meta[1], rank)

    @staticmethod
    def backward(ctx, grad_output):
        dim, L, rank, tag = ctx.meta
        return _gather_local(tag, "bwd", grad_output, dim, L, rank), None, None, None


def _exchange(tag, direction, x, split_dim, cat_dim, split_L, cat_L, rank):
    pieces = ops.split_rows(x.contiguous(), list(split_L), split_dim)
    own = pieces[rank]
    parts = []
    for src in range(len(cat_L)):
        if src == rank:
            parts.append(own)
        else:
            shape = _shape_with(own.shape, cat_dim, cat_L[src])
            t = _wire.recv(tag, direction, src, shape, x.dtype, x.device)
            parts.append(t)
    return ops.concat_rows(parts, cat_dim)


class _AllToAll(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, split_dim, cat_dim, split_L, cat_L, rank):
        ctx.meta = (split_dim, cat_dim, list(split_L), list(cat_L), rank, _tag("all_to_all"))
        return _exchange(ctx.meta[5], "fwd", tensor, split_dim, cat_dim, ctx.meta[2], ctx.meta[3], rank)

    @staticmethod
    def backward(ctx, grad_output):
        split_dim, cat_dim, split_L, cat_L, rank, tag = ctx.meta
        g = _exchange(tag, "bwd", grad_output, cat_dim, split_dim, cat_L, split_L, rank)
        return g, None, None, None, None, None


def _sum_with_peers(tag, direction, x, world: Optional[int] = None):
    x = x.contiguous()
    contribs = [x]
    n = world if world is not None else getattr(_wire, "world_size", 1)
    rank = getattr(_wire, "rank", 0)
    ordered = []
    for src in range(n):
        if src == rank:
            ordered.append(x)
        else:
            t = _wire.recv(tag, direction, src, x.shape, x.dtype, x.device, reduction=True)
            if t is not None:
                ordered.append(t)
    contribs = ordered or contribs
    flat = [c.view(1, -1) for c in contribs]
    return ops.ragged_reduce(flat, 1, 0, x.numel()).view(x.shape)


class _AllReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor):
        ctx.tag = _tag("all_reduce")
        return _sum_with_peers(ctx.tag, "fwd", tensor)

    @staticmethod
    def backward(ctx, grad_output):
        return _sum_with_peers(ctx.tag, "bwd", grad_output)


class _Replicate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor):
        ctx.tag = _tag("replicate")
        return tensor.view_as(tensor)

    @staticmethod
    def backward(ctx, grad_output):
        return _sum_with_peers(ctx.tag, "bwd", grad_output)


class _DynamicSlice(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tensor, dim, sharding_lengths, rank):
        L = list(sharding_lengths)
        ctx.meta = (dim, sum(L[:rank]), tensor.shape)
        return ops.slice_rows(tensor.contiguous(), dim, ctx.meta[1], L[rank])

    @staticmethod
    def backward(ctx, grad_output):
        dim, offset, shape = ctx.meta
        g = torch.empty(shape, dtype=grad_output.dtype, device=grad_output.device)
        ops.fill_zero(g)
        ops.place_rows(grad_output.contiguous(), g, dim, offset)
        return g, None, None, None


def all_gather(tensor, dim, sharding_lengths, rank): return _AllGather.apply(tensor, dim, sharding_lengths, rank)
def reduce_scatter(tensor, dim, sharding_lengths, rank): return _ReduceScatter.apply(tensor, dim, sharding_lengths, rank)
def dynamic_slice(tensor, dim, sharding_lengths, rank): return _DynamicSlice.apply(tensor, dim, sharding_lengths, rank)
def all_to_all(tensor, split_dim, cat_dim, split_sharding_lengths, cat_sharding_lengths, rank): return _AllToAll.apply(tensor, split_dim, cat_dim, split_sharding_lengths, cat_sharding_lengths, rank)
def all_reduce(tensor): return _AllReduce.apply(tensor)
def replicate(tensor): return _Replicate.apply(tensor)
