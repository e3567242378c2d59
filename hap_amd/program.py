"""Generator of the per-device SPMD program as a ``torch.fx`` graph.

The reference obtains this graph from its synthesizer (``hap.main``,
/root/reference/hap.rs:81-188); the search and the LP are outside this
package, so the graph is generated directly for fixed, legal plans.  Every
node uses the form the reference's code generator emits, so an executor for
these graphs is an executor for the synthesizer's output:

* inputs       placeholder -> ``.split(lengths, dim)`` -> ``getitem(rank)``  (hap.rs:2504-2520)
* parameters   replicated: ``get_attr`` -> ``collectives.replicate``          (hap.rs:2561-2568)
               ZeRO: ``get_attr`` of the dim-0 shard -> ``collectives.all_gather(p, 0, L, rank)``
                                                                             (hap.rs:2527-2547)
               sharded: ``get_attr`` of a tensor sliced in place             (hap.rs:2588-2596, 36-47)
* ops          ``F.linear(x, w, b)`` (1032), ``torch.transpose(x, a, b)`` (1213),
               ``F.multi_head_attention_forward(**kw)`` + 2 getitems (1301-1327),
               ``F.relu(x, inplace=..)`` (1417), ``F.dropout(x, p)`` (1464),
               ``operator.add`` (1515), ``operator.mul(x, num)`` (1563),
               ``F.layer_norm(x, shape)`` (1653), ``F.conv2d(x, w, b, stride, padding, (1, 1), 1)`` (1723),
               ``torch.flatten(x, start, -1)`` (1779), ``torch.log_softmax(x, dim)`` (1829),
               ``F.nll_loss(x, y, reduction=..)`` (1881), ``F.embedding(ids, table)`` (2041),
               ``models.append_cls_token`` (2093), ``models.get_cls_token`` (2141),
               ``models.top_2_gating(x, E, C, wg)`` + 2 getitems (2201-2203),
               ``torch.einsum(code, a, b)`` (2273)
* collectives  ``all_gather(t, dim, L, rank)`` (2641), ``dynamic_slice`` (2662),
               ``reduce_scatter`` (2680), ``all_reduce(t)`` (2701),
               ``all_to_all(t, split_dim, cat_dim, split_L, cat_L, rank)`` (2723-2730)
* output       the device's partial loss (hap.rs:2602-2615)

Plans (each step is a legal Hoare triple of hap.rs:2786-3419):
``ffn="column"``  batch-sharded attention, all_gather, column-sharded FFN1 on
                  the replicated rows, all_to_all, batch-sharded FFN2;
``ffn="batch"``   pure uneven data parallelism;
MoE layers        gating on replicated tokens, experts sharded over the
                  expert dimension, combine -> reduce_scatter / all_reduce
                  (``moe="experts"``); ``moe="capacity"`` / ``"hidden"`` /
                  ``"model"`` / ``"sequence"``: the capacity slots, the experts'
                  hidden features, the tokens' model dimension or their
                  positions are split instead (see ShardingPlan.moe).
``attn="heads"``  attention sharded over heads instead of samples (uneven head
                  counts: rows of the in-projection, columns of the
                  out-projection), all_gather before, reduce_scatter after;
                  a form the reference's synthesizer cannot emit.
``zero=True``     on top of any of them: every parameter that would be
                  replicated is stored as a dim-0 shard (the reference's
                  ``extra_ps`` / force_zero mode).
``shard_dim="sequence"``  (language models, ``ffn="batch"``) inputs, embedding,
                  LayerNorm, FFN, decoder and loss on the device's uneven share
                  of the POSITIONS of every sample; around attention, which
                  needs whole sequences, ``all_gather(h, 1, ..)`` before and
                  ``dynamic_slice(out, 1, ..)`` after (each rank computes the
                  attention of all samples; ``replicate``'s backward sums the
                  parameter gradients).
``embedding="features"``  the embedding table sharded on dim 1 (its output
                  gathered on dim 2), ``all_gather(.., 2, ..)`` and, for the
                  batch-sharded plans, ``dynamic_slice(.., 0, ..)`` behind it.
"""
from __future__ import annotations

import math
import operator
from typing import Optional

import torch
import torch.fx
import torch.nn as nn
import torch.nn.functional as F

from . import collectives, models
from .sharding import ShardingPlan, shard_heads_inplace, shard_inplace


class _Emitter:
    def __init__(self, module: nn.Module, plan: ShardingPlan):
        self.g = torch.fx.Graph()
        self.module = module
        self.plan = plan
        self.rank = plan.rank
        self._attr_cache = {}

    # inputs -------------------------------------------------------------
    def sharded_input(self, name: str, full_length: int, dim: int = 0):
        ph = self.g.placeholder(name)
        chunks = self.g.call_method("split", (ph, self.plan.lengths(full_length), dim))
        return self.g.call_function(operator.getitem, (chunks, self.rank))

    def whole_input(self, name: str):
        return self.g.placeholder(name)

    # parameters ---------------------------------------------------------
    def replicated(self, target: str):
        """A parameter or buffer every device needs whole: kept whole and ``replicate``d (hap.rs:2561-2568), or,
        under ``plan.zero``, stored as its dim-0 shard and ``all_gather``ed at use (get_attr_zero,
        hap.rs:2527-2547; a leading dimension of 1 keeps the replicated form, as there)."""
        if target not in self._attr_cache:
            if self.plan.zero and self._shape(target)[0] != 1:
                lengths = self.plan.lengths(self._shape(target)[0])
                shard_inplace(self.module, target, lengths, 0, self.rank)
                attr = self.g.get_attr(target)
                self._attr_cache[target] = self.g.call_function(collectives.all_gather, (attr, 0, lengths, self.rank))
            else:
                attr = self.g.get_attr(target)
                self._attr_cache[target] = self.g.call_function(collectives.replicate, (attr,))
        return self._attr_cache[target]

    def _shape(self, target: str):
        obj = self.module
        for atom in target.split("."):
            obj = getattr(obj, atom)
        return tuple(obj.shape)

    def sharded(self, target: str, full_length: int, dim: int):
        if target not in self._attr_cache:
            shard_inplace(self.module, target, self.plan.lengths(full_length), dim, self.rank)
            self._attr_cache[target] = self.g.get_attr(target)
        return self._attr_cache[target]

    def sharded_as(self, target: str, lengths, dim: int):
        """Like ``sharded`` with the lengths given (head counts scaled by the head width)."""
        if target not in self._attr_cache:
            shard_inplace(self.module, target, list(lengths), dim, self.rank)
            self._attr_cache[target] = self.g.get_attr(target)
        return self._attr_cache[target]

    def head_sharded(self, target: str, head_lengths, head_dim: int):
        if target not in self._attr_cache:
            shard_heads_inplace(self.module, target, list(head_lengths), head_dim, self.rank)
            self._attr_cache[target] = self.g.get_attr(target)
        return self._attr_cache[target]

    def call(self, fn, *args, **kwargs):
        return self.g.call_function(fn, tuple(args), kwargs or None)


def _head_parallel_attention(e: _Emitter, h, prefix: str, emsize: int, nheads: int, p: float, mask, B: int):
    """Attention sharded over heads: the batch is gathered, every device runs its (uneven) share of the heads on
    all samples with the matching rows of the in-projection and columns of the out-projection, and the partial
    outputs are reduce-scattered back to the batch sharding; the output bias is added once, after the sum."""
    plan = e.plan
    hd = emsize // nheads
    L_B, L_H = plan.lengths(B), plan.lengths(nheads)
    if min(L_H) < 1:
        raise ValueError(f"{nheads} heads over ratios {plan.ratios[0]} leave a device without a head")
    full = e.call(collectives.all_gather, h, 0, L_B, e.rank)
    partial = e.call(models.head_parallel_attention, full,
                     e.head_sharded(prefix + "self_attn.in_proj_weight", L_H, hd),
                     e.head_sharded(prefix + "self_attn.in_proj_bias", L_H, hd),
                     e.sharded_as(prefix + "self_attn.out_proj.weight", [l * hd for l in L_H], 1),
                     L_H[e.rank], mask)
    out = e.call(collectives.reduce_scatter, partial, 0, L_B, e.rank)
    out = e.call(operator.add, out, e.replicated(prefix + "self_attn.out_proj.bias"))
    out = e.call(F.dropout, out, p)
    s = e.call(operator.add, h, out)
    return e.call(F.layer_norm, s, (emsize,))


def _attention(e: _Emitter, h, prefix: str, emsize: int, nheads: int, p: float, mask, seq_lengths=None):
    """``seq_lengths``: h is sharded over positions (dim 1); attention runs on the gathered sequences and its result
    is cut back to the device's positions."""
    local = h
    if seq_lengths is not None:
        h = e.call(collectives.all_gather, h, 1, seq_lengths, e.rank)
    t = e.call(torch.transpose, h, 0, 1)
    kw = dict(query=t, key=t, value=t,
              in_proj_weight=e.replicated(prefix + "self_attn.in_proj_weight"),
              in_proj_bias=e.replicated(prefix + "self_attn.in_proj_bias"),
              out_proj_weight=e.replicated(prefix + "self_attn.out_proj.weight"),
              out_proj_bias=e.replicated(prefix + "self_attn.out_proj.bias"))
    if mask is not None:
        kw["attn_mask"] = mask
    kw.update(embed_dim_to_check=emsize, num_heads=nheads, bias_k=None, bias_v=None,
              add_zero_attn=False, dropout_p=p)
    both = e.g.call_function(F.multi_head_attention_forward, (), kw)
    out = e.call(operator.getitem, both, 0)
    e.call(operator.getitem, both, 1)            # head-averaged probabilities: bound, never consumed
    out = e.call(torch.transpose, out, 0, 1)
    if seq_lengths is not None:
        out = e.call(collectives.dynamic_slice, out, 1, seq_lengths, e.rank)
    out = e.call(F.dropout, out, p)
    s = e.call(operator.add, local, out)
    return e.call(F.layer_norm, s, (emsize,))


def _activation(e: _Emitter, x, activation: str):
    if activation == "relu":
        return e.g.call_function(F.relu, (x,), {"inplace": False})
    if activation == "gelu":
        return e.call(F.gelu, x)
    raise ValueError(f"activation {activation!r} has no handler")


def _dense_ffn(e: _Emitter, h1, prefix: str, emsize: int, nhid: int, B: int, p: float,
               activation: str, batch_sharded: bool):
    plan = e.plan
    if plan.ffn == "column" and batch_sharded:
        L_B, L_F = plan.lengths(B), plan.lengths(nhid)
        full = e.call(collectives.all_gather, h1, 0, L_B, e.rank)
        u = e.call(F.linear, full, e.sharded(prefix + "linear1.weight", nhid, 0),
                   e.sharded(prefix + "linear1.bias", nhid, 0))
        u = e.call(collectives.all_to_all, u, 0, 2, L_B, L_F, e.rank)
    else:
        u = e.call(F.linear, h1, e.replicated(prefix + "linear1.weight"), e.replicated(prefix + "linear1.bias"))
    u = _activation(e, u, activation)
    u = e.call(F.dropout, u, p)
    o = e.call(F.linear, u, e.replicated(prefix + "linear2.weight"), e.replicated(prefix + "linear2.bias"))
    o = e.call(F.dropout, o, p)
    s = e.call(operator.add, h1, o)
    return e.call(F.layer_norm, s, (emsize,))


def _moe_ffn(e: _Emitter, h1, prefix: str, emsize: int, n_expert: int, capacity: int, B: int,
             batch_sharded: bool, gating=models.top_2_gating, seqlen: Optional[int] = None):
    L_E = e.plan.lengths(n_expert)
    if batch_sharded:
        L_B = e.plan.lengths(B)
        tokens = e.call(collectives.all_gather, h1, 0, L_B, e.rank)
    else:
        tokens = h1
    routed = e.call(gating, tokens, n_expert, capacity, e.replicated(prefix + "gate_weight"))
    dispatch = e.call(operator.getitem, routed, 0)
    combine = e.call(operator.getitem, routed, 1)
    if e.plan.moe == "experts":
        # expert split: (identity, gather(1, 2)) -> gather(0, 1) / (gather(0, 0), gather(1, 1)) -> gather(0, 1) /
        # (gather(0, 1), gather(1, 2)) -> reduce (hap.rs:3316-3320, 3333-3337, 3363-3367, 3393-3397)
        dispatch = e.call(collectives.dynamic_slice, dispatch, 2, L_E, e.rank)
        combine = e.call(collectives.dynamic_slice, combine, 2, L_E, e.rank)
        w1 = e.sharded(prefix + "w1", n_expert, 0)
        w2 = e.sharded(prefix + "w2", n_expert, 0)
    elif e.plan.moe == "capacity":
        # capacity split: (identity, gather(1, 3)) -> gather(0, 2) / (identity, gather(1, 2)) -> gather(0, 2) /
        # (gather(0, 2), gather(1, 3)) -> reduce (hap.rs:3322-3326, 3357-3361, 3387-3391, 3399-3403)
        L_C = e.plan.lengths(capacity)
        dispatch = e.call(collectives.dynamic_slice, dispatch, 3, L_C, e.rank)
        combine = e.call(collectives.dynamic_slice, combine, 3, L_C, e.rank)
        w1 = e.replicated(prefix + "w1")
        w2 = e.replicated(prefix + "w2")
    elif e.plan.moe == "hidden":
        # feature split of the expert FFN: (gather(0, 2), identity) -> gather(0, 3) for the first product,
        # (gather(0, 1), gather(1, 3)) -> reduce for the second (hap.rs:3345-3349, 3369-3373)
        nhid = e._shape(prefix + "w1")[2]
        w1 = e.sharded(prefix + "w1", nhid, 2)
        w2 = e.sharded(prefix + "w2", nhid, 1)
    elif e.plan.moe == "model":
        # split of the model dimension: the tokens' columns (gather(0, 2), identity) -> gather(0, 3) for the dispatch,
        # (gather(0, 1), gather(1, 3)) -> reduce for the first product, (gather(0, 2), identity) -> gather(0, 3) for
        # the second, (gather(0, 3), identity) -> gather(0, 2) for the combine (hap.rs:3306-3310, 3331-3335,
        # 3368-3372, 3405-3409); the gating sees whole token rows
        L_D = e.plan.lengths(emsize)
        w1 = e.sharded(prefix + "w1", emsize, 1)
        w2 = e.sharded(prefix + "w2", emsize, 2)
    elif e.plan.moe == "sequence":
        # split along the sequence: tokens and dispatch tensor windowed over positions, (gather(0, 1), gather(1, 1)) ->
        # reduce (hap.rs:3300-3304); the expert products on the reduced, whole tensor (identity); the combine tensor
        # windowed over positions gives the output gathered on dim 1.  (The reference's fifth triple of the combine,
        # hap.rs:3411-3415, names dim 2 of the combine tensor next to an output gathered on dim 1; positions are the
        # only dimension of that operand which gives such an output, and that is what is emitted here.)
        L_S = e.plan.lengths(seqlen)
        dispatch = e.call(collectives.dynamic_slice, dispatch, 1, L_S, e.rank)
        combine = e.call(collectives.dynamic_slice, combine, 1, L_S, e.rank)
        w1 = e.replicated(prefix + "w1")
        w2 = e.replicated(prefix + "w2")
    else:
        raise ValueError(f"unknown MoE split {e.plan.moe!r}")
    model_split, seq_split = e.plan.moe == "model", e.plan.moe == "sequence"
    x = tokens
    if model_split:
        x = e.call(collectives.dynamic_slice, tokens, 2, L_D, e.rank)
    if seq_split:
        x = e.call(collectives.dynamic_slice, tokens, 1, L_S, e.rank)
    x = e.call(torch.einsum, "bsd,bsec->becd", x, dispatch)
    if seq_split:
        x = e.call(collectives.all_reduce, x)            # every device placed the tokens of its positions
    x = e.call(torch.einsum, "edh,becd->bech", w1, x)
    if model_split:
        x = e.call(collectives.all_reduce, x)            # every device holds a partial sum over its columns of d
    x = e.g.call_function(F.relu, (x,), {"inplace": False})
    x = e.call(torch.einsum, "ehd,bech->becd", w2, x)
    partial = e.call(torch.einsum, "becd,bsec->bsd", x, combine)
    if model_split or seq_split:
        o = e.call(collectives.all_gather, partial, 2 if model_split else 1, L_D if model_split else L_S, e.rank)
        if batch_sharded:
            o = e.call(collectives.dynamic_slice, o, 0, L_B, e.rank)
    elif batch_sharded:
        o = e.call(collectives.reduce_scatter, partial, 0, L_B, e.rank)
    else:
        o = e.call(collectives.all_reduce, partial)
    s = e.call(operator.add, h1, o)
    return e.call(F.layer_norm, s, (emsize,))


def build_program(model: nn.Module, plan: ShardingPlan, global_batch: int,
                  activation: str = "relu", batch_sharded: bool = True) -> torch.fx.GraphModule:
    """Slice ``model``'s parameters in place for ``plan.rank`` and return the
    rank's program.  ``batch_sharded=False`` keeps the batch replicated (every
    op on the whole batch; only expert weights are sharded)."""
    e = _Emitter(model, plan)
    B = global_batch
    p = float(model.dropout_p)
    d = model.emsize

    seq_lengths = None
    if plan.shard_dim not in ("batch", "sequence") or plan.embedding not in ("rows", "features"):
        raise ValueError("ShardingPlan: shard_dim is 'batch' or 'sequence', embedding is 'rows' or 'features'")
    if plan.shard_dim == "sequence" or plan.embedding == "features":
        if model.family != "lm" or not batch_sharded or plan.attn != "batch":
            raise ValueError("shard_dim='sequence' / embedding='features' are plans of the batch-attention language models")
        if plan.shard_dim == "sequence" and (plan.ffn != "batch" or any(isinstance(l, models.Top2TransformerEncoderLayer)
                                                                           for l in model.layers)):
            raise ValueError("shard_dim='sequence' goes with ffn='batch' and dense layers")
    if model.family == "lm":
        sdim = 1 if plan.shard_dim == "sequence" else 0
        extent = model.seqlen if sdim == 1 else B
        if sdim == 1:
            seq_lengths = plan.lengths(model.seqlen)
        if not batch_sharded:
            x, y = e.whole_input("x"), e.whole_input("y")
        elif plan.embedding == "features":
            x, y = e.whole_input("x"), e.sharded_input("y", extent, sdim)
        else:
            x, y = e.sharded_input("x", extent, sdim), e.sharded_input("y", extent, sdim)
        if plan.embedding == "features":
            # table sharded over the embedding width: whole ids, output gathered on dim 2 (hap.rs:3220-3224), made
            # whole by an all_gather and cut to the device's samples / positions
            L_d = plan.lengths(d)
            h = e.call(F.embedding, x, e.sharded("encoder.weight", d, 1))
            h = e.call(collectives.all_gather, h, 2, L_d, e.rank)
            h = e.call(collectives.dynamic_slice, h, sdim, plan.lengths(extent), e.rank)
        else:
            h = e.call(F.embedding, x, e.replicated("encoder.weight"))
        h = e.call(operator.mul, h, math.sqrt(d))
        if sdim == 1:
            h = e.call(operator.add, h, e.sharded("pe", model.seqlen, 1))     # [1, s, d]: the device's positions
        else:
            h = e.call(operator.add, h, e.g.get_attr("pe"))      # [1,S,d]: size-1 dim, never split
        mask = e.replicated("src_mask") if getattr(model, "src_mask", None) is not None else None
    elif model.family == "vit":
        if plan.patch_embed not in ("batch", "features"):
            raise ValueError("ShardingPlan: patch_embed is 'batch' or 'features'")
        x = e.whole_input("x") if plan.patch_embed == "features" else e.sharded_input("x", B)
        y = e.sharded_input("y", B)
        pe = model.patch_embed
        if plan.patch_embed == "features":
            # the convolution's kernel and bias sliced over the output channels, whole images: output gathered on
            # dim 1 (hap.rs:3083-3087); flatten keeps it (a communicatable tensor, hap.rs:1794), the all_gather makes it
            # whole; transpose and the class token run on the whole batch, whose rows are then cut to the device's
            # images (append_cls_token's output is communicatable, hap.rs:2107)
            if not batch_sharded or plan.zero:
                raise ValueError("patch_embed='features' is a plan of the batch-sharded ViT with whole parameters")
            L_d = plan.lengths(d)
            c = e.call(F.conv2d, x, e.sharded("patch_embed.proj.weight", d, 0), e.sharded("patch_embed.proj.bias", d, 0),
                       tuple(pe.patch_size), (0, 0), (1, 1), 1)
            c = e.call(torch.flatten, c, 2, -1)
            c = e.call(collectives.all_gather, c, 1, L_d, e.rank)
            c = e.call(torch.transpose, c, 1, 2)
            c = e.call(models.append_cls_token, c, e.replicated("cls_token"))
            c = e.call(collectives.dynamic_slice, c, 0, plan.lengths(B), e.rank)
        else:
            c = e.call(F.conv2d, x, e.replicated("patch_embed.proj.weight"), e.replicated("patch_embed.proj.bias"),
                       tuple(pe.patch_size), (0, 0), (1, 1), 1)
            c = e.call(torch.flatten, c, 2, -1)
            c = e.call(torch.transpose, c, 1, 2)
            c = e.call(models.append_cls_token, c, e.replicated("cls_token"))
        h = e.call(operator.add, c, e.replicated("pos_embed"))
        mask = None
    else:
        raise ValueError(f"model family {model.family!r} has no handler")

    for i, layer in enumerate(model.layers):
        prefix = f"layers.{i}."
        if plan.attn == "heads" and batch_sharded:
            h1 = _head_parallel_attention(e, h, prefix, d, model.nheads, p, mask, B)
        else:
            h1 = _attention(e, h, prefix, d, model.nheads, p, mask, seq_lengths)
        if isinstance(layer, models.Top2TransformerEncoderLayer):
            # the switch layer takes the top-2 layer's node forms with its own gating leaf (the reference's
            # synthesizer has no handler for models.switch_gating; its models call it at models.py:421)
            gating = (models.switch_gating if isinstance(layer, models.SwitchTransformerEncoderLayer)
                      else models.top_2_gating)
            h = _moe_ffn(e, h1, prefix, d, layer.n_expert, layer.capacity, B, batch_sharded, gating,
                         seqlen=model.seqlen + (1 if model.family == "vit" else 0))
        else:
            h = _dense_ffn(e, h1, prefix, d, model.nhid, B, p, activation, batch_sharded)

    if plan.decoder not in ("whole", "vocabulary"):
        raise ValueError("ShardingPlan: decoder is 'whole' or 'vocabulary'")
    vocab_split = plan.decoder == "vocabulary"
    if vocab_split and (not batch_sharded or plan.shard_dim != "batch" or plan.zero):
        raise ValueError("decoder='vocabulary' is a plan of the batch-sharded programs with whole parameters")

    def decode(t, cat_dim):
        """The output projection; ``cat_dim``: the logits' class dimension.  Vocabulary split: the feature partition of a linear (hap.rs:2807-2816) needs its
        input whole, so the activations are gathered over the batch, every device computes its columns of the logits
        for all samples, and one all_to_all (split along the batch, concatenated along the classes: the exchange of
        the column-sharded FFN, hap.rs:2713-2744) gives the device's samples their whole rows for log_softmax."""
        if not vocab_split:
            return e.call(F.linear, t, e.replicated("decoder.weight"), e.replicated("decoder.bias"))
        V = e._shape("decoder.weight")[0]
        L_B, L_V = plan.lengths(B), plan.lengths(V)
        full = e.call(collectives.all_gather, t, 0, L_B, e.rank)
        u = e.call(F.linear, full, e.sharded("decoder.weight", V, 0), e.sharded("decoder.bias", V, 0))
        return e.call(collectives.all_to_all, u, 0, cat_dim, L_B, L_V, e.rank)

    if model.family == "lm":
        logits = decode(h, 2)
        lp = e.call(torch.log_softmax, logits, 2)
        lp = e.call(torch.transpose, lp, 1, 2)
    else:
        c = e.call(models.get_cls_token, h)
        logits = decode(c, 1)
        lp = e.call(torch.log_softmax, logits, 1)
    loss = e.g.call_function(F.nll_loss, (lp, y), {"reduction": "sum"})
    e.g.output(loss)
    e.g.lint()
    return torch.fx.GraphModule(model, e.g)
