"""Integer shard lengths and in-place parameter slicing.

``sharding_round`` is the layout contract of the whole program: every split,
pad and concat extent is derived from it (/root/reference/hap.rs:3536-3559,
exported to Python at hap.rs:211-218 as a function that overwrites the ratio
list with the integer lengths).  The arithmetic runs in the native library
(``hapmi_sharding_round``); there is no Python fallback.

``shard_inplace`` follows split_param_or_buffer (hap.rs:36-47).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

import torch

from . import _lib


def sharding_lengths(full_length: int, ratios: Sequence[float]) -> List[int]:
    """Integer lengths for ``full_length`` units under ``ratios`` (pure)."""
    n = len(ratios)
    r = (ctypes.c_double * n)(*[float(x) for x in ratios])
    out = (ctypes.c_int64 * n)()
    _lib.check(_lib.lib().hapmi_sharding_round(int(full_length), r, n, out))
    return [int(v) for v in out]


def sharding_round(full_length: int, ratios: list) -> None:
    """Drop-in for ``hap.sharding_round``: overwrites ``ratios`` in place with
    the integer lengths (hap.rs:211-218)."""
    lengths = sharding_lengths(full_length, ratios)
    for i, v in enumerate(lengths):
        ratios[i] = v


def shard_inplace(module: torch.nn.Module, target: str, lengths: Sequence[int], dim: int, rank: int) -> None:
    """``p.data = torch.split(p.data, lengths, dim)[rank]``; a dimension of
    size 1 is left alone (the broadcast hack, hap.rs:44-45)."""
    try:
        p = module.get_parameter(target)
    except AttributeError:
        p = module.get_buffer(target)
    if p.data.shape[dim] == 1:
        return
    p.data = torch.split(p.data, list(lengths), dim)[rank].contiguous()


def shard_heads_inplace(module: torch.nn.Module, target: str, head_lengths: Sequence[int], head_dim: int,
                        rank: int) -> None:
    """Keep the q, k and v rows of this rank's heads of a packed in-projection ([3 * H * head_dim, ...] weight or
    bias): rows [lo, hi) * head_dim of each of the three blocks, stacked in q, k, v order."""
    try:
        p = module.get_parameter(target)
    except AttributeError:
        p = module.get_buffer(target)
    H = sum(head_lengths)
    if p.data.shape[0] != 3 * H * head_dim:
        raise ValueError(f"{target}: leading dimension {p.data.shape[0]} is not 3 * {H} heads * {head_dim}")
    lo = sum(head_lengths[:rank])
    blocks = p.data.view(3, H, head_dim, *p.data.shape[1:])[:, lo:lo + head_lengths[rank]]
    p.data = blocks.reshape(3 * head_lengths[rank] * head_dim, *p.data.shape[1:]).contiguous()


@dataclass
class ShardingPlan:
    """Per-segment device ratios plus this device's rank (hap.rs:865, 178-180)."""
    ratios: List[List[float]]
    rank: int
    ffn: str = "column"          # "column": FFN1 column-sharded (plan P1); "batch": pure DP (plan P2)
    segment: int = 0
    attn: str = "batch"          # "batch": attention on the device's samples; "heads": on the device's heads of every sample
    zero: bool = False           # parameters stored as dim-0 shards and all_gather-ed at use (hap.rs:2527-2547)
    shard_dim: str = "batch"     # language models: "batch" shards inputs / activations over samples (dim 0),
                                 # "sequence" over positions (dim 1: hap.rs:2500-2520 shards a placeholder on any
                                 # dimension; linear / layer_norm / embedding / add keep a gather on any leading one,
                                 # hap.rs:2795, 3061, 3214-3218, 2996; attention needs the whole sequence)
    embedding: str = "rows"      # "rows": ids sharded, table whole; "features": ids whole, table sharded on dim 1,
                                 # output gathered on dim 2 (hap.rs:3220-3224), then all_gather + dynamic_slice
    decoder: str = "whole"       # "whole": the output projection on the device's samples with the whole weight;
                                 # "vocabulary": its weight and bias sliced on dim 0 (the feature partition of a linear,
                                 # hap.rs:2807-2816): all_gather of the activations, the device's columns of the logits
                                 # for every sample, all_to_all back to whole rows of the device's samples
    patch_embed: str = "batch"   # ViT: "batch": the patch convolution on the device's images with the whole kernel;
                                 # "features": kernel and bias sliced on dim 0 and whole images (hap.rs:3083-3087),
                                 # output channels gathered behind the flatten, cut to the device's images behind the
                                 # class token
    moe: str = "experts"         # how the four MoE einsums are split (hap.rs:3285-3419): "experts": dispatch / combine
                                 # tensors sliced on dim 2, expert weights on dim 0; "capacity": dispatch / combine
                                 # sliced on dim 3 (every device takes a range of every expert's slots), expert weights
                                 # whole; "hidden": routing whole, first expert weight sliced on dim 2 and the second on
                                 # dim 1 (a feature split of the expert FFN; the second product is a partial sum, which is fed
                                 # to the combine einsum as it is and reduced after it: [B, S, d] instead of [B, E, C, d]
                                 # crosses the wire.  Equal by linearity, but not a program the reference's synthesizer
                                 # emits: it would all_reduce in front of the combine, hap.rs:3369-3373, 3385-3415);
                                 # "model": the tokens' model dimension (dispatch input sliced on dim 2, first weight
                                 # on dim 1 with its product all-reduced, second on dim 2, combine output gathered);
                                 # "sequence": tokens, dispatch and combine tensors sliced over positions (dim 1): the
                                 # dispatched tokens are all-reduced, every device runs the whole expert FFN, the
                                 # combine output is gathered on dim 1

    @property
    def world_size(self) -> int:
        return len(self.ratios[0])

    def lengths(self, full_length: int, segment: int = 0) -> List[int]:
        return sharding_lengths(full_length, self.ratios[min(segment, len(self.ratios) - 1)])
