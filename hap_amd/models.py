"""Model zoo and leaf ops of the shard program.

Mirrors the interface of /root/reference/models.py for the three families on
the hot path: ``RTransformer`` (models.py:65-88), ``VTransformer``
(models.py:147-177), ``RMoE`` (models.py:90-118) with
``Top2TransformerEncoderLayer`` (models.py:301-366), ``RSwitch`` (models.py:120-145) with
``SwitchTransformerEncoderLayer`` (models.py:368-434), and the leaf functions
the emitted program calls by name: ``top_2_gating`` (models.py:440-441,
477-502), ``switch_gating`` (436-437, 452-475), ``append_cls_token`` (443-445), ``get_cls_token`` (447-449),
``new_segment`` (531-533), ``positional_encoding`` (504-509).

The classes here are parameter containers with the reference's parameter
names; the sharded program that runs on the GPU is generated from them by
``hap_amd.program`` and executed by ``hap_amd.executor``.  The leaf functions
run hand-written HIP kernels and refuse CPU tensors.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch
import torch.fx
import torch.nn as nn


def positional_encoding(seqlen: int, emsize: int) -> np.ndarray:
    """Sinusoidal table [seqlen, emsize] in float64 (models.py:504-509):
    column j uses frequency 10000^(-2*(j//2)/emsize); even columns sin, odd cos."""
    # divide by 10000**e (not multiply by the inverse) so float64 rounding
    # agrees with the reference's table
    denom = np.power(10000.0, 2.0 * (np.arange(emsize) // 2) / emsize)
    angle = np.arange(seqlen, dtype=np.float64)[:, None] / denom[None, :]
    return np.where(np.arange(emsize)[None, :] % 2 == 0, np.sin(angle), np.cos(angle))


# ---------------------------------------------------------------------------
# leaf ops called by name from the emitted program
# ---------------------------------------------------------------------------

@torch.fx.wrap
def new_segment(x):
    """Marks the start of a new sharding-ratio segment (models.py:531-533)."""
    return x


@torch.fx.wrap
def append_cls_token(x, cls_token):
    """[N, T, d] -> [N, T+1, d] with the class token in row 0 (models.py:443-445)."""
    from . import ops
    return ops.append_cls_token(x, cls_token)


@torch.fx.wrap
def get_cls_token(x):
    """[N, T, d] -> [N, d], row 0 of every sample (models.py:447-449)."""
    from . import ops
    return ops.get_cls_token(x)


@torch.fx.wrap
def top_2_gating(gate_input, n_expert, capacity, gate_weight, train: bool = True):
    """Top-2 softmax gating with per-expert capacity (models.py:440-441, 477-502).
    Returns dense ``(dispatch, combine)``, each [B, S, E, C]; dispatch is float32."""
    from . import ops
    return ops.top_2_gating_dense(gate_input, n_expert, capacity, gate_weight)


@torch.fx.wrap
def switch_gating(gate_input, n_expert, capacity, gate_weight, train: bool = True):
    """Switch (top-1) softmax gating with per-expert capacity (models.py:436-437, 452-475).
    Returns dense ``(dispatch, combine)``, each [B, S, E, C]; dispatch is float32."""
    from . import ops
    return ops.switch_gating_dense(gate_input, n_expert, capacity, gate_weight)


@torch.fx.wrap
def head_parallel_attention(x, in_proj_weight, in_proj_bias, out_proj_weight, num_heads, attn_mask=None):
    """Self-attention over ``num_heads`` of a layer's heads: ``in_proj_weight`` [3 * num_heads * hd, d] holds the
    q, k and v rows of those heads, ``out_proj_weight`` [d, num_heads * hd] the matching columns of the output
    projection.  Returns the [B, S, d] partial output (no output bias): the sum of the partial outputs of a
    partition of the heads, plus the bias, is ``F.multi_head_attention_forward`` of the whole layer.  The
    reference has no head-sharded form (its attention handler shards the batch only, hap.rs:1243-1386)."""
    from . import ops
    return ops.head_parallel_attention(x, in_proj_weight, in_proj_bias, out_proj_weight, num_heads, attn_mask)


# ---------------------------------------------------------------------------
# parameter containers
# ---------------------------------------------------------------------------

class Top2TransformerEncoderLayer(nn.Module):
    """Self-attention + top-2 mixture-of-experts FFN (models.py:301-366).
    Parameters: self_attn.{in_proj_weight,in_proj_bias,out_proj.weight,out_proj.bias},
    gate_weight [d, E], w1 [E, d, h], w2 [E, h, d]; the two LayerNorms carry
    affine parameters that the emitted program never reads."""

    def __init__(self, d_model, nheads, d_hidden=2048, dropout=0.1, layer_norm_eps=1e-5,
                 n_expert=4, capacity=None):
        super().__init__()
        self.self_attn = nn.MultiheadAttention(d_model, nheads, dropout=dropout, batch_first=True)
        self.gate_weight = nn.Parameter(torch.empty(d_model, n_expert))
        self.w1 = nn.Parameter(torch.empty(n_expert, d_model, d_hidden))
        self.w2 = nn.Parameter(torch.empty(n_expert, d_hidden, d_model))
        for p in (self.gate_weight, self.w1, self.w2):
            nn.init.kaiming_uniform_(p, a=math.sqrt(5))
        self.norm1 = nn.LayerNorm(d_model, eps=layer_norm_eps)
        self.norm2 = nn.LayerNorm(d_model, eps=layer_norm_eps)
        self.dropout_p = dropout
        self.n_expert = n_expert
        self.capacity = capacity


class SwitchTransformerEncoderLayer(Top2TransformerEncoderLayer):
    """Self-attention + switch (top-1) mixture-of-experts FFN (models.py:368-434): the parameters of the top-2
    layer, routed by ``switch_gating``."""


def _encoder_layer(emsize, nheads, nhid, dropout):
    return nn.TransformerEncoderLayer(emsize, nheads, nhid, dropout, batch_first=True)


class RTransformer(nn.Module):
    """Post-LN transformer encoder language model (models.py:65-88)."""
    family = "lm"

    def __init__(self, ntokens, seqlen, emsize, nheads, nhid, dropout, nlayers=2, segmentation=True,
                 causal=True):
        super().__init__()
        self.ntokens, self.seqlen, self.emsize, self.nheads, self.nhid = ntokens, seqlen, emsize, nheads, nhid
        self.dropout_p = dropout
        self.register_buffer("pe", torch.tensor(positional_encoding(seqlen, emsize), dtype=torch.float32).unsqueeze(0))
        if causal:
            self.register_buffer("src_mask", torch.triu(torch.full((seqlen, seqlen), float("-inf")), diagonal=1))
        else:
            self.src_mask = None
        self.encoder = nn.Embedding(ntokens, emsize)
        self.layers = nn.ModuleList([_encoder_layer(emsize, nheads, nhid, dropout) for _ in range(nlayers)])
        self.decoder = nn.Linear(emsize, ntokens)
        self.segmentation = segmentation


class RMoE(nn.Module):
    """Transformer LM whose odd layers are top-2 MoE layers (models.py:90-118)."""
    family = "lm"

    def __init__(self, ntokens, seqlen, emsize, nheads, nhid, dropout, n_expert, capacity, nlayers,
                 segmentation=True, causal=True):
        super().__init__()
        self.ntokens, self.seqlen, self.emsize, self.nheads, self.nhid = ntokens, seqlen, emsize, nheads, nhid
        self.dropout_p = dropout
        self.n_expert, self.capacity = n_expert, capacity
        self.register_buffer("pe", torch.tensor(positional_encoding(seqlen, emsize), dtype=torch.float32).unsqueeze(0))
        if causal:
            self.register_buffer("src_mask", torch.triu(torch.full((seqlen, seqlen), float("-inf")), diagonal=1))
        else:
            self.src_mask = None
        self.encoder = nn.Embedding(ntokens, emsize)
        self.layers = nn.ModuleList([
            _encoder_layer(emsize, nheads, nhid, dropout) if i % 2 == 0 else
            Top2TransformerEncoderLayer(emsize, nheads, nhid, dropout, n_expert=n_expert, capacity=capacity)
            for i in range(nlayers)])
        self.decoder = nn.Linear(emsize, ntokens)
        self.segmentation = segmentation


class RSwitch(RMoE):
    """Transformer LM whose odd layers are switch MoE layers (models.py:120-145)."""

    def __init__(self, ntokens, seqlen, emsize, nheads, nhid, dropout, n_expert, capacity, nlayers,
                 segmentation=True, causal=True):
        super().__init__(ntokens, seqlen, emsize, nheads, nhid, dropout, n_expert, capacity, nlayers, segmentation,
                         causal)
        for i in range(1, nlayers, 2):
            self.layers[i] = SwitchTransformerEncoderLayer(emsize, nheads, nhid, dropout, n_expert=n_expert,
                                                           capacity=capacity)


class PatchEmbed(nn.Module):
    """Non-overlapping patch projection, kernel = stride (models.py:513-528)."""

    def __init__(self, img_size=(224, 224), patch_size=(16, 16), in_chans=3, embed_dim=768):
        super().__init__()
        self.img_size, self.patch_size = tuple(img_size), tuple(patch_size)
        self.grid_size = (img_size[0] // patch_size[0], img_size[1] // patch_size[1])
        self.num_patches = self.grid_size[0] * self.grid_size[1]
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=patch_size, stride=patch_size)


class VTransformer(nn.Module):
    """ViT classifier (models.py:147-177).  The reference fixes 32x32 images
    with 4x4 patches; image and patch size are parameters here."""
    family = "vit"

    def __init__(self, nclasses, seqlen, emsize=2048, nheads=4, nhid=2048, dropout=0.2, nlayers=2,
                 segmentation=True, img_size=(32, 32), patch_size=(4, 4)):
        super().__init__()
        self.nclasses, self.seqlen, self.emsize, self.nheads, self.nhid = nclasses, seqlen, emsize, nheads, nhid
        self.dropout_p = dropout
        self.patch_embed = PatchEmbed(img_size, patch_size, embed_dim=emsize)
        assert seqlen == self.patch_embed.num_patches
        self.cls_token = nn.Parameter(torch.zeros(1, 1, emsize))
        self.pos_embed = nn.Parameter(torch.zeros(1, seqlen + 1, emsize))
        self.layers = nn.ModuleList([_encoder_layer(emsize, nheads, nhid, dropout) for _ in range(nlayers)])
        self.decoder = nn.Linear(emsize, nclasses)
        self.segmentation = segmentation


def init_normal_(model: nn.Module, std: float = 0.02, seed: Optional[int] = None) -> nn.Module:
    """Weights ~ N(0, std), biases 0, LayerNorm affine left at (1, 0)."""
    gen = torch.Generator().manual_seed(seed) if seed is not None else None
    with torch.no_grad():
        for name, p in model.named_parameters():
            if ".norm" in name:
                continue
            if name.endswith("bias"):
                p.zero_()
            else:
                p.copy_(torch.randn(p.shape, generator=gen) * std)
    return model
