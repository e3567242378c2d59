"""Single-device forward of the model families, built from stock torch.nn
modules.  TEST INFRASTRUCTURE ONLY.

Used for the invariant that pins the program generator: the sum over ranks of
the per-rank partial losses of the SPMD program equals the loss of the
unsharded model (/root/reference/models.py:78-88 RTransformer.forward,
108-118 RMoE.forward, 137-145 RSwitch.forward, 163-177 VTransformer.forward, 340-366 the top-2 layer,
405-434 the switch layer).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

import hap_amd.models as product_models
from . import ops as ref


def _top2_layer(layer, x, mask):
    a = layer.self_attn(x, x, x, attn_mask=mask, need_weights=False)[0]            # models.py:346-351
    x = layer.norm1(x + a)                                                         # :341
    # the switch layer (models.py:405-434) differs from the top-2 layer in the gating call only (:421 / :354)
    gating = ref.switch_gating if isinstance(layer, product_models.SwitchTransformerEncoderLayer) else ref.top_2_gating
    dispatch, combine = gating(x, layer.n_expert, layer.capacity, layer.gate_weight)
    t = torch.einsum("bsd,bsec->becd", x, dispatch)                                # :356
    t = torch.relu(torch.einsum("edh,becd->bech", layer.w1, t))                    # :358-360
    t = torch.einsum("ehd,bech->becd", layer.w2, t)                                # :362
    return layer.norm2(x + torch.einsum("becd,bsec->bsd", t, combine))             # :364, :342


def forward(model, x, y):
    if model.family == "lm":
        h = model.encoder(x) * math.sqrt(model.emsize)
        h = h + model.pe
        mask = getattr(model, "src_mask", None)
    else:
        h = model.patch_embed.proj(x)
        h = torch.flatten(h, 2).transpose(1, 2)
        h = torch.cat((model.cls_token.expand(h.shape[0], -1, -1), h), dim=1)
        h = h + model.pos_embed
        mask = None
    for layer in model.layers:
        if isinstance(layer, product_models.Top2TransformerEncoderLayer):
            h = _top2_layer(layer, h, mask)
        else:
            h = layer(h, mask)
    if model.family == "lm":
        lp = torch.log_softmax(model.decoder(h), dim=-1)
        return F.nll_loss(lp.transpose(1, 2), y, reduction="sum")
    lp = torch.log_softmax(model.decoder(h[:, 0, :]), dim=-1)
    return F.nll_loss(lp, y, reduction="sum")
