"""Shared builders for the parity tests: configurations, seeded inputs, the CPU joint run."""
import copy

import torch

import hap_amd
from hap_amd import models
from oracle.cpu_executor import JointCPURun

RATIOS4 = [.375, .375, .125, .125]
RATIOS_E = [.3125, .3125, .1875, .1875]


def make_lm(vocab=97, S=16, d=32, H=4, F=64, layers=2, causal=True, seed=0):
    torch.manual_seed(seed)
    m = models.RTransformer(vocab, S, d, H, F, 0.0, nlayers=layers, causal=causal)
    return models.init_normal_(m, 0.02, seed)


def make_moe(vocab=61, S=16, d=32, H=4, F=48, E=8, C=6, layers=2, seed=0, std=0.5):
    torch.manual_seed(seed)
    m = models.RMoE(vocab, S, d, H, F, 0.0, E, C, layers)
    return models.init_normal_(m, std, seed)


def make_switch(vocab=61, S=16, d=32, H=4, F=48, E=8, C=6, layers=2, seed=0, std=0.5):
    torch.manual_seed(seed)
    m = models.RSwitch(vocab, S, d, H, F, 0.0, E, C, layers)
    return models.init_normal_(m, std, seed)


def make_vit(classes=10, img=16, patch=4, d=32, H=4, F=64, layers=2, seed=0):
    torch.manual_seed(seed)
    n = (img // patch) ** 2
    m = models.VTransformer(classes, n, d, H, F, 0.0, nlayers=layers, img_size=(img, img), patch_size=(patch, patch))
    return models.init_normal_(m, 0.02, seed)


def lm_batch(B, S, vocab, seed=1, mlm=False):
    g = torch.Generator().manual_seed(seed)
    if mlm:
        x = torch.randint(0, vocab, (B, S), generator=g)
        masked = torch.rand(B, S, generator=g) < 0.15
        y = torch.where(masked, x, torch.full_like(x, -100))
        return x, y
    ids = torch.randint(0, vocab, (B, S + 1), generator=g)
    return ids[:, :-1].contiguous(), ids[:, 1:].contiguous()


def vit_batch(B, img, classes, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, 3, img, img, generator=g), torch.randint(0, classes, (B,), generator=g)


def rank_programs(model, ratios, B, **kw):
    """One sliced copy of the model + its program per rank."""
    progs = []
    for r in range(len(ratios)):
        m = copy.deepcopy(model)
        plan = hap_amd.ShardingPlan([list(ratios)], r, ffn=kw.get("ffn", "column"), zero=kw.get("zero", False),
                                     attn=kw.get("attn", "batch"), shard_dim=kw.get("shard_dim", "batch"),
                                     embedding=kw.get("embedding", "rows"), moe=kw.get("moe", "experts"),
                                     decoder=kw.get("decoder", "whole"), patch_embed=kw.get("patch_embed", "batch"))
        progs.append(hap_amd.build_program(m, plan, B, activation=kw.get("activation", "relu"),
                                           batch_sharded=kw.get("batch_sharded", True)))
    return progs


def joint_cpu(model, ratios, B, dtype="fp32", **kw):
    return JointCPURun(rank_programs(model, ratios, B, **kw), dtype)


def rel_err(a, b):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def gating_vectors():
    """The hand-worked routing vectors of tests/golden/gating_vectors.json: the same data for the CPU oracle tests and
    the GPU kernel tests."""
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "gating_vectors.json")) as f:
        return json.load(f)


def gating_vector_logits(v):
    """Logits [1, S, E] whose first (and second) choices are the vector's."""
    import torch
    lg = torch.full((1, v["S"], v["E"]), v["other_logit"])
    for s, ch in enumerate(v["choices"]):
        if isinstance(ch, list):
            lg[0, s, ch[0]], lg[0, s, ch[1]] = v["first_logit"], v["second_logit"]
        else:
            lg[0, s, ch] = v["first_logit"]
    return lg
