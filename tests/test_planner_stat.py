"""Shape rules, FLOP count (hap.stat, /root/reference/hap.rs:190-209) and plan cost of hap_amd.planner.

The shape rules are pinned by the shapes the oracle's joint CPU run actually produces for every node of every
rank's program; the FLOP count by closed-form totals written out per architecture from the reference's per-op
formulas (not by re-running the counter's own rules)."""
import math

import pytest
import torch

import hap_amd
from hap_amd import models, planner
from tests import helpers
from tests.helpers import RATIOS4, RATIOS_E


def _shapes_of(v):
    if isinstance(v, (tuple, list)) and (len(v) == 0 or isinstance(v[0], torch.Tensor)):
        return [tuple(t.shape) for t in v]
    return tuple(v.shape)


CASES = {
    "lm_column": dict(make=lambda: helpers.make_lm(), ratios=RATIOS4, B=16, kw=dict(ffn="column"), batch="lm"),
    "lm_batch": dict(make=lambda: helpers.make_lm(causal=False), ratios=RATIOS4, B=11, kw=dict(ffn="batch"), batch="lm"),
    "lm_zero": dict(make=lambda: helpers.make_lm(), ratios=RATIOS4, B=16, kw=dict(ffn="column", zero=True), batch="lm"),
    "lm_heads": dict(make=lambda: helpers.make_lm(H=8), ratios=RATIOS4, B=16, kw=dict(ffn="batch", attn="heads"), batch="lm"),
    "vit": dict(make=lambda: helpers.make_vit(), ratios=RATIOS4, B=8, kw=dict(ffn="column"), batch="vit"),
    "vit_weight_split_patches": dict(make=lambda: helpers.make_vit(), ratios=RATIOS4, B=8,
                                     kw=dict(ffn="batch", patch_embed="features", decoder="vocabulary"), batch="vit"),
    "lm_vocabulary_decoder": dict(make=lambda: helpers.make_lm(), ratios=RATIOS4, B=16, kw=dict(ffn="column", decoder="vocabulary"), batch="lm"),
    "moe": dict(make=lambda: helpers.make_moe(), ratios=RATIOS_E, B=8, kw=dict(ffn="batch"), batch="lm"),
    "moe_capacity": dict(make=lambda: helpers.make_moe(C=10), ratios=RATIOS_E, B=8, kw=dict(ffn="batch", moe="capacity"), batch="lm"),
    "moe_hidden": dict(make=lambda: helpers.make_moe(C=10), ratios=RATIOS_E, B=8, kw=dict(ffn="batch", moe="hidden"), batch="lm"),
    "moe_model": dict(make=lambda: helpers.make_moe(C=10), ratios=RATIOS_E, B=8, kw=dict(ffn="batch", moe="model"), batch="lm"),
    "moe_sequence": dict(make=lambda: helpers.make_moe(C=10), ratios=RATIOS_E, B=8, kw=dict(ffn="batch", moe="sequence"), batch="lm"),
    "lm_sequence": dict(make=lambda: helpers.make_lm(), ratios=RATIOS4, B=4, kw=dict(ffn="batch", shard_dim="sequence"), batch="lm"),
    "lm_feature_embedding": dict(make=lambda: helpers.make_lm(), ratios=RATIOS4, B=8, kw=dict(ffn="column", embedding="features"), batch="lm"),
    "moe_whole_batch": dict(make=lambda: helpers.make_moe(), ratios=RATIOS_E, B=4,
                            kw=dict(ffn="batch", batch_sharded=False), batch="lm"),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_shape_rules_equal_the_shapes_a_cpu_run_produces(name):
    c = CASES[name]
    model = c["make"]()
    if c["batch"] == "lm":
        x, y = helpers.lm_batch(c["B"], model.seqlen, model.ntokens)
    else:
        x, y = helpers.vit_batch(c["B"], model.patch_embed.img_size[0], model.nclasses)
    run = helpers.joint_cpu(model, c["ratios"], c["B"], **c["kw"])
    run.forward(x, y)
    input_shape = {"x": tuple(x.shape), "y": tuple(y.shape)}
    for r, gm in enumerate(run.programs):
        inferred = planner.infer_shapes(gm, input_shape)
        checked = 0
        for node in gm.graph.nodes:
            if node.op == "output":
                continue
            got = inferred[node.name]
            want = _shapes_of(run.env[r][node.name])
            assert (list(got) if isinstance(want, list) else got) == want, (name, r, node.name, node.target)
            checked += 1
        assert checked > 20


def _lm_forward_flops(B, S, d, F, V, layers):
    """Single-device RTransformer by the reference's formulas, op by op."""
    n = B * S
    attn_block = (n * d                                  # transpose in                     hap.rs:1216
                  + 3 * S * B * d * S + 5 * S * S * B + 3 * S * B * d * S       # attention hap.rs:1330-1337
                  + n * d                                # transpose out
                  + 3 * n * d                            # dropout                          hap.rs:1467
                  + n * d                                # residual add                     hap.rs:1518
                  + 10 * n * d)                          # layer norm                       hap.rs:1656
    ffn_block = (3 * n * d * F                           # linear1                          hap.rs:1038
                 + 3 * n * F + 3 * n * F                 # relu, dropout                    hap.rs:1420, 1467
                 + 3 * n * F * d                         # linear2
                 + 3 * n * d + n * d + 10 * n * d)       # dropout, add, layer norm
    head = (n                                            # embedding                        hap.rs:2044
            + n * d + n * d)                             # scale, add positional encoding   hap.rs:1566, 1518
    tail = (3 * n * d * V                                # decoder
            + 15 * n * V                                 # log_softmax                      hap.rs:1832
            + n * V                                      # transpose
            + n * V)                                     # nll_loss: product of the input   hap.rs:1884
    return head + layers * (attn_block + ffn_block) + tail


def _one_device(model, B, **kw):
    plan = hap_amd.ShardingPlan([[1.0]], 0, ffn=kw.pop("ffn", "batch"))
    return hap_amd.build_program(model, plan, B, **kw)


def test_stat_of_the_reference_lm_configuration_is_the_closed_form():
    # config.py of the reference: 2 layers would take seconds; this is the same architecture at test size
    B, S, d, H, Fh, V, layers = 6, 16, 32, 4, 64, 97, 3
    gm = _one_device(helpers.make_lm(vocab=V, S=S, d=d, H=H, F=Fh, layers=layers), B)
    shapes = {"x": (B, S), "y": (B, S)}
    want = _lm_forward_flops(B, S, d, Fh, V, layers)
    assert planner.flops(gm, shapes) == want
    assert planner.stat(gm, {"input_shape": shapes}) == 3.0 * want


def test_stat_at_bert_large_size_without_allocating_the_model():
    B, S, d, H, Fh, V, layers = 32, 512, 1024, 16, 4096, 30522, 24
    with torch.device("meta"):
        model = models.RTransformer(V, S, d, H, Fh, 0.1, nlayers=layers, causal=False)
    gm = _one_device(model, B, activation="gelu")
    want = _lm_forward_flops(B, S, d, Fh, V, layers)
    assert planner.stat(gm, {"input_shape": {"x": (B, S), "y": (B, S)}}) == 3.0 * want
    # the count is dominated by the GEMMs' 3*m*n*k (the reference prices a multiply-add pair as 3)
    gemm = 3 * B * S * (layers * 2 * d * Fh + d * V)
    assert 0.75 < gemm / want < 1.0


def test_flops_of_vit_and_moe_ops():
    # ViT: conv2d 3*out_channels*prod(input) (hap.rs:1727), flatten/transpose prod, cls ops b*d (hap.rs:2096, 2144)
    B, img, patch, d, Fh, classes, layers = 5, 16, 4, 32, 64, 10, 1
    n_patch = (img // patch) ** 2
    S = n_patch + 1
    gm = _one_device(helpers.make_vit(classes, img, patch, d, 4, Fh, layers), B)
    n = B * S
    stem = (3 * d * B * 3 * img * img + B * d * n_patch + B * d * n_patch + B * d + B * S * d)
    block = (n * d + 6 * S * B * d * S + 5 * S * S * B + n * d + 3 * n * d + n * d + 10 * n * d
             + 3 * n * d * Fh + 6 * n * Fh + 3 * n * Fh * d + 3 * n * d + n * d + 10 * n * d)
    tail = B * d + 3 * B * d * classes + 15 * B * classes + B * classes
    assert planner.flops(gm, {"x": (B, 3, img, img), "y": (B,)}) == stem + layers * block + tail

    # MoE layer: gating 10*prod(tokens) (hap.rs:2206) and the four einsums (hap.rs:2283-2286)
    B, S, d, Fh, E, C, V = 4, 16, 32, 48, 8, 6, 61
    gm = _one_device(helpers.make_moe(V, S, d, 4, Fh, E, C, layers=2), B)
    n = B * S
    attn = n * d + 6 * S * B * d * S + 5 * S * S * B + n * d + 3 * n * d + n * d + 10 * n * d
    dense = 3 * n * d * Fh + 6 * n * Fh + 3 * n * Fh * d + 3 * n * d + n * d + 10 * n * d
    moe = (10 * n * d
           + 3 * B * S * d * E * C                       # bsd,bsec->becd
           + 3 * E * d * Fh * B * C                      # edh,becd->bech
           + 3 * B * E * C * Fh                          # relu
           + 3 * E * Fh * d * B * C                      # ehd,bech->becd
           + 3 * B * E * C * d * S                       # becd,bsec->bsd
           + n * d + 10 * n * d)
    want = (n + 2 * n * d) + 2 * attn + dense + moe + 3 * n * d * V + 15 * n * V + 2 * n * V
    assert planner.flops(gm, {"x": (B, S), "y": (B, S)}) == want


def test_sharded_programs_split_the_batch_proportional_work():
    """Pure data parallelism: every op is linear in the batch, so the ranks' counts add up to the one-device count."""
    B, ratios = 16, RATIOS4
    model = helpers.make_lm(causal=False)
    shapes = {"x": (B, model.seqlen), "y": (B, model.seqlen)}
    whole = planner.flops(_one_device(helpers.make_lm(causal=False), B), shapes)
    parts = [planner.flops(gm, shapes) for gm in helpers.rank_programs(model, ratios, B, ffn="batch")]
    assert sum(parts) == whole
    assert parts[0] == parts[1] == 3 * parts[2]          # 6 : 6 : 2 : 2 rows


def test_communication_counts_follow_the_profile_closures():
    B, ratios = 16, RATIOS4
    model = helpers.make_lm(layers=1)
    S, d, Fh = model.seqlen, model.emsize, model.nhid
    shapes = {"x": (B, S), "y": (B, S)}
    gm = helpers.rank_programs(model, ratios, B, ffn="column")[0]          # rank 0 owns 6 rows, 24 FFN columns
    tr = planner.communication(gm, shapes, 4)
    gathered = 6 * S * d * 4                                              # local shard x n_devices (hap.rs:2648-2650)
    exchanged = B * S * 24 * 4                                            # all_to_all input [B, S, F_local] (hap.rs:2737)
    assert tr.all_gather == gathered and tr.reduce_scatter == gathered
    assert tr.all_to_all == 2 * exchanged
    replicated = sum(p.numel() for n, p in gm.named_parameters() if "linear1" not in n) + model.src_mask.numel()
    assert tr.all_reduce == replicated                                    # gradient all_reduce (hap.rs:2572-2574)


def test_cost_prefers_proportional_ratios_on_uneven_devices_and_counts_the_exchange():
    B = 16

    def factory():
        with torch.device("meta"):
            return models.RTransformer(97, 16, 32, 4, 64, 0.0, nlayers=2, causal=False)

    shapes = {"x": (B, 16), "y": (B, 16)}
    fast_links = planner.ClusterInfo([3e9, 3e9, 1e9, 1e9], 1e15, 1e15, 1e15, 1e15)
    ranked = planner.choose_plan(factory, B, shapes, fast_links, forms=("batch",))
    assert [round(r, 3) for r in ranked[0].ratios] == [.375, .375, .125, .125]
    assert ranked[0].total < ranked[1].total
    # proportional split: every device computes for the same time; uniform: the slow devices take 2x the mean
    comp = [c for c, _ in ranked[0].per_device]
    assert max(comp) / min(comp) < 1.01
    uniform = ranked[1]
    assert uniform.computation == pytest.approx(uniform.per_device[2][0])
    assert uniform.per_device[2][0] == pytest.approx(3 * uniform.per_device[0][0])

    # with slow links the column plan's gathers and exchange make it dearer than pure data parallelism
    slow_links = planner.ClusterInfo([1e9] * 4, 1e6, 1e6, 1e6, 1e6)
    ranked = planner.choose_plan(factory, B, shapes, slow_links, forms=("batch", "column"))
    assert ranked[0].ffn == "batch" and ranked[-1].ffn == "column"
    assert ranked[-1].communication > ranked[0].communication


def test_calibration_divides_the_count_by_one_timed_step():
    calls = []
    clock = iter([10.0, 10.5])
    orig = planner.time.time
    planner.time.time = lambda: next(clock)
    try:
        got = planner.calibrate_device_flops(lambda: calls.append(1), 3e9, lambda: calls.append("sync"))
    finally:
        planner.time.time = orig
    assert got == math.floor(3e9 / 0.5)
    assert calls == [1] * 11 + ["sync", 1, "sync"]                        # profiler.py:21-31
