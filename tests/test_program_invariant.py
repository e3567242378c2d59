"""Pins the program generator: the sum over ranks of the per-rank partial losses and gradients of the SPMD
program equals the unsharded model built from stock torch.nn (models.py:65-88, 90-118, 147-177, 301-366),
all on the CPU in float32."""
import copy

import pytest
import torch
import torch.nn.functional as F

from helpers import (RATIOS4, RATIOS_E, joint_cpu, lm_batch, make_lm, make_moe, make_switch, make_vit, rel_err,
                     vit_batch)
from oracle import single_device
import hap_amd
from hap_amd import collectives, models


def _single(model, x, y):
    m = copy.deepcopy(model)
    m.train()
    loss = single_device.forward(m, x, y)
    loss.backward()
    return loss.detach(), dict(m.named_parameters())


def _check(model, run, x, y, sharded, whole_norm=False):
    loss1, p1 = _single(model, x, y)
    losses = run.step(x, y)
    torch.testing.assert_close(sum(l.double() for l in losses).float(), loss1, rtol=1e-5, atol=1e-5)
    W = run.W
    for name, ref_p in p1.items():
        if ref_p.grad is None:
            continue
        held = [dict(p.named_parameters()).get(name) for p in run.programs]
        if any(h is None or h.grad is None for h in held):
            assert ".norm" in name, name       # LayerNorm affine parameters are never read by the program
            continue
        grads = [h.grad for h in held]
        if name in sharded:
            dim, L = sharded[name][:2]
            if dim == "heads":                 # q, k, v rows of each rank's heads of a packed in-projection
                hd = sharded[name][2]
                blocks = ref_p.grad.view(3, sum(L), hd, *ref_p.grad.shape[1:])
                want = [b.reshape(3 * l * hd, *ref_p.grad.shape[1:]) for b, l in zip(torch.split(blocks, L, 1), L)]
            else:
                want = torch.split(ref_p.grad, L, dim)
            for r in range(W):
                if whole_norm:
                    # a shard may hold only rows whose true gradient is zero (the key bias of softmax attention):
                    # its error is measured against the whole parameter's gradient
                    assert (grads[r] - want[r]).norm() < 2e-5 * ref_p.grad.norm(), (name, r)
                else:
                    assert rel_err(grads[r], want[r]) < 2e-5, (name, r)
        else:
            for r in range(W):                 # replicate.backward all-reduces: every rank holds the full gradient
                assert rel_err(grads[r], ref_p.grad) < 2e-5, (name, r)


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_lm_spmd_equals_single_device(ffn):
    model = make_lm()
    B = 8
    x, y = lm_batch(B, 16, 97)
    run = joint_cpu(model, RATIOS4, B, ffn=ffn)
    L_F = hap_amd.sharding_lengths(64, RATIOS4)
    sharded = {}
    if ffn == "column":
        for i in range(2):
            sharded[f"layers.{i}.linear1.weight"] = (0, L_F)
            sharded[f"layers.{i}.linear1.bias"] = (0, L_F)
    _check(model, run, x, y, sharded)


def test_mlm_targets_with_ignore_index():
    model = make_lm(causal=False)
    x, y = lm_batch(8, 16, 97, mlm=True)
    _check(model, joint_cpu(model, RATIOS4, 8), x, y, {
        f"layers.{i}.linear1.{k}": (0, hap_amd.sharding_lengths(64, RATIOS4)) for i in range(2) for k in ("weight", "bias")})


def test_vit_spmd_equals_single_device():
    model = make_vit()
    x, y = vit_batch(8, 16, 10)
    _check(model, joint_cpu(model, RATIOS4, 8, ffn="batch"), x, y, {})


@pytest.mark.parametrize("batch_sharded", [True, False])
def test_moe_spmd_equals_single_device(batch_sharded):
    model = make_moe()
    B = 16 if batch_sharded else 4
    x, y = lm_batch(B, 16, 61)
    L_E = hap_amd.sharding_lengths(8, RATIOS_E)
    run = joint_cpu(model, RATIOS_E, B, ffn="batch", batch_sharded=batch_sharded)
    sharded = {"layers.1.w1": (0, L_E), "layers.1.w2": (0, L_E)}
    if not batch_sharded:
        # every rank computes the whole batch: the W partial losses are W copies of the full loss
        loss1, _ = _single(model, x, y)
        losses = run.forward(x, y)
        for l in losses:
            torch.testing.assert_close(l, loss1, rtol=1e-5, atol=1e-5)
        return
    _check(model, run, x, y, sharded)


def _zero_sharded(model, ratios, already=()):
    """Under the ZeRO form every parameter with a leading dimension other than 1 is a dim-0 shard (hap.rs:2527-2547)."""
    out = {}
    for name, p in model.named_parameters():
        if name not in already and p.shape[0] != 1:
            out[name] = (0, hap_amd.sharding_lengths(p.shape[0], ratios))
    return out


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_zero_lm_spmd_equals_single_device(ffn):
    model = make_lm()
    B = 8
    x, y = lm_batch(B, 16, 97)
    run = joint_cpu(model, RATIOS4, B, ffn=ffn, zero=True)
    # the shards are what the program's modules hold: 97 vocabulary rows over 4 ranks, 96 in_proj rows, ...
    held = dict(run.programs[2].named_parameters())
    assert held["encoder.weight"].shape[0] == hap_amd.sharding_lengths(97, RATIOS4)[2]
    assert held["layers.0.self_attn.in_proj_weight"].shape == (12, 32)
    assert run.programs[2].src_mask.shape == (2, 16)
    _check(model, run, x, y, _zero_sharded(model, RATIOS4), whole_norm=True)


def test_zero_vit_and_moe_spmd_equal_single_device():
    model = make_vit()
    x, y = vit_batch(8, 16, 10)
    run = joint_cpu(model, RATIOS4, 8, ffn="batch", zero=True)
    assert dict(run.programs[0].named_parameters())["pos_embed"].shape == (1, 17, 32)      # leading 1: left whole
    _check(model, run, x, y, _zero_sharded(model, RATIOS4), whole_norm=True)

    model = make_moe()
    x, y = lm_batch(16, 16, 61)
    run = joint_cpu(model, RATIOS_E, 16, ffn="batch", zero=True)
    _check(model, run, x, y, _zero_sharded(model, RATIOS_E), whole_norm=True)


@pytest.mark.parametrize("zero", [False, True])
def test_switch_moe_spmd_equals_single_device(zero):
    """RSwitch (models.py:120-145): the top-2 plan forms with switch gating."""
    model = make_switch()
    x, y = lm_batch(16, 16, 61)
    L_E = hap_amd.sharding_lengths(8, RATIOS_E)
    run = joint_cpu(model, RATIOS_E, 16, ffn="batch", zero=zero)
    assert sum(n.target is hap_amd.models.switch_gating for n in run.programs[0].graph.nodes) == 1
    sharded = _zero_sharded(model, RATIOS_E) if zero else {"layers.1.w1": (0, L_E), "layers.1.w2": (0, L_E)}
    _check(model, run, x, y, sharded, whole_norm=zero)


def _head_sharded(layers, L_H, hd):
    out = {}
    for i in range(layers):
        out[f"layers.{i}.self_attn.in_proj_weight"] = ("heads", L_H, hd)
        out[f"layers.{i}.self_attn.in_proj_bias"] = ("heads", L_H, hd)
        out[f"layers.{i}.self_attn.out_proj.weight"] = (1, [l * hd for l in L_H])
    return out


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_head_parallel_attention_lm_spmd_equals_single_device(ffn):
    """8 heads over ratios .375/.375/.125/.125 -> 3, 3, 1, 1 heads per device."""
    model = make_lm(H=8)
    B = 8
    x, y = lm_batch(B, 16, 97)
    run = joint_cpu(model, RATIOS4, B, ffn=ffn, attn="heads")
    L_H = hap_amd.sharding_lengths(8, RATIOS4)
    assert L_H == [3, 3, 1, 1]
    held = dict(run.programs[2].named_parameters())
    assert held["layers.0.self_attn.in_proj_weight"].shape == (3 * 1 * 4, 32)
    assert held["layers.0.self_attn.out_proj.weight"].shape == (32, 4)
    sharded = _head_sharded(2, L_H, 4)
    if ffn == "column":
        L_F = hap_amd.sharding_lengths(64, RATIOS4)
        for i in range(2):
            sharded[f"layers.{i}.linear1.weight"] = (0, L_F)
            sharded[f"layers.{i}.linear1.bias"] = (0, L_F)
    _check(model, run, x, y, sharded, whole_norm=True)


def test_head_parallel_attention_vit_with_zero_spmd_equals_single_device():
    model = make_vit(H=4)
    x, y = vit_batch(8, 16, 10)
    run = joint_cpu(model, [.25, .25, .25, .25], 8, ffn="batch", attn="heads", zero=True)
    sharded = _zero_sharded(model, [.25] * 4)
    sharded.update(_head_sharded(2, [1, 1, 1, 1], 8))
    _check(model, run, x, y, sharded, whole_norm=True)


@pytest.mark.parametrize("embedding", ["rows", "features"])
def test_sequence_sharded_lm_spmd_equals_single_device(embedding):
    """shard_dim='sequence': 19 positions over .375/.375/.125/.125 -> 7, 7, 2, 3 per device."""
    model = make_lm(S=19, d=40 if embedding == "features" else 32)
    x, y = lm_batch(6, 19, 97)
    run = joint_cpu(model, RATIOS4, 6, ffn="batch", shard_dim="sequence", embedding=embedding)
    assert hap_amd.sharding_lengths(19, RATIOS4) == [7, 7, 2, 3]
    assert run.programs[2].pe.shape == (1, 2, 40 if embedding == "features" else 32)
    sharded = {"encoder.weight": (1, hap_amd.sharding_lengths(40, RATIOS4))} if embedding == "features" else {}
    _check(model, run, x, y, sharded)


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_feature_sharded_embedding_table_spmd_equals_single_device(ffn):
    model = make_lm(d=40, H=4)
    x, y = lm_batch(8, 16, 97)
    run = joint_cpu(model, RATIOS4, 8, ffn=ffn, embedding="features")
    L_d = hap_amd.sharding_lengths(40, RATIOS4)
    assert L_d == [15, 15, 5, 5] and run.programs[3].encoder.weight.shape == (97, 5)
    sharded = {"encoder.weight": (1, L_d)}
    if ffn == "column":
        L_F = hap_amd.sharding_lengths(64, RATIOS4)
        for i in range(2):
            sharded[f"layers.{i}.linear1.weight"] = (0, L_F)
            sharded[f"layers.{i}.linear1.bias"] = (0, L_F)
    _check(model, run, x, y, sharded)


@pytest.mark.parametrize("moe", ["capacity", "hidden", "model", "sequence"])
def test_moe_capacity_and_hidden_splits_spmd_equal_single_device(moe):
    """The other legal splits of the four MoE einsums (hap.rs:3285-3419): every device takes a range of every
    expert's capacity slots with whole expert weights, or every device holds a slice of the experts' hidden
    features, or of the tokens' model dimension (columns 10 / 10 / 6 / 6 of 32), or the tokens of a range of positions
    (5 / 5 / 3 / 3 of 16); batch-sharded attention around them as in the expert split."""
    model = make_moe(C=10, F=48)                                # capacity slots 3 / 3 / 2 / 2, hidden widths 15 / 15 / 9 / 9
    B = 16
    x, y = lm_batch(B, 16, 61)
    run = joint_cpu(model, RATIOS_E, B, ffn="batch", moe=moe)
    sharded = {}
    if moe == "hidden":
        L_F = hap_amd.sharding_lengths(48, RATIOS_E)
        sharded = {"layers.1.w1": (2, L_F), "layers.1.w2": (1, L_F)}
    if moe == "model":
        L_D = hap_amd.sharding_lengths(32, RATIOS_E)
        sharded = {"layers.1.w1": (1, L_D), "layers.1.w2": (2, L_D)}
    _check(model, run, x, y, sharded)


def test_moe_hidden_split_with_deferred_reduction_in_bf16():
    """The hidden-feature split feeds the partial sums of the second expert product straight into the combine einsum
    and reduces the combined [B, S, d] tensor instead of the [B, E, C, d] one (a deliberate, linearity-based departure
    from the reference's triples, which would all_reduce in front of the combine: hap.rs:3369-3373, 3385-3415).  In
    bf16 the order of rounding and summation differs from a reference-legal form.  At this size a bf16 run differs
    from the float32 single-device model mostly through flipped routing and relu decisions, whatever the plan; so the
    deferred form is held to the bf16 tolerance on the loss and, on the expert weights' gradients, to the error that
    the reference-legal expert split shows in the same arithmetic."""
    model = make_moe(C=10, F=48)
    B = 16
    x, y = lm_batch(B, 16, 61)
    loss1, p1 = _single(model, x, y)

    def gradient_errors(moe, dims):
        run = joint_cpu(model, RATIOS_E, B, dtype="bf16", ffn="batch", moe=moe)
        total = sum(l.double() for l in run.step(x, y)).item()
        assert abs(total - loss1.item()) <= 2e-2 * abs(loss1.item()), moe
        errs = {}
        for name, dim in dims.items():
            whole = torch.cat([dict(p.named_parameters())[name].grad.float() for p in run.programs], dim)
            errs[name] = rel_err(whole, p1[name].grad)
        return errs

    legal = gradient_errors("experts", {"layers.1.w1": 0, "layers.1.w2": 0})
    deferred = gradient_errors("hidden", {"layers.1.w1": 2, "layers.1.w2": 1})
    for name in legal:
        assert deferred[name] <= 1.25 * legal[name] + 2e-2, (name, deferred[name], legal[name])


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_lm_vocabulary_split_decoder_spmd_equals_single_device(ffn):
    """The feature partition of a linear (hap.rs:2807-2816) applied to the output projection: decoder weight and bias
    sliced over the vocabulary (36 / 37 / 12 / 12 of 97), activations gathered over the batch, every rank's columns
    of the logits exchanged by one all_to_all into whole rows of its own samples (hap.rs:2713-2744), log_softmax and
    nll_loss on those."""
    model = make_lm()
    B = 8
    x, y = lm_batch(B, 16, 97)
    run = joint_cpu(model, RATIOS4, B, ffn=ffn, decoder="vocabulary")
    L_V = hap_amd.sharding_lengths(97, RATIOS4)
    # floors 36, 36, 12, 12 leave one unit: the largest deficit .375 - 36/97 is shared by ranks 0 and 1, the tie goes to the last
    assert L_V == [36, 37, 12, 12]
    sharded = {"decoder.weight": (0, L_V), "decoder.bias": (0, L_V)}
    if ffn == "column":
        L_F = hap_amd.sharding_lengths(64, RATIOS4)
        for i in range(2):
            sharded[f"layers.{i}.linear1.weight"] = (0, L_F)
            sharded[f"layers.{i}.linear1.bias"] = (0, L_F)
    _check(model, run, x, y, sharded)
    targets = [n.target for n in run.programs[0].graph.nodes if n.op == "call_function" and n.target is not collectives.replicate]
    assert targets[-4:] == [collectives.all_to_all, torch.log_softmax, torch.transpose, F.nll_loss]


@pytest.mark.parametrize("decoder", ["whole", "vocabulary"])
def test_vit_weight_split_patch_embedding_spmd_equals_single_device(decoder):
    """The convolution's weight-split triple (hap.rs:3083-3087): kernel and bias sliced over the 32 output channels
    (12 / 12 / 4 / 4), whole images in, output gathered on dim 1; the flattened output is all_gather-ed on dim 1, the
    class token is appended on the whole batch and the rows are then cut to the rank's images.  With the class head
    split over the 10 classes as well (4 / 4 / 1 / 1)."""
    model = make_vit()
    x, y = vit_batch(8, 16, 10)
    run = joint_cpu(model, RATIOS4, 8, ffn="batch", patch_embed="features", decoder=decoder)
    L_d = hap_amd.sharding_lengths(32, RATIOS4)
    sharded = {"patch_embed.proj.weight": (0, L_d), "patch_embed.proj.bias": (0, L_d)}
    if decoder == "vocabulary":
        L_C = hap_amd.sharding_lengths(10, RATIOS4)
        sharded.update({"decoder.weight": (0, L_C), "decoder.bias": (0, L_C)})
    _check(model, run, x, y, sharded)
    nodes = [n for n in run.programs[0].graph.nodes if n.op == "call_function" and n.target is not collectives.replicate]
    conv = next(n for n in nodes if n.target is F.conv2d)
    assert conv.args[0].op == "placeholder"                       # whole images
    follow = [n.target for n in nodes[nodes.index(conv) + 1: nodes.index(conv) + 6]]
    assert follow == [torch.flatten, collectives.all_gather, torch.transpose, models.append_cls_token,
                      collectives.dynamic_slice]
