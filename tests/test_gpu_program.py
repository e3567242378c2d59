"""End-to-end parity of the compiled shard program on the GPU against stock-PyTorch CPU execution of the same
generated graph (all ranks on the CPU; the GPU runs one rank with the peers' messages replayed).
Loss, every parameter gradient and the updated parameters are compared:
float32: rtol 1e-4 (norm-wise and element-wise with atol = rtol * max|ref|);
bfloat16: rtol 2e-2 norm-wise on losses, gradients and updated weights."""
import copy

import pytest
import torch

import hap_amd
from helpers import (RATIOS4, RATIOS_E, joint_cpu, lm_batch, make_lm, make_moe, make_switch, make_vit, rel_err,
                     vit_batch)

pytestmark = pytest.mark.gpu


def _check_sent_messages(ex, log, rank, dtype):
    """What this rank hands to the wire (padded shards, padded pieces, exchange pieces, all_reduce addends) is what
    the recorded run of all ranks sent from this rank: layouts exactly (pads included), values within the
    tolerance of the dtype."""
    torch.cuda.synchronize()
    sent = ex.wire.sent
    tol = 1e-4 if dtype == "fp32" else 2e-2
    checked = 0
    for (tag, direction, dst), buf in sent.items():
        want = log[(tag, direction)][rank][dst].float()
        got = buf.float().cpu()
        assert got.shape == want.shape, (tag, direction, dst)
        finite = torch.isfinite(want)                            # the oracle poisons pads with NaN
        assert torch.isfinite(got[finite]).all(), (tag, direction, dst)
        if finite.any() and want[finite].abs().max() > 0:
            err = ((got[finite] - want[finite]).norm() / want[finite].norm()).item()
            assert err < tol, (tag, direction, dst, err)
        checked += 1
    assert checked == len(sent)


def _gpu_rank(model, ratios, rank, B, x, y, log, dtype, opt, **kw):
    m = copy.deepcopy(model)
    plan = hap_amd.ShardingPlan([list(ratios)], rank, ffn=kw.get("ffn", "column"), zero=kw.get("zero", False),
                                attn=kw.get("attn", "batch"), shard_dim=kw.get("shard_dim", "batch"),
                                embedding=kw.get("embedding", "rows"), moe=kw.get("moe", "experts"))
    gm = hap_amd.build_program(m, plan, B, activation=kw.get("activation", "relu"),
                               batch_sharded=kw.get("batch_sharded", True))
    ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.ReplayWire(log, rank), rank=rank,
                                 world_size=len(ratios))
    ex.configure_optimizer(**opt)
    loss = ex.forward(x, y)
    ex.backward()
    _check_sent_messages(ex, log, rank, dtype)
    grads = {n: rec["grad"].clone().cpu() for n, rec in ex.params.items()}
    ex.step()
    torch.cuda.synchronize()
    params = {n: rec["master"].clone().cpu() for n, rec in ex.params.items()}
    return loss.item(), grads, params, ex


def _same_bits(a, b, what=("grad",)):
    """Two executors that launch the same kernels on the same data hold the same bits: every reduction of the
    library (split-K sums, bias-gradient row sums, column sums, the embedding gradient, the gradient norm) adds in
    a fixed order, so the order in which blocks run never shows."""
    torch.cuda.synchronize()
    for n, rec in a.params.items():
        for k in what:
            assert torch.equal(rec[k], b.params[n][k]), (n, k, (rec[k] - b.params[n][k]).abs().max().item())


def _compare(model, ratios, B, x, y, dtype, ranks, opt, **kw):
    run = joint_cpu(model, ratios, B, dtype, **kw)
    if opt["kind"] == "sgd":
        optims = [torch.optim.SGD(p.parameters(), lr=opt["lr"]) for p in run.programs]
    else:
        optims = [torch.optim.Adam(p.parameters(), lr=opt["lr"]) for p in run.programs]
    initial = [{n: p.detach().clone() for n, p in prog.named_parameters()} for prog in run.programs]
    losses = run.step(x, y, None)
    ref_grads = [{n: p.grad.clone() for n, p in prog.named_parameters() if p.grad is not None} for prog in run.programs]
    for o in optims:
        o.step()
    tol = 1e-4 if dtype == "fp32" else 2e-2
    ex_initial = {r: [(n, p.detach().clone()) for n, p in initial[r].items()] for r in ranks}
    for r in ranks:
        loss, grads, params, ex = _gpu_rank(model, ratios, r, B, x, y, run.world.log, dtype, opt, **kw)
        want = losses[r].float().item()
        assert abs(loss - want) <= tol * abs(want), (r, loss, want)
        assert set(grads) == set(ref_grads[r]), set(grads) ^ set(ref_grads[r])
        for n, g in grads.items():
            ref = ref_grads[r][n].float()
            assert g.shape == ref.shape, n
            err = rel_err(g, ref)
            assert err < tol, (r, n, err)
            if dtype == "fp32":
                torch.testing.assert_close(g, ref, rtol=tol, atol=tol * ref.abs().max().item())
        ref_params = dict(run.programs[r].named_parameters())
        for n, p in params.items():
            new_ref = ref_params[n].detach()
            if opt["kind"] == "sgd":
                assert rel_err(p, new_ref) < tol, (r, n)
                continue
            # Adam's first step is -lr * sign(g): where the true gradient is zero up to rounding (the key bias
            # of softmax attention, dropped experts) its sign is noise on both sides.  So (a) the update must be
            # torch.optim.Adam's on the GPU's own gradients, and (b) it must agree with the oracle's wherever
            # the oracle's gradient is clearly non-zero.
            old = dict(ex_initial[r])[n]
            twin = old.clone().requires_grad_(True)
            twin.grad = grads[n].clone()
            torch.optim.Adam([twin], lr=opt["lr"]).step()
            torch.testing.assert_close(p, twin.detach(), rtol=1e-5, atol=1e-8)
            g_ref = ref_grads[r][n].float()
            clear = g_ref.abs() > 1e-2 * g_ref.abs().max()
            if clear.any():
                assert rel_err((p - old)[clear], (new_ref - old)[clear]) < max(tol, 1e-3), (r, n)
    return run


SGD = dict(kind="sgd", lr=1e-3)
ADAM = dict(kind="adam", lr=5e-4)


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_lm_fp32_small(cuda, ffn):
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    _compare(model, RATIOS4, 8, x, y, "fp32", [0, 3], SGD, ffn=ffn)


def test_config1_full_size_fp32(cuda):
    """The reference's CPU-runnable configuration at full size: 2-layer post-LN LM, d 512, 8 heads, FFN 2048 -> 768 local, seq 128, 3 of 8, vocab 33280."""
    model = make_lm(vocab=33280, S=128, d=512, H=8, F=2048, layers=2, seed=39)
    x, y = lm_batch(8, 128, 33280, seed=39)
    _compare(model, RATIOS4, 8, x, y, "fp32", [0], SGD)


def test_lm_bf16_mlm_adam(cuda):
    model = make_lm(vocab=1003, S=32, d=64, H=4, F=128, layers=2, causal=False)
    x, y = lm_batch(8, 32, 1003, mlm=True)
    _compare(model, RATIOS4, 8, x, y, "bf16", [0, 2], ADAM)


def test_lm_gelu_fp32(cuda):
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    _compare(model, RATIOS4, 8, x, y, "fp32", [1], SGD, activation="gelu")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_vit(cuda, dtype):
    model = make_vit(img=32, patch=8, d=64, F=128)
    x, y = vit_batch(8, 32, 10)
    _compare(model, RATIOS4, 8, x, y, dtype, [0, 3], ADAM, ffn="batch")


@pytest.mark.parametrize("batch_sharded", [True, False])
def test_moe_fp32(cuda, batch_sharded):
    model = make_moe()
    B = 16 if batch_sharded else 4
    x, y = lm_batch(B, 16, 61)
    _compare(model, RATIOS_E, B, x, y, "fp32", [0, 2], ADAM, ffn="batch", batch_sharded=batch_sharded)


@pytest.mark.parametrize("dtype,batch_sharded", [("fp32", True), ("fp32", False), ("bf16", False)])
def test_switch_moe(cuda, dtype, batch_sharded):
    """RSwitch (models.py:120-145): switch-gated experts, expert-sharded, batch sharded or replicated."""
    model = make_switch() if dtype == "fp32" else make_switch(d=64, F=96, std=0.3)
    B = 16 if batch_sharded else 4
    x, y = lm_batch(B, 16, 61)
    _compare(model, RATIOS_E, B, x, y, dtype, [0, 2], ADAM, ffn="batch", batch_sharded=batch_sharded)


@pytest.mark.parametrize("moe,dtype,batch_sharded", [("capacity", "fp32", True), ("capacity", "fp32", False),
                                                      ("capacity", "bf16", False), ("hidden", "fp32", True),
                                                      ("hidden", "bf16", False), ("model", "fp32", True),
                                                      ("model", "fp32", False), ("sequence", "fp32", True),
                                                      ("sequence", "fp32", False), ("sequence", "bf16", False)])
def test_moe_capacity_and_hidden_splits(cuda, moe, dtype, batch_sharded):
    """The capacity split (dispatch / combine tensors sliced on dim 3, whole expert weights: every device works on
    a range of every expert's slots), the hidden-feature split of the expert FFN and the split of the tokens' model
    dimension (the first expert product is then a partial sum, all-reduced in the program's [B, E, C, H] order),
    and the split along the sequence (tokens and routing windowed over positions 5 / 5 / 3 / 3 of 16, the dispatched
    tokens all-reduced) (hap.rs:3285-3419), uneven over the devices, against the CPU run of all ranks."""
    # hidden widths 40 / 40 / 24 / 24 of 128 (multiples of the 16-byte vector in either type), capacity slots 3 / 3 / 2 / 2
    if moe == "model":      # model widths 20 / 20 / 12 / 12 of 64
        model = make_moe(d=64, C=10)
    else:
        model = make_moe(C=10, F=128) if dtype == "fp32" else make_moe(d=64, F=128, C=10, std=0.3)
    B = 16 if batch_sharded else 4
    x, y = lm_batch(B, 16, 61)
    _compare(model, RATIOS_E, B, x, y, dtype, [0, 2], ADAM, ffn="batch", batch_sharded=batch_sharded, moe=moe)


def test_moe_model_dimension_split_bf16_with_shared_decisions(cuda):
    """The split of the tokens' model dimension in bf16 (widths 40 / 40 / 24 / 24 of 128).  Here routed tensors cross
    the wire (the first expert product is all-reduced), and two bf16 computations of the gate differ on a few
    near-ties, which moves whole rows between slots; so, as in the full-size tests, the GPU's discrete decisions
    (chosen experts, relu masks; routing itself is checked bit for bit on the GPU's float32 logits) are handed to
    the CPU oracle, which then has to give the same loss and gradients."""
    from oracle.cpu_executor import SingleRankCPURun
    from test_gpu_full_size import _check_grads, _gpu_decisions
    # weights of std 0.05: with larger ones the attention scores of this width saturate the softmax, and its backward
    # (p * (dp - sum(dp * p)) on probabilities stored in bf16: head size 32 takes the materialised path) loses its
    # signal to cancellation, whatever the split
    model = make_moe(d=128, F=64, C=10, std=0.05)
    x, y = lm_batch(16, 16, 61)

    def program():
        return hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS_E], 0, ffn="batch", moe="model"), 16)

    wire = lambda: hap_amd.SyntheticWire(seed=3, grad_scale=1e-2)      # peers' gradients of the size of real ones
    ex = hap_amd.compile_program(program(), [x, y], dtype="bf16", wire=wire(), rank=0, world_size=4)
    loss = ex.forward(x, y).item()
    ex.backward()
    torch.cuda.synchronize()
    decisions = _gpu_decisions(ex)
    assert sum(1 for v in decisions.values() if v.dtype == torch.long) == 1          # one MoE layer's routing
    gm_ref = program()
    run = SingleRankCPURun(gm_ref, 0, 4, wire(), "fp32", wire_dtype=torch.bfloat16, decisions=decisions)
    want = run.step(x, y)[0].item()
    assert abs(loss - want) <= 2e-2 * abs(want), (loss, want)
    _check_grads({n: rec["grad"].cpu() for n, rec in ex.params.items()},
                 {n: p.grad for n, p in gm_ref.named_parameters() if p.grad is not None}, 2e-2)


def test_moe_bf16_routing_matches(cuda):
    model = make_moe(d=64, F=96, std=0.3)
    x, y = lm_batch(4, 16, 61)
    run = _compare(model, RATIOS_E, 4, x, y, "bf16", [0], ADAM, ffn="batch", batch_sharded=False)


@pytest.mark.parametrize("ffn", ["column", "batch"])
def test_zero_sharded_parameters_lm_fp32(cuda, ffn):
    """Parameters stored as dim-0 shards, all_gather-ed forward and reduce-scattered backward (hap.rs:2527-2547)."""
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    _compare(model, RATIOS4, 8, x, y, "fp32", [0, 3], SGD, ffn=ffn, zero=True)


def test_zero_sharded_parameters_bf16_adam(cuda):
    model = make_lm(vocab=1003, S=32, d=64, H=4, F=128, layers=2, causal=False)
    x, y = lm_batch(8, 32, 1003, mlm=True)
    _compare(model, RATIOS4, 8, x, y, "bf16", [0, 2], ADAM, zero=True)


def test_zero_sharded_parameters_vit_and_moe(cuda):
    model = make_vit(img=32, patch=8, d=64, F=128)
    x, y = vit_batch(8, 32, 10)
    _compare(model, RATIOS4, 8, x, y, "fp32", [0, 3], ADAM, ffn="batch", zero=True)
    model = make_moe()
    x, y = lm_batch(16, 16, 61)
    _compare(model, RATIOS_E, 16, x, y, "fp32", [0, 2], ADAM, ffn="batch", zero=True)


@pytest.mark.parametrize("dtype,ffn", [("fp32", "column"), ("fp32", "batch"), ("bf16", "column")])
def test_head_parallel_attention(cuda, dtype, ffn):
    """Attention sharded over heads (3, 3, 1, 1 of 8): uneven row split of the in-projection, uneven column
    split of the out-projection, gather before and reduce-scatter after."""
    if dtype == "fp32":
        model = make_lm(H=8)
        x, y = lm_batch(8, 16, 97)
        _compare(model, RATIOS4, 8, x, y, dtype, [0, 3], SGD, ffn=ffn, attn="heads")
    else:
        model = make_lm(vocab=211, S=32, d=512, H=8, F=256, layers=2, causal=False)      # head_dim 64: fused attention
        x, y = lm_batch(8, 32, 211, mlm=True)
        # gelu: the gradient behind a ReLU mask flips with bf16 rounding of pre-activations near zero, which at
        # this width already costs more than the tolerance on the first FFN bias
        _compare(model, RATIOS4, 8, x, y, dtype, [0, 2], ADAM, ffn=ffn, attn="heads", activation="gelu")


def test_head_parallel_attention_leaf_forward(cuda):
    """models.head_parallel_attention called directly on GPU tensors against the CPU restatement."""
    from oracle import ops as ref
    g = torch.Generator().manual_seed(4)
    b, S, d, H, hd = 2, 24, 48, 3, 8
    x = torch.randn(b, S, d, generator=g)
    w_in, b_in = torch.randn(3 * H * hd, d, generator=g) * 0.2, torch.randn(3 * H * hd, generator=g)
    w_out = torch.randn(d, H * hd, generator=g) * 0.2
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1)
    want = ref.head_parallel_attention(x, w_in, b_in, w_out, H, mask)
    got = hap_amd.models.head_parallel_attention(x.to(cuda), w_in.to(cuda), b_in.to(cuda), w_out.to(cuda), H, mask.to(cuda))
    assert rel_err(got, want) < 1e-4


def test_module_facade_is_a_drop_in(cuda):
    """worker.py:59-76 usage: loss = dmodel(x, y); loss.backward(); torch optimizer step."""
    model = make_lm()
    x, y = lm_batch(8, 16, 97)
    run = joint_cpu(model, RATIOS4, 8)
    ref_opt = torch.optim.Adam(run.programs[0].parameters(), lr=5e-4)
    losses = run.step(x, y, [ref_opt])
    m = copy.deepcopy(model)
    gm = hap_amd.build_program(m, hap_amd.ShardingPlan([RATIOS4], 0), 8)
    dmodel = hap_amd.compile(gm, [x, y], wire=hap_amd.ReplayWire(run.world.log, 0), rank=0, world_size=4)
    opt = torch.optim.Adam(dmodel.parameters(), lr=5e-4)
    dmodel.zero_grad()
    loss = dmodel(x, y)
    loss.backward()
    opt.step()
    assert abs(loss.item() - losses[0].item()) < 1e-4 * abs(losses[0].item())
    ref_params = dict(run.programs[0].named_parameters())
    for n, rec in dmodel.executor.params.items():
        g_ref = ref_params[n].grad
        clear = g_ref.abs() > 1e-2 * g_ref.abs().max()
        got, want = rec["param"].detach().cpu(), ref_params[n].detach()
        assert rel_err(got[clear], want[clear]) < 1e-3, n


@pytest.mark.parametrize("lists", [True, False])
def test_send_hooks_run_in_every_step(cuda, lists):
    """Wire.send may return a callable that the executor runs in every step once the message is complete, also in the
    steps that replay the recorded launch lists.  Three passes on three different batches: what ReplayWire's hooks
    snapshot after the third pass must be the third batch's messages (the peers' messages are the recorded run's of
    that batch, so the first two passes compute on mismatched data, which does not matter here)."""
    model = make_lm()
    batches = [lm_batch(8, 16, 97, seed=s) for s in (1, 2, 3)]
    run = joint_cpu(model, RATIOS4, 8)
    run.step(*batches[2])
    gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
    ex = hap_amd.compile_program(gm, list(batches[0]), wire=hap_amd.ReplayWire(run.world.log, 0), rank=0, world_size=4,
                                 launch_lists=lists)
    assert ex._send_hooks > 0
    first = None
    for i, (x, y) in enumerate(batches):
        ex.forward(x, y)
        ex.backward()
        torch.cuda.synchronize()
        if i == 0:
            first = {k: v.clone() for k, v in ex.wire.sent.items()}
    _check_sent_messages(ex, run.world.log, 0, "fp32")
    assert any(not torch.equal(first[k], v) for k, v in ex.wire.sent.items())
    ex.configure_optimizer(**SGD)
    with pytest.raises(RuntimeError, match="captured graph"):
        ex.capture_train_step()


def test_unsupported_nodes_raise(cuda):
    """An op outside the emitted vocabulary (hap.rs:995-2240 has no handler for it either) is refused when the program
    is compiled, not executed some other way."""
    model = make_lm()
    gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
    relu = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.nn.functional.relu)
    relu.target = torch.tanh
    relu.kwargs = {}
    gm.recompile()
    with pytest.raises(ValueError, match="no handler"):
        hap_amd.compile_program(gm, [(8, 16), (8, 16)])


@pytest.mark.parametrize("dtype,opt", [("fp32", SGD), ("bf16", ADAM)])
def test_hip_graph_replays_equal_eager_steps(cuda, dtype, opt):
    """A captured training step replayed several times (with unrelated eager work and synchronisations between the
    replays) gives the same losses and parameters as eager steps."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2)        # head_dim 64: the fused attention path in bf16
    x, y = lm_batch(8, 32, 211)

    def build():
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                     rank=0, world_size=4)
        ex.configure_optimizer(**opt, clip_grad_norm=0.5)
        return ex

    eager, graphed = build(), build()
    ref_losses = [eager.train_step(x, y).item() for _ in range(5)]
    losses = [graphed.train_step(x, y).item()]                           # warm-up: first launches happen eagerly
    replay = graphed.capture_train_step()
    for i in range(4):
        junk = torch.randn(256, 256, device=cuda) @ torch.randn(256, 256, device=cuda)   # eager work in between
        torch.cuda.synchronize()
        losses.append(replay().item())
        assert torch.isfinite(junk).all()
    # same kernels, same data, fixed summation orders: the replayed steps give the eager steps' bits
    assert losses == ref_losses
    _same_bits(graphed, eager, ("grad", "master"))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_side_stream_weight_gradients_equal_main_stream(cuda, dtype):
    """With overlap_wgrad=True the weight-gradient GEMMs run on a second stream.  Compared with the main-stream order
    the loss and every gradient must come out bit-identical, repeatedly."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=3)
    x, y = lm_batch(8, 32, 211)

    def build(overlap):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        return hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, overlap_wgrad=overlap, wgrad_group=1)

    a, b = build(True), build(False)
    assert a._side_stream is not None and b._side_stream is None
    for _ in range(4):
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        assert la == lb
        _same_bits(a, b)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_relu_mask_in_the_data_gradient_equals_the_separate_pass(cuda, dtype):
    """relu_mask_in_dgrad=True folds relu's backward into the epilogue of the second FFN linear's data-gradient
    GEMM (c_relu_mask): same loss, same gradients as the separate elementwise pass."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2)
    x, y = lm_batch(8, 32, 211)

    def build(masked, in_split=False):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        return hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, relu_mask_in_dgrad=masked, relu_bwd_in_split=in_split)

    a, b = build(True), build(False)
    la = a.forward(x, y).item()
    a.backward()
    lb = b.forward(x, y).item()
    b.backward()
    torch.cuda.synchronize()
    assert la == lb
    _same_bits(a, b)
    assert len(a.bwd) == len(b.bwd) - 2                          # one relu-backward launch per layer gone


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_relu_backward_in_the_split_of_the_exchange_equals_the_separate_pass(cuda, dtype):
    """Default: the backward all_to_all's copying split applies the mask of the relu that follows the forward
    exchange (hapmi_split_rows_relu_bwd).  Same loss, bit-equal messages and gradients as the separate pass."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2)
    x, y = lm_batch(8, 32, 211)

    def build(in_split):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        return hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, relu_bwd_in_split=in_split, relu_mask_in_dgrad=False)

    a, b = build(True), build(False)
    la = a.forward(x, y).item()
    a.backward()
    lb = b.forward(x, y).item()
    b.backward()
    torch.cuda.synchronize()
    assert la == lb
    _same_bits(a, b)
    assert len(a.bwd) == len(b.bwd) - 2


@pytest.mark.parametrize("form", ["heads", "moe", "zero"])
def test_in_place_receives_survive_training_steps(cuda, form):
    """The stand-in wires deliver a message once, when the program is compiled.  Where it is delivered into a buffer
    of the executor (receive_in_place), no launch of a later step may have written there: three optimizer steps give
    the same losses and parameters as with separate receive buffers, for the forms with gathers and reduce-scatters
    in both directions."""
    if form == "moe":
        model, ratios, kw, B = make_moe(), RATIOS_E, dict(ffn="batch"), 16
        x, y = lm_batch(B, 16, 61)
    else:
        model, ratios, B = make_lm(vocab=211, S=32, d=64, H=4, F=128, layers=2), RATIOS4, 8
        kw = dict(ffn="column", attn="heads") if form == "heads" else dict(ffn="column", zero=True)
        x, y = lm_batch(B, 32, 211)

    def build(in_place):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([ratios], 0, **kw), B)
        ex = hap_amd.compile_program(gm, [x, y], dtype="fp32", wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                     rank=0, world_size=4, receive_in_place=in_place)
        ex.configure_optimizer(**SGD)
        return ex

    a, b = build(True), build(False)
    for _ in range(3):
        la, lb = a.train_step(x, y).item(), b.train_step(x, y).item()
        assert la == lb
    # a buffer overwritten by a later launch would differ by the size of its values; nothing may differ at all
    _same_bits(a, b, ("grad", "master"))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_pieces_received_in_place_equal_the_copied_concatenation(cuda, dtype):
    """receive_in_place: the backward all_to_all of the column-sharded FFN hands the wire the row ranges of its
    result (Wire.recv(into=...)) instead of concatenating separate buffers.  Same loss, bit-equal gradients, also
    on a second step (the peers' rows must have survived the first)."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2)
    x, y = lm_batch(8, 32, 211)

    def build(in_place):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        return hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, receive_in_place=in_place)

    a, b = build(True), build(False)
    assert a._wire_backed and not b._wire_backed
    for _ in range(2):
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        assert la == lb
        _same_bits(a, b)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("ffn,zero", [("column", False), ("batch", False), ("column", True)])
def test_weight_gradients_of_consecutive_layers_in_one_launch_equal_single_launches(cuda, dtype, ffn, zero):
    """wgrad_group: the same linear's weight gradients of several layers share a launch (pointer lists) and are
    held back until the group is full.  The gradient buffers they read alias across residual adds and would be
    accumulated into in place before the launch: those sums go to new buffers instead.  Same loss and gradients as
    one launch per weight gradient, for groups that fill (2 of 4 layers), do not fill (8) and the plan forms."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=4, causal=(ffn == "column"))
    x, y = lm_batch(8, 32, 211)

    def build(group):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0, ffn=ffn, zero=zero), 8)
        return hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, wgrad_group=group)

    ref = build(1)
    lr = ref.forward(x, y).item()
    ref.backward()
    for group in (2, 8):
        a = build(group)
        la = a.forward(x, y).item()
        a.backward()
        torch.cuda.synchronize()
        assert la == lr
        assert len(a.bwd) < len(ref.bwd)
        for n, rec in a.params.items():
            ga, gb = rec["grad"], ref.params[n]["grad"]
            torch.testing.assert_close(ga, gb, rtol=1e-4, atol=2e-5 * max(gb.abs().max().item(), 1e-6), msg=lambda m: f"{n}: {m}")
        # a second step over the recorded launch lists gives the same gradients again
        a.forward(x, y)
        a.backward()
        torch.cuda.synchronize()
        for n, rec in a.params.items():
            torch.testing.assert_close(rec["grad"], ref.params[n]["grad"], rtol=1e-4, atol=2e-5 * max(ref.params[n]["grad"].abs().max().item(), 1e-6))


@pytest.mark.parametrize("dtype,opt,zero", [("fp32", ADAM, False), ("bf16", ADAM, False), ("bf16", SGD, False),
                                            ("bf16", ADAM, True)])
def test_optimizer_overlapped_with_backward_equals_the_separate_step(cuda, dtype, opt, zero):
    """train_step() updates every stretch of the flat parameter buffer on a second stream as soon as backward is
    done with it.  Same losses and parameters as backward followed by one optimizer launch, over several steps,
    host-launched (first step closures, later steps recorded launch lists) and replayed from a HIP graph."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=3)
    x, y = lm_batch(8, 32, 211)

    def build(overlap):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0, zero=zero), 8)
        ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                     rank=0, world_size=4, overlap_optimizer=overlap, optimizer_chunk_min=1024,
                                     wgrad_group=1)
        ex.configure_optimizer(**opt)
        return ex

    a, b = build(True), build(False)
    assert a._opt_chunks is not None and b._opt_chunks is None
    assert sum(len(v) for v in a._opt_chunks.values()) >= 3                 # several stretches, several ready points
    assert len(a._opt_chunks) >= 2
    a.load_inputs(x, y)
    b.load_inputs(x, y)

    for _ in range(3):
        la, lb = a.train_step().item(), b.train_step().item()
        assert la == lb
        _same_bits(a, b, ("grad", "master"))
    ra, rb = a.capture_train_step(), b.capture_train_step()
    for _ in range(3):
        la, lb = ra().item(), rb().item()
        assert la == lb
        _same_bits(a, b, ("grad", "master"))


@pytest.mark.parametrize("family", ["lm", "vit", "moe"])
def test_recorded_launch_lists_equal_closure_execution(cuda, family):
    """By default the library calls of the first forward / backward / optimizer phase are recorded and later
    phases replay the recorded calls.  Against an executor that runs its closures every time: identical losses,
    gradients and parameters, bit for bit, over repeated passes and optimizer steps."""
    if family == "lm":
        model, (x, y), ratios, B, kw = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2), lm_batch(8, 32, 211), RATIOS4, 8, {}
    elif family == "vit":
        model, (x, y), ratios, B, kw = make_vit(img=32, patch=8, d=64, F=128), vit_batch(8, 32, 10), RATIOS4, 8, dict(ffn="batch")
    else:
        model, (x, y), ratios, B, kw = make_moe(), lm_batch(4, 16, 61), RATIOS_E, 4, dict(ffn="batch", batch_sharded=False)

    def build(lists):
        plan = hap_amd.ShardingPlan([list(ratios)], 0, ffn=kw.get("ffn", "column"))
        gm = hap_amd.build_program(copy.deepcopy(model), plan, B, batch_sharded=kw.get("batch_sharded", True))
        ex = hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                     rank=0, world_size=len(ratios), launch_lists=lists)
        ex.configure_optimizer(kind="adam", lr=5e-4, clip_grad_norm=0.5)
        return ex

    a, b = build(True), build(False)
    assert a.launch_lists and not b.launch_lists
    for it in range(3):
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        assert la == lb, it
        _same_bits(a, b)
    assert ("fwd", torch.cuda.current_stream().cuda_stream) in a._lists and not b._lists
    for it in range(3):
        la, lb = a.train_step(x, y).item(), b.train_step(x, y).item()
        assert la == lb, it
    _same_bits(a, b, ("grad", "master"))


def test_exchange_read_and_written_in_pieces_bf16(cuda):
    """all_to_all -> relu -> linear in bf16 with piece boundaries on multiples of 128 (FFN 1024 over ratios
    .375/.375/.125/.125 -> 384, 384, 128, 128): the second FFN linear reads the exchanged pieces where they lie (relu
    on load) and its backward writes the pieces of the backward exchange; no concatenating / splitting copy is
    launched.  Against the CPU run of all ranks with replayed messages (every message this rank sends is compared
    too), and against the executor that keeps the copies."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=1024, layers=2, causal=False)
    x, y = lm_batch(8, 32, 211, mlm=True)
    run = _compare(model, RATIOS4, 8, x, y, "bf16", [0, 3], SGD)

    def build(in_pieces):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        return hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                       rank=0, world_size=4, exchange_in_pieces=in_pieces)

    a, b = build(True), build(False)
    kinds = [v.kind for v in a.env.values() if hasattr(v, "kind")]
    assert kinds.count("pieces") >= 2 and "pieces" not in [v.kind for v in b.env.values() if hasattr(v, "kind")]
    assert len(a.fwd) < len(b.fwd)
    for _ in range(2):                                       # the second pass replays the recorded launch lists
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        assert abs(la - lb) <= 1e-3 * abs(lb)
        for n, rec in a.params.items():
            gb = b.params[n]["grad"]
            if gb.norm().item() > 0:
                assert rel_err(rec["grad"], gb) < 1e-2, n


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_sequence_sharded_program(cuda, dtype):
    """Inputs, embedding, LayerNorm, FFN, decoder and loss on the device's uneven share of the POSITIONS (placeholder
    split on dim 1, hap.rs:2500-2520; gathers on dim 1 through linear / layer_norm / embedding / add,
    hap.rs:2795, 3061, 3214-3218, 2996); all_gather(dim 1) before and dynamic_slice(dim 1) behind attention."""
    if dtype == "fp32":
        model = make_lm(S=19)                                          # 19 positions over 4 devices: 7, 7, 2, 3
        x, y = lm_batch(6, 19, 97)
        _compare(model, RATIOS4, 6, x, y, dtype, [0, 2, 3], SGD, ffn="batch", shard_dim="sequence")
    else:
        model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2, causal=False)
        x, y = lm_batch(6, 32, 211, mlm=True)
        _compare(model, RATIOS4, 6, x, y, dtype, [0, 3], SGD, ffn="batch", shard_dim="sequence")


@pytest.mark.parametrize("shard_dim,ffn", [("batch", "column"), ("batch", "batch"), ("sequence", "batch")])
def test_embedding_table_sharded_over_features(cuda, shard_dim, ffn):
    """F.embedding with whole ids and the table sharded on dim 1 gives its output gathered on dim 2 (hap.rs:3220-3224);
    all_gather(dim 2) and dynamic_slice behind it."""
    model = make_lm(d=64, H=4)                                         # 64 columns over 4 devices: 24, 24, 8, 8
    x, y = lm_batch(8, 16, 97)
    _compare(model, RATIOS4, 8, x, y, "fp32", [0, 3], ADAM, ffn=ffn, shard_dim=shard_dim, embedding="features")
