"""F.dropout with p > 0 (hap.rs:1447-1491; the reference trains with dropout = 0.1, config.py:33) and the dropout of
the attention probabilities (hap.rs:1257, 1307).

The reference draws its masks from torch's generator, whose stream no GPU kernel can reproduce, so bitwise equality
with a torch run is out of reach by construction: PARITY UNPINNED for the particular masks.  What is checked:
* the keep decisions are integer work and equal the CPU restatement oracle.ops.dropout_keep bit for bit (which
  tests/test_oracle_dropout.py holds to the statistics of a Bernoulli(1 - p) mask);
* p = 0 is the identity, kept elements are scaled by 1 / (1 - p), dropped ones are zero, forward and backward of a
  node use one mask, another step / node / seed gives another;
* whole programs with dropout in every place the generator puts it: loss and every gradient against the CPU
  oracle running the same graph with the GPU's masks (SingleRankCPURun(decisions=...)), at 1e-4 / 2e-2;
* a step replayed from a HIP graph draws a new mask every replay and equals the eager step of the same number."""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import hap_amd
from hap_amd import ops
from helpers import RATIOS4, lm_batch, make_lm, make_vit, rel_err, vit_batch
from oracle import ops as ref
from oracle.cpu_executor import SingleRankCPURun

pytestmark = pytest.mark.gpu


def _state(cuda, seed, step):
    return torch.tensor([seed, step], dtype=torch.int64, device=cuda)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dropout_kernel(cuda, dtype):
    g = torch.Generator().manual_seed(3)
    n = 1_000_003
    x = (torch.randn(n, generator=g) + 3).to(dtype).to(cuda)
    st = _state(cuda, 17, 4)
    y = torch.empty_like(x)
    ops.dropout(x, y, 0.0, st, 5)
    assert torch.equal(y, x)                                                   # p = 0: identity
    p = 0.1
    ops.dropout(x, y, p, st, 5)
    keep = ops.dropout_mask(n, p, st, 5).bool()
    want_keep = ref.dropout_keep(17, 4, 5, p, n)
    assert torch.equal(keep.cpu(), want_keep)                                  # the oracle's bits
    assert torch.equal(y != 0, keep)                                           # x > 0 everywhere: zero iff dropped
    want = (x.float() * (1.0 / (1.0 - p))).to(dtype)
    assert torch.equal(y[keep], want[keep])
    assert abs(keep.double().mean().item() - (1 - p)) < 4.5 * math.sqrt(p * (1 - p) / n) + 2.0 ** -16
    assert abs(y.double().mean().item() / x.double().mean().item() - 1) < 2e-3  # unbiased
    # backward = the same call on the gradient: same mask; in place allowed
    gy = torch.randn(n, generator=g).to(dtype).to(cuda)
    gx = gy.clone()
    ops.dropout(gx, gx, p, st, 5)
    assert torch.equal(gx != 0, keep & (gy != 0))
    # another node, step or seed: another mask
    for other in (ops.dropout_mask(n, p, st, 6), ops.dropout_mask(n, p, _state(cuda, 17, 5), 5),
                  ops.dropout_mask(n, p, _state(cuda, 18, 4), 5)):
        assert 0.14 < (other.bool() != keep).double().mean().item() < 0.22     # 2 p (1 - p) = 0.18
    ops.rng_advance(st)
    assert st.tolist() == [17, 5]
    assert torch.equal(ops.dropout_mask(n, p, st, 5), ops.dropout_mask(n, p, _state(cuda, 17, 5), 5))
    ops.dropout(x, y, 1.0, st, 5)
    assert not y.any()                                                         # p = 1: everything dropped


@pytest.mark.parametrize("dtype,width", [(torch.float32, 96), (torch.bfloat16, 1024), (torch.bfloat16, 100), (torch.float32, 37)])
def test_dropout_inside_the_residual_layer_norm(cuda, dtype, width):
    """LN(dropout(x) + res) in one kernel and its two-result backward against the three separate kernels (dropout,
    add + layer_norm, their backwards): the same decisions, and values equal to the last bit of the storage type
    (both round where the separate kernels store)."""
    rows, p, sid = 37, 0.3, 9
    g = torch.Generator().manual_seed(width)
    x = torch.randn(rows, width, generator=g).to(dtype).to(cuda)
    res = torch.randn(rows, width, generator=g).to(dtype).to(cuda)
    dy = torch.randn(rows, width, generator=g).to(dtype).to(cuda)
    st = _state(cuda, 5, 2)
    xd, y0, y1 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    r0, r1 = torch.empty(rows, device=cuda), torch.empty(rows, device=cuda)
    ops.dropout(x, xd, p, st, sid)
    ops.add_layernorm_fwd(xd, res, y0, r0)
    ops.add_layernorm_fwd(x, res, y1, r1, drop=(p, st, sid))
    # float32: the fused kernel may contract x * scale + res into one fused multiply-add
    same = torch.equal if dtype == torch.bfloat16 else (lambda u, v: torch.allclose(u, v, rtol=1e-5, atol=1e-6))
    assert same(y0, y1) and same(r0, r1)
    dx0, dd0, dx1, dd1 = (torch.empty_like(x) for _ in range(4))
    ops.layernorm_bwd(dy, y0, r0, None, dx0)
    ops.dropout(dx0, dd0, p, st, sid)
    ops.layernorm_bwd(dy, y1, r1, None, dx1, dd1, (p, st, sid))
    assert same(dx0, dx1) and same(dd0, dd1)
    keep = ops.dropout_mask(rows * width, p, st, sid).view(rows, width).bool()
    assert torch.equal(dd1 != 0, keep & (dx1 != 0))
    with pytest.raises(ValueError):
        ops.layernorm_bwd(dy, y1, r1, None, dx1, dx1, (p, st, sid))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dim", [0, 2])
def test_relu_and_dropout_inside_the_concatenating_copy(cuda, dtype, dim):
    """dropout(relu(cat(pieces))) in the copy of an all_to_all against concat, relu and dropout as separate kernels
    (bit for bit), and its backward -- split of g * (dropped output > 0) / (1 - p) -- against dropout's and relu's
    backward kernels followed by the split."""
    p, sid = 0.3, 4
    g = torch.Generator().manual_seed(3 + dim)
    lengths = [8, 24, 0, 16]
    shape = [6, 5, 48]
    pieces = []
    for l in lengths:
        sh = list(shape)
        sh[dim] = l
        pieces.append(torch.randn(*sh, generator=g).to(dtype).to(cuda))
    shape[dim] = sum(lengths)
    st = _state(cuda, 21, 6)
    want = torch.empty(*shape, dtype=dtype, device=cuda)
    ops.concat_rows(pieces, dim, want, "relu")
    ops.dropout(want, want, p, st, sid)
    got = ops.concat_rows(pieces, dim, torch.empty_like(want), "relu", drop=(p, st, sid))
    assert torch.equal(got, want)
    keep = ops.dropout_mask(want.numel(), p, st, sid).view(want.shape).bool()
    assert torch.equal(got != 0, keep & (torch.cat(pieces, dim) > 0))
    dy = torch.randn(*shape, generator=g).to(dtype).to(cuda)
    tmp = torch.empty_like(dy)
    ops.dropout(dy, tmp, p, st, sid)
    ops.act_bwd(tmp, want, tmp, "relu")
    want_pieces = ops.split_rows(tmp, lengths, dim)
    got_pieces = ops.split_rows(dy, lengths, dim, relu_of=got, scale=1.0 / (1.0 - p))
    for a, b in zip(got_pieces, want_pieces):
        assert torch.equal(a, b)


@pytest.mark.parametrize("cfg,in_dtype,out_dtype", [(0, "bf16", "bf16"), (1, "bf16", "bf16"), (4, "bf16", "bf16"),
                                                    (7, "bf16", "bf16"), (7, "bf16", "fp32"), (9, "bf16", "bf16"),
                                                    (10, "fp32", "fp32"), (-1, "fp32", "fp32"), (-1, "bf16", "bf16")])
def test_relu_and_dropout_in_the_gemm_epilogue(cuda, cfg, in_dtype, out_dtype):
    """dropout(relu(x W^T + b)) from the GEMM's epilogue against the same GEMM with relu followed by the dropout
    kernel: identical bits (the epilogue rounds a 2-byte result before scaling it, as the stored activation would
    be), on a shape with partial tiles in M and N and a tile-aligned one, through several tile configurations."""
    from hap_amd._lib import lib
    tin = torch.bfloat16 if in_dtype == "bf16" else torch.float32
    tout = torch.bfloat16 if out_dtype == "bf16" else torch.float32
    p, sid = 0.25, 13
    st = _state(cuda, 77, 1)
    try:
        lib().hapmi_gemm_tuning(cfg, 1 if cfg >= 0 else 0)
        for (M, N, K) in [(424, 520, 192), (768, 512, 256)]:
            g = torch.Generator().manual_seed(M)
            A = torch.randn(M, K, generator=g).to(tin).to(cuda)
            B = torch.randn(N, K, generator=g).to(tin).to(cuda)
            bias = torch.randn(N, generator=g).to(cuda)
            want = torch.empty(M, N, dtype=tout, device=cuda)
            ops.gemm(A, B, want, M, N, K, transB=True, bias=bias, act="relu")
            ops.dropout(want, want, p, st, sid)
            got = torch.full((M, N), float("nan"), dtype=tout, device=cuda)
            ops.gemm(A, B, got, M, N, K, transB=True, bias=bias, act="relu", drop=(p, st, sid))
            if cfg >= 0:
                assert torch.equal(got, want), (M, N, K)
            else:       # left to itself the library may split the plain GEMM's reduction (another summation order)
                assert torch.equal(got != 0, want != 0) and torch.allclose(got.float(), want.float(), rtol=1e-2 if tout == torch.bfloat16 else 1e-4, atol=1e-4)
            assert 0.3 < (got != 0).float().mean().item() < 0.45      # half pass relu, three quarters of those are kept
    finally:
        lib().hapmi_gemm_tuning(-1, 0)
    with pytest.raises(ops._lib.HapmiError):                           # a padded leading dimension has no flat index
        ops.gemm(A, B, torch.empty(M, N + 8, dtype=tout, device=cuda), M, N, K, transB=True, ldc=N + 8, act="relu",
                 drop=(p, st, sid))


def _masks_from_oracle(ex, step):
    """The decisions the CPU oracle is given: relu masks from the GPU (see test_gpu_full_size), dropout masks from
    the oracle's own restatement of the keep function for the executor's seed, the step count and the node ids."""
    seed = int(ex.rng_state[0].item())
    assert int(ex.rng_state[1].item()) == step
    out = {}
    gpu_masks = ex.dropout_masks()
    for i, node in enumerate(ex.gm.graph.nodes):
        if node.op != "call_function":
            continue
        if node.target is F.dropout and float(node.args[1]) > 0:
            shape = ex.env[node].shape                     # a dropout inside a neighbouring kernel has no tensor
            out[node.name] = ref.dropout_keep(seed, step, i, float(node.args[1]), math.prod(shape)).view(shape)
        elif node.target is F.multi_head_attention_forward and float(node.kwargs["dropout_p"]) > 0:
            p, sid, shape, S = ex.env[node].meta["dropout"]
            assert sid == i
            n = shape[0] * shape[1] * shape[2] * shape[3]
            out[node.name] = ref.dropout_keep(seed, step, i, p, n).view(shape)[..., :S]
        elif node.target is F.relu:
            v = ex.env[node]
            out[node.name] = (torch.cat([t > 0 for t in v.meta["pieces"]], dim=-1) if v.kind == "pieces" else v.t > 0).cpu()
            continue
        else:
            continue
        assert torch.equal(gpu_masks[node.name].cpu(), out[node.name]), node.name
    return out


def test_relu_and_dropout_written_piece_by_piece(cuda):
    """dropout(relu(.)) of the pieces of an all_to_all without concatenating them: every piece equals its columns of
    the concatenated result that the separate kernels give (bit for bit), also in place."""
    p, sid, rows = 0.3, 4, 45
    g = torch.Generator().manual_seed(8)
    widths = [128, 384, 64, 8]
    src = [torch.randn(rows, w, generator=g).bfloat16().to(cuda) for w in widths]
    st = _state(cuda, 2, 9)
    want = torch.relu(torch.cat(src, 1))
    ops.dropout(want, want, p, st, sid)
    dst = [torch.full_like(t, float("nan")) for t in src]
    ops.relu_dropout_pieces(src, dst, p, st, sid)
    for d, w in zip(dst, torch.split(want, widths, 1)):
        assert torch.equal(d, w)
    ops.relu_dropout_pieces(src, src, p, st, sid)
    for d, w in zip(src, torch.split(want, widths, 1)):
        assert torch.equal(d, w)


def test_program_with_dropout_on_exchange_pieces(cuda):
    """all_to_all -> relu -> dropout -> linear with piece boundaries on multiples of 128: the linear reads dropped
    pieces and its backward writes the pieces of the backward exchange.  The same program with the concatenating
    copies takes the same decisions, so losses and gradients agree to bf16 rounding; and against the CPU oracle
    given the masks."""
    model = make_lm(vocab=211, S=32, d=64, H=1, F=1024, layers=2, causal=False)
    model.dropout_p = 0.1
    x, y = lm_batch(8, 32, 211, mlm=True)

    def program():
        return hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)

    def build(in_pieces):
        return hap_amd.compile_program(program(), [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=3),
                                       rank=0, world_size=4, exchange_in_pieces=in_pieces, dropout_seed=5)

    a, b = build(True), build(False)
    kinds = [v.kind for v in a.env.values() if hasattr(v, "kind")]
    assert kinds.count("pieces") >= 4 and "pieces" not in [v.kind for v in b.env.values() if hasattr(v, "kind")]
    for step in (1, 2):
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        ma, mb = a.dropout_masks(), b.dropout_masks()
        assert set(ma) == set(mb) and all(torch.equal(ma[k], mb[k]) for k in ma)
        assert abs(la - lb) <= 1e-3 * abs(lb)
        for n, rec in a.params.items():
            gb = b.params[n]["grad"]
            if gb.norm().item() > 0:
                assert rel_err(rec["grad"], gb) < 1e-2, n
        decisions = _masks_from_oracle(a, step)
        gm_ref = program()
        run = SingleRankCPURun(gm_ref, 0, 4, hap_amd.SyntheticWire(seed=3), "fp32", wire_dtype=torch.bfloat16,
                               decisions=decisions)
        want = run.step(x, y)[0].item()
        assert abs(la - want) <= 2e-2 * abs(want), (step, la, want)
        ref_grads = {n: p_.grad for n, p_ in gm_ref.named_parameters() if p_.grad is not None}
        scale = max(g.norm().item() for g in ref_grads.values())
        for n, rec in a.params.items():
            if ref_grads[n].norm().item() > 1e-4 * scale:
                assert rel_err(rec["grad"], ref_grads[n]) < 2e-2, (step, n)


@pytest.mark.parametrize("family,dtype", [("lm", "fp32"), ("lm", "bf16"), ("vit", "fp32"), ("vit", "bf16")])
def test_program_with_dropout_against_the_oracle_given_the_masks(cuda, family, dtype):
    if family == "lm":
        model = make_lm(vocab=211, S=32, d=64, H=1 if dtype == "bf16" else 4, F=128, layers=2)
        x, y = lm_batch(8, 32, 211)
        kw = {}
    else:
        model = make_vit(img=32, patch=8, d=64, H=1 if dtype == "bf16" else 4, F=128)
        x, y = vit_batch(8, 32, 10)
        kw = dict(ffn="batch")
    model.dropout_p = 0.1

    def program():
        return hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0, **kw), 8)

    gm = program()
    n_drop = sum(1 for n in gm.graph.nodes if n.op == "call_function" and n.target is F.dropout)
    assert n_drop >= 6
    ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=hap_amd.SyntheticWire(seed=3), rank=0, world_size=4,
                                 dropout_seed=1234)
    tol = 1e-4 if dtype == "fp32" else 2e-2
    for step in (1, 2):                                       # the second step draws other masks
        loss = ex.forward(x, y).item()
        ex.backward()
        torch.cuda.synchronize()
        decisions = _masks_from_oracle(ex, step)
        assert sum(1 for v in decisions.values() if not v.all()) >= n_drop
        gm_ref = program()
        run = SingleRankCPURun(gm_ref, 0, 4, hap_amd.SyntheticWire(seed=3), "fp32",
                               wire_dtype=torch.bfloat16 if dtype == "bf16" else None, decisions=decisions)
        want = run.step(x, y)[0].item()
        assert abs(loss - want) <= tol * abs(want), (step, loss, want)
        ref_grads = {n: p.grad for n, p in gm_ref.named_parameters() if p.grad is not None}
        assert set(ref_grads) == set(ex.params)
        scale = max(g.norm().item() for g in ref_grads.values())
        for n, rec in ex.params.items():
            if ref_grads[n].norm().item() > 1e-4 * scale:
                assert rel_err(rec["grad"], ref_grads[n]) < tol, (step, n)
        if step == 1:
            first = decisions
    assert any(not torch.equal(first[k], decisions[k]) for k in first if "dropout" in k)


@pytest.mark.parametrize("family", ["lm", "vit"])
def test_fused_and_separate_dropouts_take_the_same_decisions(cuda, family):
    """The same bf16 program with every dropout inside a neighbouring kernel (the default) and with every dropout as
    a pass of its own (fuse_dropout=False, attention through the materialised probabilities): the keep decisions
    are identical, node by node, so losses and gradients agree to bf16 rounding."""
    if family == "lm":
        model = make_lm(vocab=211, S=32, d=64, H=1, F=1024, layers=2, causal=False)
        x, y = lm_batch(8, 32, 211, mlm=True)
        kw = {}
    else:
        model = make_vit(img=32, patch=8, d=64, H=1, F=128)
        x, y = vit_batch(8, 32, 10)
        kw = dict(ffn="batch")
    model.dropout_p = 0.2

    def build(fuse):
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0, **kw), 8)
        return hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=3), rank=0,
                                       world_size=4, dropout_seed=11, fuse_dropout=fuse)

    a, b = build(True), build(False)
    assert len(a.fwd) < len(b.fwd)
    for _ in range(2):
        la = a.forward(x, y).item()
        a.backward()
        lb = b.forward(x, y).item()
        b.backward()
        torch.cuda.synchronize()
        ma, mb = a.dropout_masks(), b.dropout_masks()
        assert len(ma) >= 7 and set(ma) == set(mb)
        for k in ma:
            assert torch.equal(ma[k], mb[k]), k
        assert abs(la - lb) <= 2e-3 * abs(lb)
        for n, rec in a.params.items():
            gb = b.params[n]["grad"]
            if gb.norm().item() > 0:       # two bf16 computations with different rounding points: twice the bar each has against the oracle
                assert rel_err(rec["grad"], gb) < 4e-2, n


def test_dropout_is_active_and_unbiased_in_a_program(cuda):
    """Against the same program without dropout: the loss differs (dropout is on), and over many steps the mean of
    a dropped activation equals the undropped one (kept elements are scaled by 1 / (1 - p))."""
    model = make_lm(vocab=211, S=32, d=64, H=4, F=128, layers=1)
    x, y = lm_batch(8, 32, 211)
    plain = hap_amd.compile_program(hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8),
                                    [x, y], wire=hap_amd.SyntheticWire(seed=3), rank=0, world_size=4)
    model.dropout_p = 0.5
    gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
    ex = hap_amd.compile_program(gm, [x, y], wire=hap_amd.SyntheticWire(seed=3), rank=0, world_size=4)
    base = plain.forward(x, y).item()
    losses = [ex.forward(x, y).item() for _ in range(20)]
    assert len(set(losses)) == 20 and all(abs(l - base) > 1e-6 * base for l in losses)
    # a dropout that has a tensor of its own (those in front of a residual layer_norm run inside its kernel)
    node = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target is F.dropout and ex.env[n].t is not None)
    src, out = ex.env[node.args[0]], ex.env[node]
    acc, acc_src = torch.zeros_like(out.t, dtype=torch.float64), torch.zeros_like(out.t, dtype=torch.float64)
    for _ in range(200):                                                       # the input varies too (attention dropout)
        ex.forward(x, y)
        acc += out.t.double()
        acc_src += src.t.double()
    err = ((acc - acc_src).norm() / acc_src.norm()).item()
    assert err < 3.0 / math.sqrt(200), err                                     # ~ sqrt(p / (1 - p) / 200) = 0.07


def test_graph_replays_draw_new_masks_and_equal_eager_steps(cuda):
    model = make_lm(vocab=211, S=32, d=64, H=1, F=128, layers=2)
    model.dropout_p = 0.1
    x, y = lm_batch(8, 32, 211)

    def build():
        gm = hap_amd.build_program(copy.deepcopy(model), hap_amd.ShardingPlan([RATIOS4], 0), 8)
        ex = hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=3, grad_scale=1e-2),
                                     rank=0, world_size=4, dropout_seed=7)
        ex.configure_optimizer(kind="adam", lr=5e-4, clip_grad_norm=0.5)
        return ex

    eager, graphed = build(), build()
    ref_losses = [eager.train_step(x, y).item() for _ in range(5)]
    losses = [graphed.train_step(x, y).item()]
    replay = graphed.capture_train_step()            # capture runs no kernels: the step count stays where it is
    for _ in range(4):
        torch.cuda.synchronize()
        losses.append(replay().item())
    assert losses == ref_losses
    assert graphed.rng_state.tolist() == eager.rng_state.tolist() == [7, 5]
    for n, rec in graphed.params.items():
        assert torch.equal(rec["master"], eager.params[n]["master"]), n
