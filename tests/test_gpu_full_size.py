"""The benchmark configurations at their full per-kernel shapes (every GEMM, attention, gating, collective copy
and optimizer launch has the shape it has in the benchmark), one rank whose peers send SEEDED N(0, 1) activations and
N(0, 1e-3) gradients (hap_amd.SyntheticWire: the same tensors on both sides, so every row of a gathered tensor and
every column of an exchanged one carries signal), against the CPU oracle (stock PyTorch eager + autograd on the
same generated graph: the reference's arithmetic), which tests/test_oracle_single_rank.py pins on the CPU.

Tolerances are the stated ones and no wider: float32 runs 1e-4 (against the oracle in float64), bf16 runs 2e-2
(against the oracle in float32), on the loss, norm-wise on every gradient that carries signal, and on the updated
weights.

Discrete decisions are checked apart from the continuous arithmetic.  A program takes two kinds: the sign of a
ReLU's argument and the two experts a token is routed to.  Both are step functions: an argument within rounding
distance of the step turns a rounding-sized difference between two runs into a whole-sized one (one flipped
element of a 25 M element mask is 2e-4 of that gradient's norm), which no tolerance on the results can tell
from a wrong result.  So each test
  (1) runs the oracle freely and compares the loss;
  (2) takes the GPU's decisions (the masks its ReLUs applied, the experts its gating chose) and runs the oracle
      again with them (oracle.cpu_executor.SingleRankCPURun(decisions=...));
  (3) requires that the GPU's decisions differ from what that oracle run would have chosen itself only where
      its argument lies within a few roundings of the step, and prints how many do;
  (4) holds every gradient and updated weight to the stated tolerance against that run.
Routing itself is integer work and bit-exact: the oracle's gating applied to the float32 logits the GPU computed
gives the GPU's dispatch mask and combine weights.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import bench
import hap_amd
from hap_amd import models, ops
from helpers import rel_err
from oracle import ops as ref_ops
from oracle.cpu_executor import SingleRankCPURun

pytestmark = pytest.mark.gpu

SEED = 11


def _cpu_run(name, layers, wire_dtype, double=False, opt=False, decisions=None, **kw):
    gm, x, y, meta = bench.build_workload(name, layers_override=layers, **kw)
    if double:
        gm = gm.double()
    run = SingleRankCPURun(gm, 0, len(meta["ratios"]), hap_amd.SyntheticWire(seed=SEED), "fp32", wire_dtype=wire_dtype,
                           decisions=decisions)
    torch.set_num_threads(16)
    optim = [torch.optim.Adam(gm.parameters(), lr=meta["opt"]["lr"])] if opt else None
    before = {n: p.detach().clone() for n, p in gm.named_parameters()} if opt else None
    loss = run.step(x, y, optimizers=optim)[0].item()
    grads = {n: p.grad for n, p in gm.named_parameters() if p.grad is not None}
    return run, gm, loss, grads, before


def _gpu_run(name, layers, dtype, opt=False, wire=None, **kw):
    gm, x, y, meta = bench.build_workload(name, layers_override=layers, **kw)
    ex = hap_amd.compile_program(gm, [x, y], dtype=dtype, wire=wire or hap_amd.SyntheticWire(seed=SEED), rank=0,
                                 world_size=len(meta["ratios"]))
    before = {n: rec["master"].clone() for n, rec in ex.params.items()} if opt else None
    if opt:
        ex.configure_optimizer(**meta["opt"])
    loss = ex.forward(x, y)
    ex.backward()
    torch.cuda.synchronize()
    grads = {n: rec["grad"].clone() for n, rec in ex.params.items()}
    if opt:
        ex.step()
        torch.cuda.synchronize()
    return ex, loss.item(), grads, before


def _gpu_decisions(ex):
    """The decisions the GPU run took, by node name: the masks its ReLUs applied, the experts its gating chose.
    Routing is integer work: the oracle's gating applied to the float32 logits the GPU computed must give the
    GPU's dispatch mask and combine weights bit for bit."""
    decisions = {}
    for node in ex.gm.graph.nodes:
        if node.op != "call_function":
            continue
        if node.target is F.relu:
            v = ex.env[node]
            if v.kind == "pieces":                                            # an exchange read in place: relu on load
                decisions[node.name] = torch.cat([t > 0 for t in v.meta["pieces"]], dim=-1).cpu()
                continue
            act = v.t.permute(1, 0, 2, 3) if v.kind == "expert" else v.t      # experts are stored expert-major
            decisions[node.name] = (act > 0).cpu()
        elif node.target is models.top_2_gating:
            v = ex.env[node]
            r, lg = v.meta["r"], v.meta["logits"].cpu()
            E, C = v.meta["E"], v.meta["C"]
            d_same, c_same = ref_ops.top_2_gating(lg, E, C, torch.eye(E))
            got_d, got_c = ops.top2_densify(r, E, C)
            assert torch.equal(got_d.cpu().bool(), d_same.bool()), node.name
            torch.testing.assert_close(got_c.cpu(), c_same, rtol=1e-5, atol=1e-7)
            decisions[node.name] = r["index"].cpu().long()
    return decisions


def _check_decisions(ex, run, decisions, eps, params_before=None):
    """``run``: the oracle run that was given the GPU's decisions.  Its own arguments of the step functions say
    which decisions it would have taken itself: a ReLU mask may differ from the GPU's only where the oracle's
    argument is within 16 roundings (``eps`` relative to the tensor's root mean square) of zero; expert choices
    only for tokens whose deciding gate probabilities are closer to each other than twice the distance between
    the two runs' probabilities of that token."""
    for node in ex.gm.graph.nodes:
        if node.op != "call_function" or node.name not in decisions:
            continue
        if node.target is F.relu:
            mask = decisions[node.name]
            z = run.env[0][node.args[0].name].detach()
            assert mask.shape == z.shape, (node.name, mask.shape, z.shape)
            flipped = mask != (z > 0)
            n, rms = int(flipped.sum()), z.double().pow(2).mean().sqrt().item()
            worst = z[flipped].abs().max().item() if n else 0.0
            print(f"    {node.name}: {n} of {z.numel()} mask elements differ from the oracle's own choice "
                  f"(largest |argument| among them {worst:.2e}, rms of the argument {rms:.2e})")
            assert worst <= 16 * eps * rms, (node.name, worst, rms)
        else:
            lg = ex.env[node].meta["logits"].cpu()
            x0 = run.env[0][node.args[0].name].detach()
            src = node.args[3]                          # replicate(get_attr): the gate weight as it was in this step
            while src.op == "call_function":
                src = src.args[0]
            wg = params_before[src.target] if params_before is not None else run.programs[0].get_parameter(src.target).detach()
            p0 = torch.softmax(x0.double() @ wg.double(), dim=2)
            top3 = p0.topk(3, dim=2)
            moved = (torch.softmax(lg.double(), dim=2) - p0).abs().amax(dim=2)
            near_tie = ((top3.values[..., 1] - top3.values[..., 2]) <= 2 * moved) | \
                       ((top3.values[..., 0] - top3.values[..., 1]) <= 2 * moved)
            differs = (decisions[node.name] != top3.indices[..., :2]).any(dim=2)
            print(f"    {node.name}: {int(differs.sum())} of {differs.numel()} tokens routed differently from the oracle's "
                  f"own choice, {int(near_tie.sum())} tokens whose deciding gate probabilities are closer than twice the "
                  f"distance between the runs (largest distance {moved.max().item():.2e})")
            assert not (differs & ~near_tie).any(), node.name
            assert differs.float().mean().item() < 0.05, node.name


def _check_grads(grads, want, tol, floor=1e-4):
    assert set(grads) == set(want)
    scale = max(g.norm().item() for g in want.values())
    rows = []
    for n, g in grads.items():
        ref = want[n]
        if ref.norm().item() < floor * scale:       # no signal (a gradient that is zero up to rounding on both sides)
            continue
        rows.append((rel_err(g, ref), n))
    rows.sort(reverse=True)
    print("    largest gradient errors:", ", ".join(f"{n} {e:.2e}" for e, n in rows[:4]))
    assert rows[0][0] < tol, rows[0]


def _full_check(name, layers, dtype, opt=False, **kw):
    bf16 = dtype == "bf16"
    tol, eps = (2e-2, 2.0 ** -8) if bf16 else (1e-4, 2.0 ** -23)
    wire_dtype = torch.bfloat16 if bf16 else torch.float32
    free, _, want, _, _ = _cpu_run(name, layers, wire_dtype, double=not bf16, **kw)
    ex, loss, grads, before = _gpu_run(name, layers, dtype, opt=opt, **kw)
    print(f"\n  {name}, {layers} layer(s), {dtype}: loss {loss:.6f}, free oracle {want:.6f}")
    assert abs(loss - want) <= tol * abs(want), (loss, want)
    del free
    decisions = _gpu_decisions(ex)
    run, gm_ref, shared_loss, ref_grads, before_ref = _cpu_run(name, layers, wire_dtype, double=not bf16, opt=opt,
                                                                 decisions=decisions, **kw)
    assert abs(loss - shared_loss) <= tol * abs(shared_loss), (loss, shared_loss)
    _check_decisions(ex, run, decisions, eps, before_ref)
    _check_grads(grads, ref_grads, tol)
    return ex, run, gm_ref, grads, ref_grads, before, before_ref


def test_wire_requests_of_gpu_and_cpu_runs_match(cuda):
    """The executor and the CPU oracle ask the wire for the same messages (tag, direction, sender, shape)."""
    class Recording(hap_amd.SyntheticWire):
        def __init__(self):
            super().__init__(seed=SEED)
            self.requests = set()

        def recv(self, tag, direction, src, shape, dtype, device, reduction=False, into=None):
            if not (tag.startswith("replicate") and not self.reduce_params):
                self.requests.add((tag, direction, src, tuple(shape)))
            return super().recv(tag, direction, src, shape, dtype, device, reduction=reduction, into=into)

    for name in ("lm", "moe"):
        wire_gpu, wire_cpu = Recording(), Recording()
        _gpu_run(name, 2, "fp32", wire=wire_gpu)
        gm, x, y, meta = bench.build_workload(name, layers_override=2)
        SingleRankCPURun(gm, 0, len(meta["ratios"]), wire_cpu).step(x, y)
        assert wire_gpu.requests and wire_gpu.requests == wire_cpu.requests, name


def test_lm_config1_full_size_fp32(cuda):
    """benchmark configuration 1 (bench.py --workload lm) whole (2 layers, float32): the GPU against the float64 CPU run at 1e-4."""
    _full_check("lm", 2, "fp32")


def test_bert_large_shard_full_width_bf16(cuda):
    _full_check("bert", 2, "bf16")


def test_bert_large_shard_full_width_bf16_with_dropout(cuda):
    """Two layers of benchmark configuration 2 (bench.py --workload bert) with the reference's default dropout probability (config.py:33) at the real
    shapes: F.dropout in front of both residual LayerNorms and behind the FFN's relu (on the exchange's pieces),
    dropout_p on the probabilities of the fused attention (b 12, 16 heads, S 512).  The masks cannot be those of a
    torch run (PARITY UNPINNED for the particular masks); the GPU's are checked against the CPU restatement of the
    generator bit for bit and handed, with the relu masks, to the oracle, which must then give the GPU's loss and
    gradients within the bf16 tolerance."""
    p, seed = 0.1, 77
    gm, x, y, meta = bench.build_workload("bert", layers_override=2, dropout=p)
    W = len(meta["ratios"])
    ex = hap_amd.compile_program(gm, [x, y], dtype="bf16", wire=hap_amd.SyntheticWire(seed=SEED), rank=0, world_size=W,
                                 dropout_seed=seed)
    kinds = [v.kind for v in ex.env.values() if hasattr(v, "kind")]
    assert "pieces" in kinds and "dropped" in kinds                    # the dropouts run inside their neighbours
    loss = ex.forward(x, y).item()
    ex.backward()
    torch.cuda.synchronize()
    grads = {n: rec["grad"].clone() for n, rec in ex.params.items()}
    decisions = _gpu_decisions(ex)
    masks = {k: v.cpu() for k, v in ex.dropout_masks().items()}
    assert len(masks) >= 8                                             # per layer: 3 F.dropout + the attention's
    for i, node in enumerate(ex.gm.graph.nodes):                        # stream id = the node's index in the program
        if node.name in masks:
            m = masks[node.name]
            if node.target is F.dropout:
                want = ref_ops.dropout_keep(seed, 1, i, p, m.numel()).view(m.shape)
            else:
                _, _, shape, S = ex.env[node].meta["dropout"]
                want = ref_ops.dropout_keep(seed, 1, i, p, math.prod(shape)).view(shape)[..., :S]
            assert torch.equal(m, want), node.name
            assert abs(m.float().mean().item() - (1 - p)) < 2e-3, node.name
    decisions.update(masks)
    gm_ref, _, _, _ = bench.build_workload("bert", layers_override=2, dropout=p)
    run = SingleRankCPURun(gm_ref, 0, W, hap_amd.SyntheticWire(seed=SEED), "fp32", wire_dtype=torch.bfloat16,
                           decisions=decisions)
    torch.set_num_threads(16)
    want = run.step(x, y)[0].item()
    print(f"\n  bert with dropout {p}, 2 layers, bf16: loss {loss:.6f}, oracle with the GPU's masks {want:.6f}")
    assert abs(loss - want) <= 2e-2 * abs(want), (loss, want)
    _check_grads(grads, {n: q.grad for n, q in gm_ref.named_parameters() if q.grad is not None}, 2e-2)


def _full_check_with_adam_step(name, layers, lr=5e-4):
    """The whole workload in bf16 with one Adam step: loss, gradients (``_full_check``), then the updated float32
    masters, the bf16 shadows that the next step reads, and the size of the first update."""
    ex, run, gm_ref, grads, ref_grads, before, before_ref = _full_check(name, layers, "bf16", opt=True)
    ref_after = dict(gm_ref.named_parameters())
    worst_w, worst_u = ("", 0.0), ("", 0.0)
    for n, rec in ex.params.items():
        if n not in ref_grads:                        # a parameter the program never reads (LayerNorm affine)
            continue
        new, old, new_ref = rec["master"], before[n], ref_after[n].detach()
        torch.testing.assert_close(old.cpu(), before_ref[n], rtol=0, atol=0)
        # the update is torch.optim.Adam's on the GPU's own gradients ...
        twin = old.clone().requires_grad_(True)
        twin.grad = grads[n]
        torch.optim.Adam([twin], lr=lr).step()
        torch.testing.assert_close(new, twin.detach(), rtol=1e-5, atol=1e-8)
        # ... the bf16 shadow that the next step reads is the rounded master ...
        torch.testing.assert_close(rec["shadow"], new.to(torch.bfloat16), rtol=0, atol=0)
        # ... and it agrees with the oracle's.  Adam's first step is -lr * sign(g) (up to eps): where the oracle's
        # gradient is zero up to rounding (the key bias of softmax attention, embedding rows of absent tokens) the
        # sign is noise on both sides, so those elements are left out: an element counts when its gradient is above a
        # hundredth of the tensor's largest and above 8 times the root-mean-square difference between the two runs'
        # gradients of this tensor (the tolerance on gradients allows 2e-2 of the norm; deep in a 24-layer backward
        # pass the runs are 1-2e-2 apart, and a smaller element's sign can differ)
        g_ref = ref_grads[n].float()
        apart = (grads[n].cpu().float() - g_ref).pow(2).mean().sqrt()
        clear = g_ref.abs() > torch.maximum(1e-2 * g_ref.abs().max(), 8 * apart)
        if not clear.any():
            continue
        new_c, ref_c = new.cpu()[clear], new_ref[clear]
        err = rel_err(new_c, ref_c)
        if err > worst_w[1]:
            worst_w = (n, err)
        assert err < 2e-2, (n, err)
        du, du_ref = new_c - old.cpu()[clear], ref_c - before_ref[n][clear]
        err_u = rel_err(du, du_ref)
        if err_u > worst_u[1]:
            worst_u = (n, err_u)
        assert err_u < 2e-2, (n, err_u)
        assert (du.abs() - lr).abs().max() < 0.02 * lr, n
    print("    after one Adam step: worst weight error", worst_w, "worst update error", worst_u)


def test_bert_large_shard_full_depth_bf16_adam_step(cuda):
    """All 24 layers of benchmark configuration 2 (bench.py --workload bert) with one Adam step: loss, gradients and updated weights."""
    _full_check_with_adam_step("bert", 24)


def test_vit_large_shard_full_depth_bf16_adam_step(cuda):
    """All 24 layers of benchmark configuration 3 (bench.py --workload vit: ViT-L/16, 48 of 128 images) with one Adam
    step: loss, gradients, updated masters and their bf16 shadows."""
    _full_check_with_adam_step("vit", 24)


def test_moe_shard_full_depth_bf16_adam_step(cuda):
    """All 12 layers (six of them top-2 MoE layers, 5 of 16 experts local, C = 80) of benchmark configuration 4
    (bench.py --workload moe) in bf16 with one Adam step."""
    _full_check_with_adam_step("moe", 12)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_moe_shard_capacity_40(cuda, dtype):
    """Benchmark configuration 4 with the capacity factor 1.25 read literally: C = ceil(512 / 16 * 1.25) = 40 slots
    per expert (the reference's config.py:25-28 doubles the factor for models whose name ends in `moe`, which gives the
    80 of the other tests); two layers at full width.  At this shape nearly every second choice is dropped at either
    capacity (the reference queues them behind the sum of the expert's first-choice positions, models.py:486: 528 for 32
    first choices); at C = 40 some first choices of the busiest experts are dropped as well."""
    _full_check("moe", 2, dtype, capacity=40)


def test_vit_large_shard_full_width_bf16(cuda):
    _full_check("vit", 1, "bf16")


def test_moe_shard_full_width_fp32(cuda):
    _full_check("moe", 2, "fp32")


def test_moe_shard_full_width_bf16(cuda):
    """Benchmark configuration 4 (bench.py --workload moe) in its own element type (routing: bit-exact on the GPU's own float32 logits; against the
    float32 oracle only tokens with a near-tie may differ, and they are counted)."""
    _full_check("moe", 2, "bf16")
