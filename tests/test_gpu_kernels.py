"""Single-kernel parity through the C ABI against stock PyTorch on the CPU (the library routines the emitted
program calls in the reference: F.linear, F.layer_norm, softmax, log_softmax + nll_loss, F.embedding, relu,
torch.optim).  Tolerances: float32 rtol 1e-4; bfloat16 rtol 2e-2 (inputs are rounded to bf16 on both sides)."""
import math

import numpy as np

import pytest
import torch
import torch.nn.functional as F

from hap_amd import ops
from helpers import rel_err

pytestmark = pytest.mark.gpu
DT = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def close(got, want, dtype, scale=1.0):
    got, want = got.float().cpu(), want.float()
    tol = TOL[dtype] * scale
    assert rel_err(got, want) < tol, rel_err(got, want)
    torch.testing.assert_close(got, want, rtol=tol, atol=tol * max(want.abs().max().item(), 1e-6))


GEMM_SHAPES = [(128, 128, 64), (384, 768, 512), (100, 52, 72), (257, 136, 200), (33, 1000, 96), (64, 16, 768),
               (512, 264, 1096)]


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("tA,tB", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_layouts_and_ragged_edges(cuda, dtype, tA, tB, M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    epv = 4 if dtype == torch.float32 else 8
    if (tA and M % epv) or ((not tA) and K % epv) or (tB and K % epv) or ((not tB) and N % epv):
        pytest.skip("leading dimension must be a multiple of the vector width")
    A = torch.randn((K, M) if tA else (M, K), generator=g).to(dtype)
    B = torch.randn((N, K) if tB else (K, N), generator=g).to(dtype)
    bias = torch.randn(N, generator=g)
    ldc = (N + 3) // 4 * 4
    C = torch.zeros(M, ldc, dtype=dtype, device=cuda)
    ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=bool(tA), transB=bool(tB), ldc=ldc, bias=bias.to(cuda))
    opA = A.double().t() if tA else A.double()
    opB = B.double().t() if tB else B.double()
    want = opA @ opB + bias.double()
    close(C[:, :N], want, dtype)
    assert (C[:, N:] == 0).all()


@pytest.mark.parametrize("dtype", DT)
def test_gemm_epilogue_accumulate_alpha_act_batch(cuda, dtype):
    g = torch.Generator().manual_seed(2)
    b1, b2, M, N, K = 3, 2, 40, 24, 64
    A = torch.randn(b1, b2, M, K, generator=g).to(dtype)
    B = torch.randn(b1, b2, K, N, generator=g).to(dtype)
    C0 = torch.randn(b1, b2, M, N, generator=g)
    C = C0.clone().to(cuda)                                   # float32 output from either input type
    ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, alpha=0.5, accumulate=True, batch1=b1, batch2=b2,
             strideA=(b2 * M * K, M * K), strideB=(b2 * K * N, K * N), strideC=(b2 * M * N, M * N))
    close(C, C0.double() + 0.5 * (A.double() @ B.double()), dtype)
    for act, fn in (("relu", torch.relu), ("gelu", F.gelu)):
        out = torch.empty(M, N, dtype=dtype, device=cuda)
        ops.gemm(A[0, 0].to(cuda), B[0, 0].to(cuda), out, M, N, K, act=act)
        close(out, fn(A[0, 0].double() @ B[0, 0].double()), dtype)


def test_gemm_refuses_misaligned(cuda):
    from hap_amd._lib import HapmiError
    a = torch.zeros(8, 10, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(HapmiError):
        ops.gemm(a, a, torch.zeros(8, 8, dtype=torch.bfloat16, device=cuda), 8, 8, 10, transB=True)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,width", [(384, 512), (37, 768), (5, 1024), (9, 100), (3, 2048), (4, 520), (6, 1030), (7, 1032), (2, 8)])
def test_add_layernorm_forward_backward(cuda, dtype, rows, width):
    g = torch.Generator().manual_seed(rows)
    x, r = torch.randn(rows, width, generator=g).to(dtype), torch.randn(rows, width, generator=g).to(dtype)
    dy = torch.randn(rows, width, generator=g).to(dtype)
    y = torch.empty(rows, width, dtype=dtype, device=cuda)
    rstd = torch.empty(rows, dtype=torch.float32, device=cuda)
    ops.add_layernorm_fwd(x.to(cuda), r.to(cuda), y, rstd)
    s = (x + r).double().requires_grad_(True)                 # the sum is rounded to the storage type first
    want = F.layer_norm(s, (width,))
    close(y, want.detach(), dtype)
    dx = torch.empty_like(y)
    ops.layernorm_bwd(dy.to(cuda), y, rstd, None, dx)
    want.backward(dy.double())
    close(dx, s.grad, dtype)
    dx2 = torch.empty_like(y)
    ops.layernorm_bwd(dy.to(cuda), y, rstd, dy.to(cuda), dx2)
    close(dx2, s.grad + dy.double(), dtype)
    # without a residual
    ops.add_layernorm_fwd(x.to(cuda), None, y, rstd)
    close(y, F.layer_norm(x.double(), (width,)), dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("S,ld", [(128, 128), (197, 200), (16, 16), (512, 512)])
def test_softmax_with_mask_forward_backward(cuda, dtype, S, ld):
    g = torch.Generator().manual_seed(S)
    rows = 3 * S
    x = torch.randn(rows, ld, generator=g).to(dtype)
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1)
    p = x.clone().to(cuda)
    ops.softmax_fwd(p, mask.to(cuda), p, rows, S, ld, S)
    want = torch.softmax(x[:, :S].double().view(3, S, S) + mask.double(), dim=-1).view(rows, S)
    close(p[:, :S], want, dtype)
    assert torch.equal(p[:, S:].cpu(), x[:, S:])              # pad columns untouched
    assert (p[:, :S].cpu().view(3, S, S).triu(1) == 0).all()   # causal: nothing above the diagonal
    dp = torch.randn(rows, ld, generator=g).to(dtype)
    ds = dp.clone().to(cuda)
    ops.softmax_bwd(ds, p, ds, rows, S, ld)
    pw = p[:, :S].double().cpu()
    wantd = pw * (dp[:, :S].double() - (dp[:, :S].double() * pw).sum(-1, keepdim=True))
    close(ds[:, :S], wantd, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,V,ld", [(24, 33280, 33280), (17, 30522, 30528), (8, 1000, 1000), (5, 97, 100)])
def test_logsoftmax_nll_and_gradient(cuda, dtype, rows, V, ld):
    g = torch.Generator().manual_seed(V)
    logits = (torch.randn(rows, ld, generator=g) * 3).to(dtype)
    tgt = torch.randint(0, V, (rows,), generator=g)
    tgt[::3] = -100
    row_loss = torch.empty(rows, dtype=torch.float32, device=cuda)
    loss = torch.empty(1, dtype=torch.float32, device=cuda)
    buf = logits.clone().to(cuda)
    ops.logsoftmax_nll(buf, tgt.to(cuda), row_loss, buf, rows, V, ld)
    ops.sum_f32(row_loss, loss)
    x = logits[:, :V].double().requires_grad_(True)
    want = F.nll_loss(torch.log_softmax(x, dim=1), tgt, reduction="sum")
    want.backward()
    assert abs(loss.item() - want.item()) <= 1e-5 * abs(want.item())
    close(buf[:, :V], x.grad, dtype)
    assert (buf[::3, :V] == 0).all()


@pytest.mark.parametrize("dtype", DT)
def test_embedding_forward_backward(cuda, dtype):
    g = torch.Generator().manual_seed(1)
    V, d, n, S = 211, 48, 60, 20
    table = torch.randn(V, d, generator=g).to(dtype)
    pe = torch.randn(S, d, generator=g).to(dtype)
    ids = torch.randint(0, V, (n,), generator=g)
    ids[5] = ids[6] = ids[7]                                    # collisions in the scatter-add
    out = torch.empty(n, d, dtype=dtype, device=cuda)
    ops.embedding_fwd(ids.to(cuda), table.to(cuda), pe.to(cuda), out, S, math.sqrt(d))
    want = (F.embedding(ids, table) * math.sqrt(d)).float() + pe.float()[torch.arange(n) % S]
    close(out, want, dtype)
    plain = torch.empty(n, d, dtype=dtype, device=cuda)
    ops.embedding_fwd(ids.to(cuda), table.to(cuda), None, plain, 1, 1.0)
    assert torch.equal(plain.cpu(), F.embedding(ids, table))       # a pure row gather is exact
    dout = torch.randn(n, d, generator=g).to(dtype)
    dt = torch.zeros(V, d, dtype=torch.float32, device=cuda)
    ops.embedding_bwd(ids.to(cuda), dout.to(cuda), dt, 1.0)
    wantg = torch.zeros(V, d, dtype=torch.float64).index_add_(0, ids, dout.double())
    close(dt, wantg, torch.float32)


def test_embedding_backward_rows_wider_than_one_wave_holds(cuda):
    """Rows wider than the 2048 columns a wave keeps in registers are cut into column blocks; bf16 gradients of
    repeated ids are added in token order (bit-exact against the same order on the CPU)."""
    g = torch.Generator().manual_seed(2)
    V, d, n = 37, 2048 * 2 + 72, 150
    ids = torch.randint(0, V, (n,), generator=g)
    dout = torch.randn(n, d, generator=g).bfloat16()
    dt = torch.zeros(V, d, dtype=torch.float32, device=cuda)
    ops.embedding_bwd(ids.to(cuda), dout.to(cuda), dt, 1.0)
    want = torch.zeros(V, d, dtype=torch.float32)
    for t in range(n):
        want[ids[t]] += dout[t].float()
    assert torch.equal(dt.cpu(), want)


@pytest.mark.parametrize("dtype", DT)
def test_elementwise_and_reductions(cuda, dtype):
    g = torch.Generator().manual_seed(4)
    n = 4099
    a, b = torch.randn(n, generator=g).to(dtype), torch.randn(n, generator=g).to(dtype)
    da, db = a.to(cuda), b.to(cuda)
    out = torch.empty_like(da)
    ops.add(da, db, out)
    assert torch.equal(out.cpu(), a + b)
    ops.scale(da, 1.5, out)
    assert torch.equal(out.cpu(), (a.float() * 1.5).to(dtype))
    ops.act_fwd(da, out, "relu")
    assert torch.equal(out.cpu(), torch.relu(a))
    y = out.clone()
    ops.act_bwd(db, y, out, "relu")
    assert torch.equal(out.cpu(), torch.where(a > 0, b, torch.zeros_like(b)))
    ops.act_fwd(da, out, "gelu")
    close(out, F.gelu(a.double()), dtype)
    ops.act_bwd(db, da, out, "gelu")
    ad = a.double().requires_grad_(True)
    F.gelu(ad).backward(b.double())
    close(out, ad.grad, dtype)
    x = torch.randn(300, 72, generator=g).to(dtype)
    cs = torch.empty(72, dtype=torch.float32, device=cuda)
    ops.colsum(x.to(cuda), cs, 300, 72)
    close(cs, x.double().sum(0), torch.float32)
    ops.colsum(x.to(cuda), cs, 300, 72, accumulate=True)
    close(cs, 2 * x.double().sum(0), torch.float32)
    big, small = torch.randn(6, 5, 8, generator=g).to(dtype), torch.randn(1, 5, 8, generator=g).to(dtype)
    o3 = torch.empty(6, 5, 8, dtype=dtype, device=cuda)
    ops.add_bcast_rows(big.to(cuda), small.to(cuda), o3, 30, 5, 8)
    assert torch.equal(o3.cpu(), big + small)


def test_patchify_and_cls_pos(cuda):
    g = torch.Generator().manual_seed(6)
    b, C, gh, gw, ph, pw, d = 3, 3, 4, 5, 4, 2, 16
    x = torch.randn(b, C, gh * ph, gw * pw, generator=g)
    w = torch.randn(d, C, ph, pw, generator=g)
    cols = torch.empty(b * gh * gw, C * ph * pw, dtype=torch.float32, device=cuda)
    ops.patchify(x.to(cuda), cols, b, C, gh, gw, ph, pw)
    got = cols.cpu() @ w.view(d, -1).t()
    want = torch.flatten(F.conv2d(x, w, None, (ph, pw)), 2).transpose(1, 2).reshape(b * gh * gw, d)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    T = gh * gw
    patches, cls, pos = torch.randn(b, T, d, generator=g), torch.randn(1, 1, d, generator=g), torch.randn(1, T + 1, d, generator=g)
    out = torch.empty(b, T + 1, d, device=cuda)
    ops.append_cls_pos(patches.to(cuda), cls.to(cuda), pos.to(cuda), out, b, T, d)
    assert torch.equal(out.cpu(), torch.cat((cls.expand(b, -1, -1), patches), dim=1) + pos)


def test_optimizers_match_torch(cuda):
    g = torch.Generator().manual_seed(8)
    n = 1003
    p0 = torch.randn(n, generator=g)
    grads = [torch.randn(n, generator=g) for _ in range(3)]
    # SGD
    ref = p0.clone().requires_grad_(True)
    opt = torch.optim.SGD([ref], lr=1e-3)
    p = p0.clone().to(cuda)
    for gr in grads:
        ref.grad = gr.clone()
        opt.step()
        ops.sgd_step(p, gr.to(cuda), None, 1e-3)
    torch.testing.assert_close(p.cpu(), ref.detach(), rtol=1e-6, atol=1e-7)
    # Adam with a bf16 shadow
    ref = p0.clone().requires_grad_(True)
    opt = torch.optim.Adam([ref], lr=5e-4)
    p, m, v = p0.clone().to(cuda), torch.zeros(n, device=cuda), torch.zeros(n, device=cuda)
    sh = torch.empty(n, dtype=torch.bfloat16, device=cuda)
    for i, gr in enumerate(grads):
        ref.grad = gr.clone()
        opt.step()
        ops.adam_step(p, gr.to(cuda), m, v, sh, 5e-4, 0.9, 0.999, 1e-8, i + 1)
    torch.testing.assert_close(p.cpu(), ref.detach(), rtol=1e-5, atol=1e-7)
    assert torch.equal(sh.cpu(), p.cpu().bfloat16())
    # first Adam step is -lr * sign(g) up to eps
    p1, m1, v1 = torch.zeros(n, device=cuda), torch.zeros(n, device=cuda), torch.zeros(n, device=cuda)
    ops.adam_step(p1, grads[0].to(cuda), m1, v1, None, 5e-4, 0.9, 0.999, 1e-8, 1)
    torch.testing.assert_close(p1.cpu(), -5e-4 * torch.sign(grads[0]), rtol=1e-4, atol=1e-9)
    # gradient clipping coefficient (clip_grad_norm_)
    ss, coef = torch.full((1,), 7.0, device=cuda), torch.zeros(1, device=cuda)     # the old content is overwritten
    ops.sumsq(grads[0].to(cuda), ss)
    ops.clip_coef(ss, 0.5, coef)
    want = min(1.0, 0.5 / (grads[0].norm().item() + 1e-6))
    assert abs(coef.item() - want) < 1e-6 * want


@pytest.mark.parametrize("cfg", list(range(10)))
@pytest.mark.parametrize("tA,tB", [(0, 1), (0, 0), (1, 0), (1, 1)])
def test_gemm_every_tile_configuration_and_layout(cuda, cfg, tA, tB):
    """bf16 operands in all four storage layouts through every tile configuration: a shape with ragged edges in
    M, N and K (several tiles of the small configurations, one partial tile of the large ones) and a tile-aligned
    one, bf16 and float32 outputs, bias and accumulation."""
    from hap_amd._lib import lib
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        for (M, N, K) in [(424, 520, 1000), (768, 512, 256)]:
            g = torch.Generator().manual_seed(M + cfg)
            A = torch.randn((K, M) if tA else (M, K), generator=g).bfloat16()
            B = torch.randn((N, K) if tB else (K, N), generator=g).bfloat16()
            bias = torch.randn(N, generator=g)
            opA = A.double().t() if tA else A.double()
            opB = B.double().t() if tB else B.double()
            want = opA @ opB + bias.double()
            for out_dtype in (torch.bfloat16, torch.float32):
                C = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
                ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=bool(tA), transB=bool(tB), bias=bias.to(cuda))
                close(C, want, torch.bfloat16)
            start = torch.randn(M, N, generator=g)
            C = start.clone().to(cuda)
            ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=bool(tA), transB=bool(tB), accumulate=True)
            close(C, want - bias.double() + start.double(), torch.bfloat16)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("cfg", [0, 1, 7])
@pytest.mark.parametrize("act", ["none", "relu", "gelu"])
def test_gemm_scale_bias_activation_in_every_epilogue(cuda, cfg, act):
    """alpha, bias and activation applied by the epilogue, bf16 and float32 outputs, with and without bias, ragged
    and tile-aligned shapes."""
    from hap_amd._lib import lib
    fn = {"none": lambda t: t, "relu": torch.relu, "gelu": torch.nn.functional.gelu}[act]
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        for (M, N, K) in [(424, 520, 328), (512, 512, 128)]:
            g = torch.Generator().manual_seed(M + cfg)
            A = torch.randn(M, K, generator=g).bfloat16()
            B = torch.randn(N, K, generator=g).bfloat16()
            bias = torch.randn(N, generator=g)
            for with_bias in (True, False):
                for alpha in (1.0, 0.25):
                    want = alpha * (A.double() @ B.double().t())
                    if with_bias:
                        want = want + bias.double()
                    want = fn(want)
                    for out_dtype in (torch.bfloat16, torch.float32):
                        C = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
                        ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transB=True, alpha=alpha,
                                 bias=bias.to(cuda) if with_bias else None, act=act if act != "none" else None)
                        close(C, want, torch.bfloat16)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("cfg", [0, 10, 11])
@pytest.mark.parametrize("tA,tB", [(0, 1), (0, 0), (1, 0), (1, 1)])
def test_gemm_float32_tile_configurations_and_layouts(cuda, cfg, tA, tB):
    """float32 operands in all four storage layouts through the three tile configurations that take them (128 x 128
    and the small 64 x 64 / 64 x 128 tiles): ragged edges in M, N and K and a tile-aligned shape, float32 and bf16
    outputs, bias and accumulation, against float64."""
    from hap_amd._lib import lib
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        for (M, N, K) in [(200, 136, 300), (384, 512, 256)]:
            g = torch.Generator().manual_seed(M + cfg)
            A = torch.randn((K, M) if tA else (M, K), generator=g)
            B = torch.randn((N, K) if tB else (K, N), generator=g)
            bias = torch.randn(N, generator=g)
            want = (A.double().t() if tA else A.double()) @ (B.double().t() if tB else B.double()) + bias.double()
            for out_dtype in (torch.float32, torch.bfloat16):
                C = torch.full((M, N), float("nan"), dtype=out_dtype, device=cuda)
                ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=bool(tA), transB=bool(tB), bias=bias.to(cuda))
                close(C, want, out_dtype)
            start = torch.randn(M, N, generator=g)
            C = start.clone().to(cuda)
            ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=bool(tA), transB=bool(tB), accumulate=True)
            close(C, want - bias.double() + start.double(), torch.float32)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("cfg", [0, 1, 10, 11])
def test_gemm_split_k_and_tile_configs(cuda, dtype, cfg):
    """Forced tile configuration and K splits (workspace partial sums + ordered reduction) give the same product."""
    from hap_amd._lib import lib
    g = torch.Generator().manual_seed(5)
    M, N, K = 200, 136, 2048
    A = torch.randn(K, M, generator=g).to(dtype)
    B = torch.randn(K, N, generator=g).to(dtype)
    bias = torch.randn(N, generator=g)
    C0 = torch.randn(M, N, generator=g)
    ws = torch.empty(8 * M * N, dtype=torch.float32, device=cuda)
    want = A.double().t() @ B.double() + bias.double()
    try:
        for splits in (1, 3, 8):
            lib().hapmi_gemm_tuning(cfg, splits)
            C = C0.clone().to(cuda)
            ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=True, bias=bias.to(cuda), accumulate=True, workspace=ws)
            close(C, want + C0.double(), dtype)
            out = torch.empty(M, N, dtype=dtype, device=cuda)
            ops.gemm(A.to(cuda), B.to(cuda), out, M, N, K, transA=True, bias=bias.to(cuda), act="relu", workspace=ws)
            close(out, torch.relu(want), dtype)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("dtype,cfg", [(torch.float32, 0), (torch.float32, 10), (torch.float32, 11), (torch.bfloat16, 0), (torch.bfloat16, 1), (torch.bfloat16, 2),
                                       (torch.bfloat16, 3), (torch.bfloat16, 4), (torch.bfloat16, 5), (torch.bfloat16, 6), (torch.bfloat16, 7), (torch.bfloat16, 8), (torch.bfloat16, 9)])
@pytest.mark.parametrize("tB", [False, True])
def test_gemm_row_sums_of_a_transposed_operand(cuda, dtype, cfg, tB):
    """a_rowsum: the weight-gradient call dW = dY^T X also returns the column sums of dY (the bias gradient),
    added into a caller-cleared float32 vector -- for every tile configuration, with and without K splits,
    ragged M / N / K, on top of earlier contents."""
    from hap_amd._lib import lib
    g = torch.Generator().manual_seed(11 + cfg)
    M, N, K = 328, 520, 1000                                   # not multiples of any tile; K not a multiple of 64
    A = torch.randn(K, M, generator=g).to(dtype)
    B = (torch.randn(N, K, generator=g) if tB else torch.randn(K, N, generator=g)).to(dtype)
    start = torch.randn(M, generator=g)
    want_c = A.double().t() @ (B.double().t() if tB else B.double())
    want_rs = start.double() + A.double().sum(0)
    ws = torch.empty(8 * M * 520, dtype=torch.float32, device=cuda)
    try:
        for splits in (1, 4):
            lib().hapmi_gemm_tuning(cfg, splits)
            C = torch.empty(M, N, dtype=torch.float32, device=cuda)
            rs = start.clone().to(cuda)
            ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transA=True, transB=tB, workspace=ws, a_rowsum=rs)
            close(C, want_c, dtype)
            tol = 1e-5 if dtype == torch.float32 else 1e-4       # float32 sums of exactly represented inputs
            torch.testing.assert_close(rs.cpu().double(), want_rs, rtol=tol, atol=tol * K ** 0.5)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)
    with pytest.raises(Exception):
        ops.gemm(A.t().contiguous().to(cuda), B.to(cuda), C, M, N, K, transA=False, transB=tB, a_rowsum=rs)


@pytest.mark.parametrize("dtype,out_dtype,cfg,splits,accumulate", [
    (torch.bfloat16, torch.bfloat16, 0, 1, False), (torch.bfloat16, torch.bfloat16, 1, 1, False),
    (torch.bfloat16, torch.bfloat16, 3, 1, False), (torch.bfloat16, torch.bfloat16, 0, 4, False),
    (torch.bfloat16, torch.bfloat16, 0, 1, True), (torch.bfloat16, torch.float32, 5, 1, False),
    (torch.float32, torch.float32, 0, 1, False), (torch.float32, torch.float32, 0, 4, True)])
@pytest.mark.parametrize("shape", [(256, 512, 192), (328, 520, 1000)])
def test_gemm_relu_mask_on_the_result(cuda, dtype, out_dtype, cfg, splits, accumulate, shape):
    """c_relu_mask: C = (mask > 0) * (A B) (+ C): the relu backward of the tensor whose gradient the call computes,
    in every store path (16-byte bf16 stores, float32 staging, split-K reduction, accumulation, ragged edges)."""
    from hap_amd._lib import lib
    M, N, K = shape
    g = torch.Generator().manual_seed(M + cfg + splits)
    A = torch.randn(M, K, generator=g).to(dtype)
    B = torch.randn(K, N, generator=g).to(dtype)
    mask = torch.relu(torch.randn(M, N, generator=g)).to(out_dtype)         # a relu output: zeros and positives
    start = torch.randn(M, N, generator=g).to(out_dtype)
    want = (A.double() @ B.double()) * (mask > 0)
    if accumulate:
        want = want + start.double()
    ws = torch.empty(8 * M * 520, dtype=torch.float32, device=cuda)
    try:
        lib().hapmi_gemm_tuning(cfg, splits)
        C = start.clone().to(cuda)
        ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, workspace=ws, accumulate=accumulate, relu_mask=mask.to(cuda))
        close(C, want, dtype if out_dtype == torch.float32 else out_dtype)
        assert (C.cpu()[mask == 0] == (start[mask == 0] if accumulate else 0)).all()
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("dtype", DT)
def test_gemm_relu_mask_with_a_batch(cuda, dtype):
    """c_relu_mask next to batch strides: problem z's mask lies at C's offset of problem z (the expert FFN's data
    gradient: every local expert is one problem)."""
    g = torch.Generator().manual_seed(9)
    E, M, N, K = 3, 136, 72, 200
    A = torch.randn(E, M, K, generator=g).to(dtype)
    B = torch.randn(E, N, K, generator=g).to(dtype)
    mask = torch.relu(torch.randn(E, M, N, generator=g)).to(dtype)
    C = torch.empty(E, M, N, dtype=dtype, device=cuda)
    ops.gemm(A.to(cuda), B.to(cuda), C, M, N, K, transB=True, batch1=E, strideA=(M * K, 0), strideB=(N * K, 0),
             strideC=(M * N, 0), relu_mask=mask.to(cuda))
    want = torch.einsum("emk,enk->emn", A.double(), B.double()) * (mask > 0)
    close(C, want, dtype)
    assert (C.cpu()[mask == 0] == 0).all()


@pytest.mark.parametrize("dtype,out_dtype,cfg,splits", [
    (torch.bfloat16, torch.bfloat16, 0, 1), (torch.bfloat16, torch.bfloat16, 7, 1), (torch.bfloat16, torch.float32, 5, 1),
    (torch.bfloat16, torch.bfloat16, 1, 3), (torch.float32, torch.float32, 0, 1), (torch.float32, torch.float32, 0, 2)])
@pytest.mark.parametrize("shape", [(256, 512, 192), (328, 520, 1000)])
def test_gemm_accumulates_onto_a_separate_addend(cuda, dtype, out_dtype, cfg, splits, shape):
    """c_addend: C = addend + A B with C only written, bit-equal to accumulating in place into a copy of the
    addend, in every store path; the addend itself is left untouched."""
    from hap_amd._lib import lib
    M, N, K = shape
    g = torch.Generator().manual_seed(M + cfg + splits)
    A = torch.randn(M, K, generator=g).to(dtype).to(cuda)
    B = torch.randn(K, N, generator=g).to(dtype).to(cuda)
    R = torch.randn(M, N, generator=g).to(out_dtype).to(cuda)
    ws = torch.empty(8 * M * 520, dtype=torch.float32, device=cuda)
    try:
        lib().hapmi_gemm_tuning(cfg, splits)
        in_place = R.clone()
        ops.gemm(A, B, in_place, M, N, K, workspace=ws, accumulate=True)
        keep = R.clone()
        C = torch.full((M, N), 7.0, dtype=out_dtype, device=cuda)
        ops.gemm(A, B, C, M, N, K, workspace=ws, accumulate=True, addend=R)
        assert torch.equal(C, in_place) and torch.equal(R, keep)
        close(C, A.double().cpu() @ B.double().cpu() + keep.double().cpu(), dtype if out_dtype == torch.float32 else out_dtype)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)
    with pytest.raises(TypeError):
        ops.gemm(A, B, C, M, N, K, addend=R)                               # without accumulate


@pytest.mark.parametrize("cfg", [0, 1, 5, 6, 7, 9])
@pytest.mark.parametrize("n,accumulate", [(1, False), (3, True), (8, False), (16, False)])
def test_gemm_group_of_weight_gradients_behind_pointer_lists(cuda, cfg, n, accumulate):
    """A_list / B_list / C_list / a_rowsum_list: n weight gradients dW = dY^T X (+ column sums of dY) of one
    shape in one launch, bit-equal to n single launches of the same tile configuration, and close to float64."""
    from hap_amd._lib import lib
    rows, d_out, d_in = 520, 200, 328                                      # ragged against every tile size
    g = torch.Generator().manual_seed(cfg * 31 + n)
    dY = [torch.randn(rows, d_out, generator=g).bfloat16().to(cuda) for _ in range(n)]
    X = [torch.randn(rows, d_in, generator=g).bfloat16().to(cuda) for _ in range(n)]
    start = [torch.randn(d_out, d_in, generator=g).to(cuda) for _ in range(n)]
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        single, single_b = [t.clone() for t in start], [torch.zeros(d_out, device=cuda) for _ in range(n)]
        for z in range(n):
            ops.gemm(dY[z], X[z], single[z], d_out, d_in, rows, transA=True, accumulate=accumulate, a_rowsum=single_b[z])
        W, b = [t.clone() for t in start], [torch.zeros(d_out, device=cuda) if z != 1 else None for z in range(n)]
        ops.gemm_group(dY, X, W, d_out, d_in, rows, transA=True, accumulate=accumulate, a_rowsums=b)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)
    for z in range(n):
        assert torch.equal(W[z], single[z]), z
        want = dY[z].double().t() @ X[z].double() + (start[z].double() if accumulate else 0)
        close(W[z], want.cpu(), torch.bfloat16)
        if b[z] is not None:
            torch.testing.assert_close(b[z].cpu(), dY[z].float().sum(0).cpu(), rtol=1e-4, atol=1e-3)
    with pytest.raises(ValueError):
        ops.gemm_group(dY * 17, X * 17, W * 17, d_out, d_in, rows, transA=True)


def test_gemm_group_float32_and_plain_layout(cuda):
    g = torch.Generator().manual_seed(5)
    A = [torch.randn(70, 96, generator=g).to(cuda) for _ in range(4)]
    B = [torch.randn(40, 96, generator=g).to(cuda) for _ in range(4)]
    C = [torch.empty(70, 40, device=cuda) for _ in range(4)]
    ops.gemm_group(A, B, C, 70, 40, 96, transB=True, alpha=0.5)
    for z in range(4):
        torch.testing.assert_close(C[z].cpu(), 0.5 * (A[z].double() @ B[z].double().t()).float().cpu(), rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("S,causal", [(16, True), (128, True), (197, False), (512, False), (200, True), (64, False),
                                      (16, "flag"), (128, "flag"), (200, "flag"), (512, "flag"), (129, "flag")])
def test_fused_attention_forward_backward(cuda, S, causal):
    """Fused bf16 attention against the explicit softmax(QK^T * scale + mask) V of
    F.multi_head_attention_forward, computed in float64 from the same bf16 inputs.  causal = True hands the
    kernels the additive mask, "flag" the causal flag instead (no mask read, key tiles above the diagonal skipped)."""
    g = torch.Generator().manual_seed(S)
    b, H, hd = 2, 3, 64
    E = H * hd
    qkv = torch.randn(b, S, 3 * E, generator=g).bfloat16()
    dout = torch.randn(b, S, E, generator=g).bfloat16()
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1) if causal else None
    scale = 1.0 / math.sqrt(hd)
    out = torch.empty(b, S, E, dtype=torch.bfloat16, device=cuda)
    lse = torch.empty(b, H, S, dtype=torch.float32, device=cuda)
    dq = qkv.to(cuda)
    flag = causal == "flag"
    dmask = mask.to(cuda) if causal is True else None
    ops.attention_fwd(dq, dmask, out, lse, b, S, H, scale, causal=flag)
    x = qkv.double().requires_grad_(True)
    q, k, v = [t.view(b, S, H, hd).transpose(1, 2) for t in x.split(E, dim=2)]
    sc = q @ k.transpose(-1, -2) * scale
    if causal:
        sc = sc + mask.double()
    want = (torch.softmax(sc, -1) @ v).transpose(1, 2).reshape(b, S, E)
    close(out, want.detach(), torch.bfloat16)
    torch.testing.assert_close(lse.cpu(), torch.logsumexp(sc, -1).float().detach(), rtol=1e-3, atol=1e-3)
    want.backward(dout.double())
    dqkv = torch.full((b, S, 3 * E), float("nan"), dtype=torch.bfloat16, device=cuda)
    delta = torch.empty(b, H, S, dtype=torch.float32, device=cuda)
    ops.attention_bwd(dq, out, dout.to(cuda), lse, dmask, dqkv, delta, b, S, H, scale, causal=flag)
    for name, got, ref in zip("qkv", dqkv.float().cpu().split(E, dim=2), x.grad.split(E, dim=2)):
        assert rel_err(got, ref) < 2e-2, (name, rel_err(got, ref))


def _keep_words_to_masks(keep_rows, keep_cols, b, H, S):
    """Unpacks the two bit-word layouts of attention_keep_bits into bool [b*H, S(q), S(k)] tensors."""
    n_kt = (S + 63) // 64
    rows = keep_rows.cpu().numpy().astype(np.uint32).reshape(b * H, S, n_kt, 2)
    cols = keep_cols.cpu().numpy().astype(np.uint32).reshape(b * H, S, 2 * n_kt)
    k = np.arange(n_kt * 64)
    kt, t, g, h, e = k // 64, (k // 32) % 2, (k // 8) % 4, (k // 4) % 2, k % 4
    from_rows = ((rows[:, :, kt, h] >> (16 * t + 4 * g + e).astype(np.uint32)) & 1).astype(bool)[:, :, :S]
    q = np.arange(S)
    from_cols = ((cols[:, :, q // 32] >> (q % 32).astype(np.uint32)) & 1).astype(bool)       # [bh, k, q]
    return torch.from_numpy(from_rows), torch.from_numpy(from_cols).transpose(1, 2)


@pytest.mark.parametrize("S", [1, 16, 64, 65, 129, 197, 512])
def test_attention_keep_words_are_the_dropout_kernels_decisions(cuda, S):
    """Both bit layouts of attention_keep_bits hold exactly the decisions that the dropout kernel takes for a
    [b*H, S, row_len] tensor of probabilities under the same state and stream id (bit-exact)."""
    b, H, p, sid = 2, 3, 0.25, 11
    Sp = (S + 7) // 8 * 8
    state = torch.tensor([1234, 5], dtype=torch.int64, device=cuda)
    n = ops.attention_keep_words(b, S, H)
    kr = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    kc = torch.full((n,), -1, dtype=torch.int32, device=cuda)
    ops.attention_keep_bits(kr, kc, b, S, H, Sp, p, state, sid)
    want = ops.dropout_mask(b * H * S * Sp, p, state, sid).view(b * H, S, Sp)[:, :, :S].bool().cpu()
    got_rows, got_cols = _keep_words_to_masks(kr, kc, b, H, S)
    assert torch.equal(got_rows, want)
    assert torch.equal(got_cols, want)
    if S >= 16:
        assert 0.70 < want.float().mean().item() < 0.80
    # query bits beyond S inside a column's last word are zero
    n_kt = (S + 63) // 64
    cols = kc.cpu().numpy().astype(np.uint32).reshape(b * H, S, 2 * n_kt)
    qq = np.arange(S, n_kt * 64)
    if len(qq):
        assert not ((cols[:, :, qq // 32] >> (qq % 32).astype(np.uint32)) & 1).any()


@pytest.mark.parametrize("S,causal", [(8, False), (16, False), (64, True), (65, "flag"), (129, "flag"), (197, False),
                                      (512, False), (512, "flag"), (200, True)])
def test_fused_attention_with_dropout_of_the_probabilities(cuda, S, causal):
    """out = dropout(softmax(QK^T * scale + mask)) V (F.multi_head_attention_forward with dropout_p > 0) and its
    gradients, in float64 from the same bf16 inputs with the keep decisions of the dropout kernel."""
    g = torch.Generator().manual_seed(S + 1)
    b, H, hd, p, sid = 2, 3, 64, 0.2, 7
    E, Sp = H * hd, (S + 7) // 8 * 8
    qkv = torch.randn(b, S, 3 * E, generator=g).bfloat16()
    dout = torch.randn(b, S, E, generator=g).bfloat16()
    mask = torch.triu(torch.full((S, S), float("-inf")), diagonal=1) if causal else None
    scale = 1.0 / math.sqrt(hd)
    state = torch.tensor([99, 3], dtype=torch.int64, device=cuda)
    n = ops.attention_keep_words(b, S, H)
    kr = torch.empty(n, dtype=torch.int32, device=cuda)
    kc = torch.empty(n, dtype=torch.int32, device=cuda)
    ops.attention_keep_bits(kr, kc, b, S, H, Sp, p, state, sid)
    keep = ops.dropout_mask(b * H * S * Sp, p, state, sid).view(b, H, S, Sp)[..., :S].bool().cpu()
    out = torch.empty(b, S, E, dtype=torch.bfloat16, device=cuda)
    lse = torch.empty(b, H, S, dtype=torch.float32, device=cuda)
    dq = qkv.to(cuda)
    flag = causal == "flag"
    dmask = mask.to(cuda) if causal is True else None
    ops.attention_fwd(dq, dmask, out, lse, b, S, H, scale, causal=flag, keep_rows=kr, p=p)
    x = qkv.double().requires_grad_(True)
    q, k, v = [t.view(b, S, H, hd).transpose(1, 2) for t in x.split(E, dim=2)]
    sc = q @ k.transpose(-1, -2) * scale
    if causal:
        sc = sc + mask.double()
    P = torch.softmax(sc, -1) * keep.double() / (1.0 - p)
    want = (P @ v).transpose(1, 2).reshape(b, S, E)
    close(out, want.detach(), torch.bfloat16)
    torch.testing.assert_close(lse.cpu(), torch.logsumexp(sc, -1).float().detach(), rtol=1e-3, atol=1e-3)
    want.backward(dout.double())
    dqkv = torch.full((b, S, 3 * E), float("nan"), dtype=torch.bfloat16, device=cuda)
    delta = torch.empty(b, H, S, dtype=torch.float32, device=cuda)
    ops.attention_bwd(dq, out, dout.to(cuda), lse, dmask, dqkv, delta, b, S, H, scale, causal=flag, keep_rows=kr,
                      keep_cols=kc, p=p)
    for name, got, ref in zip("qkv", dqkv.float().cpu().split(E, dim=2), x.grad.split(E, dim=2)):
        assert rel_err(got, ref) < 2e-2, (name, rel_err(got, ref))


def test_adam_with_device_step_state_matches_torch(cuda):
    """The graph-capturable Adam (step count and bias corrections advanced on the device)."""
    g = torch.Generator().manual_seed(21)
    n = 777
    p0 = torch.randn(n, generator=g)
    ref = p0.clone().requires_grad_(True)
    opt = torch.optim.Adam([ref], lr=5e-4)
    p, m, v = p0.clone().to(cuda), torch.zeros(n, device=cuda), torch.zeros(n, device=cuda)
    state = torch.zeros(4, device=cuda)
    for i in range(5):
        gr = torch.randn(n, generator=g)
        ref.grad = gr.clone()
        opt.step()
        ops.adam_step_dev(p, gr.to(cuda), m, v, None, 5e-4, 0.9, 0.999, 1e-8, state)
    torch.testing.assert_close(p.cpu(), ref.detach(), rtol=1e-5, atol=1e-7)
    assert state[0].item() == 5.0


def test_gemm_plans_round_trip_through_a_file(cuda, tmp_path):
    """Plans pinned by autotuning are written to and re-pinned from a JSON file."""
    from hap_amd._lib import lib
    M, N, K = 256, 384, 512
    A0, B0 = torch.randn(M, K).bfloat16(), torch.randn(N, K).bfloat16()
    A, B = A0.to(cuda), B0.to(cuda)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=cuda)
    ops.clear_gemm_plans()
    try:
        ops.record_gemms(True)
        ops.gemm(A, B, C, M, N, K, transB=True)
        (args, _keep), = ops.record_gemms(False)
        cfg, splits, _us = ops.autotune_gemm(args, None, repeats=1)
        path = str(tmp_path / "plans.json")
        assert ops.save_gemm_plans(path) == 1
        ops.clear_gemm_plans()
        assert ops.load_gemm_plans(path) == 1
        assert ops._pinned_plans[(M, N, K, 1, 0, 1, 1, 1)] == (cfg, splits)
        ops.gemm(A, B, C, M, N, K, transB=True)
        close(C, A0.double() @ B0.double().t(), torch.bfloat16)
    finally:
        ops.clear_gemm_plans()


def test_reductions_give_the_same_bits_every_time(cuda):
    """The reductions that many blocks share add in a fixed order (no float atomics): the embedding gradient, column
    sums over several slabs of rows, the gradient norm, and the bias gradient that a weight-gradient GEMM takes
    along (also with the reduction split over K and for several problems in one launch)."""
    g = torch.Generator().manual_seed(21)
    # embedding gradient with heavy collisions: equal to the token-ordered float32 sum, bit for bit
    V, d, n = 50, 200, 1500
    ids = torch.randint(0, 7, (n,), generator=g) * 7
    dout = torch.randn(n, d, generator=g)
    want = torch.zeros(V, d)
    for t in range(n):
        want[ids[t]] += dout[t]
    runs = []
    for _ in range(3):
        dt = torch.zeros(V, d, device=cuda)
        ops.embedding_bwd(ids.to(cuda), dout.to(cuda), dt, 1.0)
        runs.append(dt.cpu())
    assert torch.equal(runs[0], want)
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
    # column sums over 3000 rows (24 slabs) and the sum of squares of 1.3 M elements
    x = torch.randn(3000, 264, generator=g).to(cuda)
    big = torch.randn(1_300_003, generator=g).to(cuda)
    outs = []
    for _ in range(3):
        cs = torch.empty(264, device=cuda)
        ops.colsum(x, cs, 3000, 264)
        ss = torch.empty(1, device=cuda)
        ops.sumsq(big, ss)
        outs.append((cs.cpu(), ss.cpu()))
    torch.testing.assert_close(outs[0][0].double(), x.cpu().double().sum(0), rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(outs[0][1].double(), big.cpu().double().pow(2).sum().reshape(1), rtol=1e-6, atol=0)
    for o in outs[1:]:
        assert torch.equal(o[0], outs[0][0]) and torch.equal(o[1], outs[0][1])
    # bias gradient as row sums of dY in dW = dY^T X: one problem (with and without a K split), then a group
    for dtype in (torch.bfloat16, torch.float32):
        rows, n_out, n_in = 4096, 320, 256
        dy = torch.randn(rows, n_out, generator=g).to(dtype).to(cuda)
        xx = torch.randn(rows, n_in, generator=g).to(dtype).to(cuda)
        ref = dy.double().sum(0).cpu()
        for splits in (0, 4):
            ops.lib().hapmi_gemm_tuning(-1, splits)
            try:
                got = []
                for _ in range(3):
                    gw = torch.empty(n_out, n_in, device=cuda)
                    gb = torch.zeros(n_out, device=cuda)
                    ops.gemm(dy, xx, gw, n_out, n_in, rows, transA=True, a_rowsum=gb)
                    got.append((gw.cpu(), gb.cpu()))
            finally:
                ops.lib().hapmi_gemm_tuning(-1, 0)
            torch.testing.assert_close(got[0][1].double(), ref, rtol=1e-5, atol=1e-3)
            for o in got[1:]:
                assert torch.equal(o[0], got[0][0]) and torch.equal(o[1], got[0][1])
        dys = [torch.randn(rows, n_out, generator=g).to(dtype).to(cuda) for _ in range(3)]
        xs = [torch.randn(rows, n_in, generator=g).to(dtype).to(cuda) for _ in range(3)]
        got = []
        for _ in range(2):
            gws = [torch.empty(n_out, n_in, device=cuda) for _ in range(3)]
            gbs = [torch.zeros(n_out, device=cuda), None, torch.ones(n_out, device=cuda)]
            ops.gemm_group(dys, xs, gws, n_out, n_in, rows, transA=True, a_rowsums=gbs)
            got.append([t.cpu() for t in gws] + [gbs[0].cpu(), gbs[2].cpu()])
        torch.testing.assert_close(got[0][3].double(), dys[0].double().sum(0).cpu(), rtol=1e-5, atol=1e-3)
        torch.testing.assert_close(got[0][4].double(), 1 + dys[2].double().sum(0).cpu(), rtol=1e-5, atol=1e-3)
        for u, v in zip(got[0], got[1]):
            assert torch.equal(u, v)


def _pieces(full, lengths, cuda, wide_first=True):
    """Split a [rows, sum(lengths)] CPU tensor into GPU pieces: the first a row-range view of a wider, taller
    tensor (its leading dimension differs from its length, as the own piece of an all_to_all does), the others
    contiguous tensors of their own."""
    out, pos = [], 0
    for i, l in enumerate(lengths):
        part = full[:, pos:pos + l]
        if i == 0 and wide_first:
            host = torch.full((full.shape[0] + 5, l + 16), float("nan"), dtype=full.dtype)
            host[3:3 + full.shape[0], :l] = part
            out.append(host.to(cuda)[3:3 + full.shape[0], :l])
        else:
            out.append(part.contiguous().to(cuda))
        pos += l
    return out


@pytest.mark.parametrize("cfg", [-1, 5, 6, 7, 8, 9])
def test_gemm_a_in_pieces_along_k_with_relu(cuda, cfg):
    """The linear behind an all_to_all + relu reads the received pieces in place: A = relu(cat(pieces, dim 1))."""
    from hap_amd._lib import lib
    g = torch.Generator().manual_seed(31 + cfg)
    M, N, lengths = 300, 200, [384, 384, 128, 128]
    K = sum(lengths)
    act = torch.randn(M, K, generator=g).bfloat16()
    W = torch.randn(N, K, generator=g).bfloat16()
    bias = torch.randn(N, generator=g)
    pieces = _pieces(act, lengths, cuda)
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        for relu in (True, False):
            src = torch.relu(act.double()) if relu else act.double()
            want = src @ W.double().t() + bias.double()
            C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
            ops.gemm(None, W.to(cuda), C, M, N, K, transB=True, bias=bias.to(cuda), a_segments=pieces, a_relu=relu)
            close(C, want, torch.bfloat16)
        # relu on a plain operand
        C = torch.full((M, N), float("nan"), dtype=torch.float32, device=cuda)
        ops.gemm(act.to(cuda), W.to(cuda), C, M, N, K, transB=True, a_relu=True)
        close(C, torch.relu(act.double()) @ W.double().t(), torch.bfloat16)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


@pytest.mark.parametrize("cfg,lengths", [(-1, [384, 384, 128, 128]), (0, [384, 384, 128, 128]), (7, [384, 384, 128, 128]),
                                         (8, [256, 128, 640]), (1, [768, 256]), (3, [768, 256]), (4, [384, 576]),
                                         (9, [384, 576]), (6, [512, 512])])
def test_gemm_result_and_operand_in_pieces_along_n(cuda, cfg, lengths):
    """Backward of that linear: the data gradient dY W written as the pieces of the backward all_to_all, masked with
    relu's derivative taken from the forward pieces; the weight gradient dY^T relu(cat(pieces)) with its bias
    gradient, alone and for several layers in one launch."""
    from hap_amd._lib import lib
    g = torch.Generator().manual_seed(41 + max(cfg, 0))
    rows, d_out = 300, 200
    F_ = sum(lengths)
    pre = torch.randn(rows, F_, generator=g).bfloat16()                 # the forward pieces (pre-activation)
    dy = torch.randn(rows, d_out, generator=g).bfloat16()
    W = torch.randn(d_out, F_, generator=g).bfloat16()                  # second linear's weight [d_out, F]
    fwd_pieces = _pieces(pre, lengths, cuda)
    want_dx = (dy.double() @ W.double()) * (pre.double() > 0)
    # the result's pieces have the layout of the forward pieces (the mask is read at the result's addresses)
    outs = _pieces(torch.full((rows, F_), float("nan"), dtype=torch.bfloat16), lengths, cuda)
    try:
        lib().hapmi_gemm_tuning(cfg, 1)
        ops.gemm(dy.to(cuda), W.to(cuda), None, rows, F_, d_out, c_segments=outs, mask_segments=fwd_pieces)
        close(torch.cat(outs, 1), want_dx, torch.bfloat16)
        outs2 = [torch.full((rows, l), float("nan"), dtype=torch.bfloat16, device=cuda) for l in lengths]
        ops.gemm(dy.to(cuda), W.to(cuda), None, rows, F_, d_out, c_segments=outs2)
        close(torch.cat(outs2, 1), dy.double() @ W.double(), torch.bfloat16)
        # weight gradient [d_out, F] = dY^T relu(pre), bias gradient = column sums of dY
        want_dw = dy.double().t() @ torch.relu(pre.double())
        gw = torch.full((d_out, F_), float("nan"), device=cuda)
        gb = torch.zeros(d_out, device=cuda)
        ops.gemm(dy.to(cuda), None, gw, d_out, F_, rows, transA=True, b_segments=fwd_pieces, b_relu=True, a_rowsum=gb)
        close(gw, want_dw, torch.bfloat16)
        torch.testing.assert_close(gb.cpu().double(), dy.double().sum(0), rtol=1e-4, atol=1e-3)
        # three layers in one launch
        pres = [torch.randn(rows, F_, generator=g).bfloat16() for _ in range(3)]
        dys = [torch.randn(rows, d_out, generator=g).bfloat16() for _ in range(3)]
        gws = [torch.full((d_out, F_), float("nan"), device=cuda) for _ in range(3)]
        ops.gemm_group([t.to(cuda) for t in dys], [_pieces(t, lengths, cuda) for t in pres],
                       gws, d_out, F_, rows, transA=True, b_relu=True)
        for z in range(3):
            close(gws[z], dys[z].double().t() @ torch.relu(pres[z].double()), torch.bfloat16)
    finally:
        lib().hapmi_gemm_tuning(-1, 0)


def test_gemm_pieces_are_checked(cuda):
    from hap_amd._lib import HapmiError
    x = torch.zeros(64, 96, dtype=torch.bfloat16, device=cuda)
    y = torch.zeros(64, 160, dtype=torch.bfloat16, device=cuda)
    W = torch.zeros(32, 256, dtype=torch.bfloat16, device=cuda)
    C = torch.zeros(64, 32, dtype=torch.bfloat16, device=cuda)
    with pytest.raises(HapmiError, match="multiple of 64"):            # a piece boundary inside a k-tile
        ops.gemm(None, W, C, 64, 32, 256, transB=True, a_segments=[x, y])
    outs = [torch.zeros(64, 96, dtype=torch.bfloat16, device=cuda), torch.zeros(64, 160, dtype=torch.bfloat16, device=cuda)]
    with pytest.raises(HapmiError, match="multiple of 64"):
        ops.gemm(C, torch.zeros(32, 256, dtype=torch.bfloat16, device=cuda), None, 64, 256, 32, c_segments=outs)
    with pytest.raises(ValueError, match="add up"):
        ops.gemm(None, W, C, 64, 32, 256, transB=True, a_segments=[y])
    f = torch.zeros(64, 128, device=cuda)
    with pytest.raises(HapmiError, match="bf16"):
        ops.gemm(None, torch.zeros(32, 256, device=cuda), torch.zeros(64, 32, device=cuda), 64, 32, 256, transB=True,
                 a_segments=[f, f])


