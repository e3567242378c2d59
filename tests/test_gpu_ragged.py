"""Device-local halves of the uneven collectives through the C ABI, bit-exact against the reference's own
torch.cat / torch.split / slicing on the CPU (/root/reference/collectives.py:9-29, 88-103, 146-166)."""
import pytest
import torch

from hap_amd import ops
from hap_amd._lib import HapmiError
from oracle.ops import _accumulate

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float32, torch.int64, torch.int16]


def rnd(shape, dtype, g):
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype)
    return torch.randint(-1000, 1000, shape, generator=g).to(dtype)


CASES = [  # (shape of the full tensor, dim, lengths)
    ((10, 6), 0, [1, 2, 3, 4]),
    ((5, 10), 1, [1, 2, 3, 4]),
    ((4, 10, 24), 1, [3, 3, 1, 3]),
    ((8, 16, 40), 0, [3, 3, 1, 1]),
    ((3, 5, 48), 2, [18, 18, 6, 6]),
    ((7, 9), 1, [4, 0, 5, 0]),               # zero-length shards
    ((6, 7, 3), 1, [2, 5]),                  # odd inner size: narrow vector path
    ((2, 1, 4096), 1, [1]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,dim,L", CASES)
def test_pad_split_concat_slice_layouts(cuda, dtype, shape, dim, L):
    g = torch.Generator().manual_seed(11)
    full = rnd(shape, dtype, g)
    m = max(L)
    shards = list(torch.split(full, L, dim=dim))
    dfull = full.to(cuda)
    # pad: head equals the shard, tail keeps what the buffer held before (the reference leaves it uninitialised)
    for sh in shards:
        out = torch.full(ops._with_dim(sh.shape, dim, m), 7, dtype=dtype, device=cuda)
        ops.pad_rows(sh.contiguous().to(cuda), dim, m, out)
        head, tail = out.cpu().split([sh.shape[dim], m - sh.shape[dim]], dim=dim)
        assert torch.equal(head, sh) and (tail == 7).all()
    # split + pad
    outs = [torch.full(ops._with_dim(shape, dim, m), 7, dtype=dtype, device=cuda) for _ in L]
    ops.split_pad(dfull, L, dim, m, outs)
    for o, sh in zip(outs, shards):
        head, tail = o.cpu().split([sh.shape[dim], m - sh.shape[dim]], dim=dim)
        assert torch.equal(head, sh) and (tail == 7).all()
    # unpad + concat of those padded slices gives the full tensor back
    assert torch.equal(ops.unpad_concat(outs, L, dim).cpu(), full)
    # unpadded split / concat
    pieces = ops.split_rows(dfull, L, dim)
    for p, sh in zip(pieces, shards):
        assert torch.equal(p.cpu(), sh)
    assert torch.equal(ops.concat_rows(pieces, dim).cpu(), full)
    # dynamic_slice and its inverse
    for r in range(len(L)):
        off = sum(L[:r])
        s = ops.slice_rows(dfull, dim, off, L[r])
        assert torch.equal(s.cpu(), shards[r])
        back = torch.zeros(shape, dtype=dtype, device=cuda)
        ops.place_rows(s, back, dim, off)
        want = torch.zeros(shape, dtype=dtype)
        want.narrow(dim, off, L[r]).copy_(shards[r])
        assert torch.equal(back.cpu(), want)


def test_fused_entry_points_with_empty_shards_and_misaligned_pieces(cuda):
    g = torch.Generator().manual_seed(6)
    # zero-length pieces are skipped by the masked split
    dy = torch.randn(4, 64, generator=g).bfloat16().to(cuda)
    y = torch.relu(torch.randn(4, 64, generator=g)).bfloat16().to(cuda)
    pieces = ops.split_rows(dy, [32, 0, 32, 0], 1, relu_of=y)
    want = torch.where(y > 0, dy, torch.zeros_like(dy))
    assert [tuple(p.shape) for p in pieces] == [(4, 32), (4, 0), (4, 32), (4, 0)]
    assert torch.equal(torch.cat(pieces, dim=1), want)
    # pieces that are not whole 16-byte vectors are refused (the executor then keeps relu's backward as its own pass)
    with pytest.raises(HapmiError):
        ops.split_rows(dy, [30, 34], 1, relu_of=y)
    # an empty output of the reduction with an addend is a no-op
    parts = [torch.randn(6, 8, generator=g).to(cuda) for _ in range(3)]
    empty = ops.ragged_reduce(parts, 0, 2, 0, addend=torch.empty(0, 8, device=cuda))
    assert tuple(empty.shape) == (0, 8)
    # a misaligned addend takes the scalar path and gives the same sum
    base = torch.randn(4 * 8 + 1, generator=g).to(cuda)
    addend = base[1:].view(4, 8)
    got = ops.ragged_reduce(parts, 0, 1, 4, addend=addend)
    want = parts[0][1:5] + parts[1][1:5] + parts[2][1:5] + addend
    assert torch.equal(got, want)


def test_split_pad_skips_a_missing_slice_and_unpad_concat_a_slice_in_place(cuda):
    g = torch.Generator().manual_seed(8)
    L, m = [5, 5, 2], 5
    full = torch.randn(12, 16, generator=g).bfloat16()
    outs = [torch.full((m, 16), 7.0, dtype=torch.bfloat16, device=cuda), None,
            torch.full((m, 16), 7.0, dtype=torch.bfloat16, device=cuda)]
    ops.split_pad(full.to(cuda), L, 0, m, outs)
    assert torch.equal(outs[0].cpu(), full[:5]) and torch.equal(outs[2].cpu()[:2], full[10:]) and (outs[2].cpu()[2:] == 7).all()
    # a slice of the longest length that already lies at its rows of the result is not copied (and not needed elsewhere)
    dst = torch.full((12, 16), 3.0, dtype=torch.bfloat16, device=cuda)
    mine = dst.narrow(0, 5, 5)
    mine.copy_(full[5:10])
    ops.unpad_concat([outs[0], mine, outs[2]], L, 0, dst)
    assert torch.equal(dst.cpu(), full)


def test_concat_leaves_a_piece_that_is_already_in_place(cuda):
    g = torch.Generator().manual_seed(4)
    pieces = [torch.randn(n, 24, generator=g).bfloat16().to(cuda) for n in (3, 5, 2)]
    out = torch.full((10, 24), 7.0, dtype=torch.bfloat16, device=cuda)
    mine = out.narrow(0, 3, 5)
    mine.copy_(pieces[1])
    ops.concat_rows([pieces[0], mine, pieces[2]], 0, out)
    assert torch.equal(out, torch.cat(pieces, dim=0))
    # with an activation the piece in place is processed like the others
    out2 = torch.empty(10, 24, dtype=torch.bfloat16, device=cuda)
    mine2 = out2.narrow(0, 3, 5)
    mine2.copy_(pieces[1])
    ops.concat_rows([pieces[0], mine2, pieces[2]], 0, out2, act="relu")
    assert torch.equal(out2, torch.relu(torch.cat(pieces, dim=0)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_concat_with_fused_relu(cuda, dtype):
    g = torch.Generator().manual_seed(3)
    pieces = [torch.randn(3, 8, n, generator=g).to(dtype) for n in (48, 48, 16, 16)]
    out = ops.concat_rows([p.to(cuda) for p in pieces], 2, act="relu")
    assert torch.equal(out.cpu(), torch.relu(torch.cat(pieces, dim=2)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape,dim,L", [((6, 5, 128), 2, [48, 48, 16, 16]), ((3, 40, 8), 1, [18, 18, 2, 2]),
                                         ((16, 64), 1, [64]), ((520, 1040), 1, [392, 392, 128, 128])])
def test_split_with_fused_relu_backward(cuda, dtype, shape, dim, L):
    """Pieces of dy * (y > 0), y the output of a relu (with exact zeros, negative zeros and NaN among its values),
    against F.relu's own backward (threshold_backward) on the CPU."""
    g = torch.Generator().manual_seed(5)
    pre = torch.randn(shape, generator=g)
    pre.view(-1)[::7] = 0.0
    y = torch.relu(pre).to(dtype)
    y.view(-1)[3] = float("nan")
    y.view(-1)[5] = -0.0
    y.view(-1)[11] = float("inf")
    dy = torch.randn(shape, generator=g).to(dtype)
    want = torch.where(y > 0, dy, torch.zeros_like(dy))
    pieces = ops.split_rows(dy.to(cuda), L, dim, relu_of=y.to(cuda))
    for got, ref in zip(pieces, torch.split(want, L, dim=dim)):
        assert torch.equal(got.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                           ref.contiguous().view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # autograd's relu backward agrees wherever y is a number
    yy = pre.clone().requires_grad_(True)
    torch.relu(yy).backward(dy.float())
    ok = ~torch.isnan(y.float()) & (y.float() == torch.relu(pre).to(dtype).float())
    assert torch.equal(torch.cat([p.cpu() for p in pieces], dim=dim).float()[ok], yy.grad.to(dtype).float()[ok])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [1, 2, 3, 4, 8])
@pytest.mark.parametrize("shape,dim,off,length", [((40, 64), 0, 7, 20), ((4, 10, 24), 1, 3, 4), ((5, 9, 7), 1, 0, 9),
                                                  ((3, 64), 1, 8, 48)])
def test_ragged_reduce_bit_exact(cuda, dtype, W, shape, dim, off, length):
    g = torch.Generator().manual_seed(W)
    parts = [torch.randn(shape, generator=g).to(dtype) for _ in range(W)]
    got = ops.ragged_reduce([p.to(cuda) for p in parts], dim, off, length)
    want = _accumulate([p.narrow(dim, off, length) for p in parts])
    assert torch.equal(got.cpu(), want)
    # one more term of the output's shape, added last: into a separate output and in place
    g0 = torch.randn(want.shape, generator=g).to(dtype)
    acc = parts[0].narrow(dim, off, length).float()
    for p in parts[1:]:
        acc = acc + p.narrow(dim, off, length).float()
    want_add = (acc + g0.float()).to(dtype)
    got_add = ops.ragged_reduce([p.to(cuda) for p in parts], dim, off, length, addend=g0.to(cuda))
    assert torch.equal(got_add.cpu(), want_add)
    inplace = g0.to(cuda)
    ops.ragged_reduce([p.to(cuda) for p in parts], dim, off, length, out=inplace, addend=inplace)
    assert torch.equal(inplace.cpu(), want_add)


def test_config5_shapes_round_trip_and_reduce(cuda):
    """8 ragged bf16 shards [S_i, 4096], S_i in [1000, 3000] from the seed: pad to max, split, concat, reduce."""
    g = torch.Generator().manual_seed(39)
    S = torch.randint(1000, 3001, (8,), generator=g).tolist()
    m, total = max(S), sum(S)
    shards = [torch.randn(s, 4096, generator=g).bfloat16().to(cuda) for s in S]
    padded = [ops.pad_rows(x, 0, m) for x in shards]
    full = ops.unpad_concat(padded, S, 0)
    assert full.shape == (total, 4096)
    assert torch.equal(full, torch.cat(shards, dim=0))                        # layout, checked on the GPU side
    again = ops.split_pad(full, S, 0, m)
    for a, x, s in zip(again, shards, S):
        assert torch.equal(a[:s], x)
    # reduce-scatter layout: 8 virtual ranks each hold a full [total, 4096] tensor
    fulls_cpu = [torch.randn(total, 4096, generator=g).bfloat16() for _ in range(8)]
    fulls = [f.to(cuda) for f in fulls_cpu]
    off = 0
    acc = torch.zeros(total, 4096, dtype=torch.float32)                         # the reference sum: on the CPU
    for f in fulls_cpu:
        acc += f.float()                                                        # same rank order, float32
    want = acc.bfloat16()
    for r, s in enumerate(S):
        out = ops.ragged_reduce(fulls, 0, off, s)
        assert torch.equal(out.cpu(), want[off:off + s])
        off += s


def test_bad_arguments_are_refused(cuda):
    from hap_amd._lib import HapmiError
    x = torch.zeros(4, 8, device=cuda)
    with pytest.raises(HapmiError):
        ops.slice_rows(x, 0, 3, 2)
    with pytest.raises(HapmiError):
        ops.pad_rows(x, 0, 3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_multi_shard_launches_match_single_ones(cuda, dtype):
    g = torch.Generator().manual_seed(17)
    L = [5, 0, 9, 2]
    shards = [torch.randn(3, l, 24, generator=g).to(dtype).to(cuda) for l in L]
    padded = ops.pad_rows_multi(shards, 1, 9, [torch.full((3, 9, 24), 7, dtype=dtype, device=cuda) for _ in L])
    for p, s, l in zip(padded, shards, L):
        assert torch.equal(p[:, :l], s) and (p[:, l:] == 7).all()
    fulls = [torch.randn(3, 16, 24, generator=g).to(dtype).to(cuda) for _ in range(4)]
    offs = [0, 5, 5, 14]
    outs = ops.ragged_reduce_multi(fulls, 1, offs, L)
    for o, off, l in zip(outs, offs, L):
        assert torch.equal(o, ops.ragged_reduce(fulls, 1, off, l))
