"""Tensor-level wrappers over the C ABI of libhapmi.so.

Every function takes torch tensors that live on the GPU, passes raw device
pointers to the library and enqueues on torch's current stream.  CPU tensors
are refused: there is no fallback path.
"""
from __future__ import annotations

import ctypes
import math
from typing import List, Optional, Sequence

import torch

from . import _lib
from ._lib import ACT_GELU, ACT_NONE, ACT_RELU, BF16, F32, GemmArgs, GemmSegments, check, lib

_ACT = {None: ACT_NONE, "none": ACT_NONE, "relu": ACT_RELU, "gelu": ACT_GELU, "sigmoid": _lib.ACT_SIGMOID}


def dtype_code(t) -> int:
    dt = t if isinstance(t, torch.dtype) else t.dtype
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise TypeError(f"dtype {dt} is not handled by the HIP kernels (float32 / bfloat16 only)")


def _dev(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise _lib.HapmiError("the HIP kernels take GPU tensors only; got a CPU tensor (no CPU fallback exists)")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _i64(vals: Sequence[int]):
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def _ptrs(tensors: Sequence[Optional[torch.Tensor]]):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else 0 for t in tensors])


def init():
    check(lib().hapmi_init())


def _need(t: Optional[torch.Tensor], n_elems: int, what: str, offset: int = 0):
    """Host-side bounds check: the kernel will touch elements [offset, offset + n_elems) of ``t``."""
    if t is None:
        return
    if offset < 0 or n_elems < 0 or offset + n_elems > t.numel():
        raise _lib.HapmiError(f"{what}: the kernel would access elements [{offset}, {offset + n_elems}) of a buffer "
                              f"that holds {t.numel()}")
    if not t.is_contiguous():
        raise _lib.HapmiError(f"{what}: buffer must be contiguous")


def _span(rows: int, cols: int, ld: int) -> int:
    """Elements spanned by a [rows, cols] block with row stride ld."""
    return 0 if rows <= 0 or cols <= 0 else (rows - 1) * ld + cols


# ---------------------------------------------------------------------------
# layout helpers: a tensor sharded on `dim` is [outer, len, inner]
# ---------------------------------------------------------------------------

def _oli(shape, dim):
    outer = 1
    for s in shape[:dim]:
        outer *= s
    inner = 1
    for s in shape[dim + 1:]:
        inner *= s
    return outer, shape[dim], inner


def _with_dim(shape, dim, n):
    return tuple(shape[:dim]) + (n,) + tuple(shape[dim + 1:])


def pad_rows(src: torch.Tensor, dim: int, padded_len: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """collectives.padded: copy ``src`` into the head of a buffer whose ``dim`` is ``padded_len`` long."""
    _dev(src, out)
    assert src.is_contiguous()
    outer, length, inner = _oli(src.shape, dim)
    if out is None:
        out = torch.empty(_with_dim(src.shape, dim, padded_len), dtype=src.dtype, device=src.device)
    _need(out, outer * padded_len * inner, "pad_rows dst")
    if out.dtype != src.dtype:
        raise TypeError("pad_rows: dtype mismatch")
    check(lib().hapmi_pad_rows(_ptr(src), _ptr(out), outer, length, padded_len, inner * src.element_size(), _stream()))
    return out


def unpad_concat(slices: Sequence[torch.Tensor], lengths: Sequence[int], dim: int,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(*slices, out)
    ref = slices[0]
    outer, _, inner = _oli(ref.shape, dim)
    # a slice that lies at its place in ``out`` may hold its payload only: the padded length is the longest one's
    padded_len = max([sl.shape[dim] for sl in slices] + [int(n) for n in lengths])
    if out is None:
        out = torch.empty(_with_dim(ref.shape, dim, sum(lengths)), dtype=ref.dtype, device=ref.device)
    off = 0
    for sl, n in zip(slices, lengths):
        # a slice that already lies at its place in ``out`` (one contiguous range) is left where it is by the kernel
        # and only has to hold its payload rows
        in_place = outer == 1 and sl.data_ptr() == out.data_ptr() + off * inner * out.element_size()
        _need(sl, outer * (n if in_place else padded_len) * inner, "unpad_concat slice")
        if sl.dtype != ref.dtype:
            raise TypeError("unpad_concat: dtype mismatch")
        off += n
    _need(out, outer * sum(lengths) * inner, "unpad_concat dst")
    if out.numel() == 0:
        return out
    check(lib().hapmi_unpad_concat(_ptrs(slices), _i64(lengths), len(lengths), _ptr(out), outer, padded_len,
                                   inner * ref.element_size(), _stream()))
    return out


def split_pad(src: torch.Tensor, lengths: Sequence[int], dim: int, padded_len: int,
              outs: Optional[Sequence[Optional[torch.Tensor]]] = None) -> List[torch.Tensor]:
    """Padded pieces of ``src`` along ``dim``; a ``None`` entry of ``outs`` is a piece that is not produced."""
    _dev(src)
    assert src.is_contiguous()
    outer, total, inner = _oli(src.shape, dim)
    assert total == sum(lengths)
    if outs is None:
        outs = [torch.empty(_with_dim(src.shape, dim, padded_len), dtype=src.dtype, device=src.device) for _ in lengths]
    for o in outs:
        if o is not None:
            _dev(o)
            _need(o, outer * padded_len * inner, "split_pad slice")
    if src.numel() == 0:
        return list(outs)
    check(lib().hapmi_split_pad(_ptr(src), _ptrs(outs), _i64(lengths), len(lengths), outer, padded_len,
                                inner * src.element_size(), _stream()))
    return list(outs)


def slice_rows(src: torch.Tensor, dim: int, offset: int, length: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(src, out)
    assert src.is_contiguous()
    outer, src_len, inner = _oli(src.shape, dim)
    if out is None:
        out = torch.empty(_with_dim(src.shape, dim, length), dtype=src.dtype, device=src.device)
    _need(out, outer * length * inner, "slice_rows dst")
    if out.numel() == 0:
        return out
    check(lib().hapmi_slice_rows(_ptr(src), _ptr(out), outer, src_len, offset, length, inner * src.element_size(), _stream()))
    return out


def place_rows(src: torch.Tensor, dst: torch.Tensor, dim: int, offset: int) -> torch.Tensor:
    _dev(src, dst)
    outer, length, inner = _oli(src.shape, dim)
    o2, dst_len, i2 = _oli(dst.shape, dim)
    if (o2, i2) != (outer, inner) or not src.is_contiguous() or not dst.is_contiguous() or src.dtype != dst.dtype:
        raise _lib.HapmiError("place_rows: source and destination do not agree outside the sliced dimension")
    if src.numel() == 0:
        return dst
    check(lib().hapmi_place_rows(_ptr(src), _ptr(dst), outer, dst.shape[dim], offset, length,
                                 inner * src.element_size(), _stream()))
    return dst


def split_rows(src: torch.Tensor, lengths: Sequence[int], dim: int,
               outs: Optional[Sequence[Optional[torch.Tensor]]] = None,
               relu_of: Optional[torch.Tensor] = None, scale: float = 1.0) -> List[torch.Tensor]:
    """Pieces of ``src`` along ``dim``; with ``relu_of`` (a relu's forward output of src's shape) the pieces
    are those of ``src * (relu_of > 0) * scale`` (scale != 1: relu followed by dropout, relu_of being the dropped
    output and scale dropout's 1 / (1 - p))."""
    _dev(src)
    assert src.is_contiguous()
    outer, total, inner = _oli(src.shape, dim)
    assert total == sum(lengths)
    if outs is None:
        outs = [torch.empty(_with_dim(src.shape, dim, l), dtype=src.dtype, device=src.device) for l in lengths]
    for o, l in zip(outs, lengths):
        if o is not None:
            _dev(o)
            _need(o, outer * l * inner, "split_rows piece")
    if src.numel() == 0:
        return list(outs)
    if relu_of is not None:
        _dev(relu_of)
        assert relu_of.is_contiguous() and relu_of.shape == src.shape and relu_of.dtype == src.dtype
        if scale != 1.0:
            check(lib().hapmi_split_rows_relu_bwd_scaled(_ptr(src), _ptr(relu_of), _ptrs(outs), _i64(lengths),
                                                         len(lengths), outer, inner * src.element_size(),
                                                         ctypes.c_float(scale), dtype_code(src), _stream()))
        else:
            check(lib().hapmi_split_rows_relu_bwd(_ptr(src), _ptr(relu_of), _ptrs(outs), _i64(lengths), len(lengths),
                                                  outer, inner * src.element_size(), dtype_code(src), _stream()))
        return list(outs)
    check(lib().hapmi_split_rows(_ptr(src), _ptrs(outs), _i64(lengths), len(lengths), outer,
                                 inner * src.element_size(), _stream()))
    return list(outs)


def concat_rows(pieces: Sequence[torch.Tensor], dim: int, out: Optional[torch.Tensor] = None,
                act: Optional[str] = None, drop=None) -> torch.Tensor:
    """``drop`` = (p, rng_state, stream_id) with act = "relu": out = dropout(relu(cat(pieces))), the decisions
    being those ``dropout`` takes for ``out`` under the same three."""
    _dev(*pieces, out)
    ref = pieces[0]
    lengths = [p.shape[dim] for p in pieces]
    outer, _, inner = _oli(ref.shape, dim)
    if out is None:
        out = torch.empty(_with_dim(ref.shape, dim, sum(lengths)), dtype=ref.dtype, device=ref.device)
    for p_, l in zip(pieces, lengths):
        _need(p_, outer * l * inner, "concat_rows piece")
        if p_.dtype != ref.dtype:
            raise TypeError("concat_rows: dtype mismatch")
    _need(out, outer * sum(lengths) * inner, "concat_rows dst")
    if out.numel() == 0:
        return out
    if drop is not None:
        if act != "relu":
            raise ValueError("concat_rows: dropout rides on a fused relu only")
        p, rng_state, stream_id = drop
        _dev(rng_state)
        _check_rng(rng_state, "concat_rows")
        check(lib().hapmi_concat_rows_relu_dropout(_ptrs(pieces), _i64(lengths), len(lengths), _ptr(out), outer,
                                                   inner * ref.element_size(), ctypes.c_float(p), _ptr(rng_state),
                                                   int(stream_id), dtype_code(ref), _stream()))
        return out
    check(lib().hapmi_concat_rows(_ptrs(pieces), _i64(lengths), len(lengths), _ptr(out), outer,
                                  inner * ref.element_size(), _ACT[act], dtype_code(ref) if _ACT[act] else 0, _stream()))
    return out


def relu_dropout_pieces(src: Sequence[torch.Tensor], dst: Sequence[torch.Tensor], p: float, rng_state, stream_id: int):
    """dst[i] = the columns of dropout(relu(cat(src, dim 1))) that piece i holds ([rows, width_i] each, contiguous),
    with the decisions ``dropout`` takes for the concatenated [rows, sum(width)] tensor."""
    _dev(*src, *dst, rng_state)
    _check_rng(rng_state, "relu_dropout_pieces")
    rows = src[0].shape[0]
    widths = []
    for a, b in zip(src, dst):
        if a.dim() != 2 or a.shape != b.shape or a.dtype != src[0].dtype or b.dtype != a.dtype or a.shape[0] != rows:
            raise ValueError("relu_dropout_pieces: pieces are [rows, width_i] tensors of one dtype, dst like src")
        _need(a, a.numel(), "relu_dropout_pieces src")
        _need(b, b.numel(), "relu_dropout_pieces dst")
        widths.append(a.shape[1])
    check(lib().hapmi_relu_dropout_pieces(_ptrs(src), _ptrs(dst), _i64(widths), len(widths), rows, ctypes.c_float(p),
                                          _ptr(rng_state), int(stream_id), dtype_code(src[0]), _stream()))


def ragged_reduce(contribs: Sequence[torch.Tensor], dim: int, offset: int, length: int,
                  out: Optional[torch.Tensor] = None, addend: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = sum_w contribs[w].narrow(dim, offset, length) in rank order, float32 accumulation; ``addend`` (out's
    shape, may be ``out``) is added to the sum last."""
    _dev(*contribs, out, addend)
    ref = contribs[0]
    outer, src_len, inner = _oli(ref.shape, dim)
    if out is None:
        out = torch.empty(_with_dim(ref.shape, dim, length), dtype=ref.dtype, device=ref.device)
    for c in contribs:
        _need(c, outer * src_len * inner, "ragged_reduce contribution")
        if c.dtype != ref.dtype:
            raise TypeError("ragged_reduce: dtype mismatch")
    _need(out, outer * length * inner, "ragged_reduce dst")
    if out.dtype != ref.dtype:
        raise TypeError("ragged_reduce: dtype mismatch")
    if addend is not None:
        _need(addend, outer * length * inner, "ragged_reduce addend")
        if addend.dtype != ref.dtype:
            raise TypeError("ragged_reduce: dtype mismatch")
    if out.numel() == 0:
        return out
    if addend is not None:
        check(lib().hapmi_ragged_reduce_add(_ptrs(contribs), len(contribs), _ptr(out), _ptr(addend), outer, src_len,
                                            offset, length, inner, dtype_code(ref), _stream()))
        return out
    check(lib().hapmi_ragged_reduce(_ptrs(contribs), len(contribs), _ptr(out), outer, src_len, offset, length, inner,
                                    dtype_code(ref), _stream()))
    return out


def ragged_reduce_multi(contribs: Sequence[torch.Tensor], dim: int, offsets: Sequence[int], lengths: Sequence[int],
                        outs: Optional[Sequence[torch.Tensor]] = None) -> List[torch.Tensor]:
    """One launch for several output shards: outs[r] = sum_w contribs[w].narrow(dim, offsets[r], lengths[r])."""
    _dev(*contribs)
    ref = contribs[0]
    outer, src_len, inner = _oli(ref.shape, dim)
    if outs is None:
        outs = [torch.empty(_with_dim(ref.shape, dim, l), dtype=ref.dtype, device=ref.device) for l in lengths]
    for c in contribs:
        _need(c, outer * src_len * inner, "ragged_reduce contribution")
        if c.dtype != ref.dtype:
            raise TypeError("ragged_reduce: dtype mismatch")
    for o, off, l in zip(outs, offsets, lengths):
        _dev(o)
        _need(o, outer * l * inner, "ragged_reduce dst")
        if o.dtype != ref.dtype or off < 0 or off + l > src_len:
            raise _lib.HapmiError("ragged_reduce_multi: bad output shard")
    check(lib().hapmi_ragged_reduce_multi(_ptrs(contribs), len(contribs), _ptrs(outs), _i64(offsets), _i64(lengths),
                                          len(lengths), outer, src_len, inner, dtype_code(ref), _stream()))
    return list(outs)


def pad_rows_multi(srcs: Sequence[torch.Tensor], dim: int, padded_len: int,
                   outs: Optional[Sequence[torch.Tensor]] = None) -> List[torch.Tensor]:
    """collectives.padded for several shards in one launch."""
    _dev(*srcs)
    ref = srcs[0]
    outer, _, inner = _oli(ref.shape, dim)
    lengths = [s.shape[dim] for s in srcs]
    if outs is None:
        outs = [torch.empty(_with_dim(ref.shape, dim, padded_len), dtype=ref.dtype, device=ref.device) for _ in srcs]
    for s, o, l in zip(srcs, outs, lengths):
        _dev(o)
        _need(s, outer * l * inner, "pad_rows_multi src")
        _need(o, outer * padded_len * inner, "pad_rows_multi dst")
        if o.dtype != ref.dtype or s.dtype != ref.dtype:
            raise TypeError("pad_rows_multi: dtype mismatch")
    check(lib().hapmi_pad_rows_multi(_ptrs(srcs), _ptrs(outs), _i64(lengths), len(srcs), outer, padded_len,
                                     inner * ref.element_size(), _stream()))
    return list(outs)


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------

_gemm_ws: Optional[torch.Tensor] = None


def set_gemm_workspace(t: Optional[torch.Tensor]) -> None:
    """Scratch buffer for split-K partial sums and the partial sums of the deterministic reductions (bias
    gradients, column sums), shared by all calls that follow (one stream)."""
    global _gemm_ws
    _gemm_ws = t


def _workspace(device) -> torch.Tensor:
    """The installed workspace, or a 64 MiB one made on first use (calls outside an executor, e.g. tests)."""
    global _gemm_ws
    if _gemm_ws is None or _gemm_ws.device != device:
        _gemm_ws = torch.empty(16 << 20, dtype=torch.float32, device=device)
    return _gemm_ws


def _segments(pieces: Sequence[torch.Tensor], rows: int, what: str) -> GemmSegments:
    """Description of an operand / result that exists as pieces along its column dimension: every piece a 2-d view
    [rows, len] with unit column stride (its row stride is the piece's leading dimension)."""
    if not 1 <= len(pieces) <= _lib.GEMM_MAX_SEGMENTS:
        raise ValueError(f"{what}: 1..{_lib.GEMM_MAX_SEGMENTS} pieces expected")
    g = GemmSegments()
    g.n = len(pieces)
    pos = 0
    for i, t in enumerate(pieces):
        _dev(t)
        if t.dim() != 2 or t.shape[0] != rows or t.stride(1) != 1 or t.dtype != pieces[0].dtype:
            raise ValueError(f"{what}: piece {i} must be a [rows, len] view with unit column stride of one element type")
        g.begin[i] = pos
        g.ld[i] = t.stride(0) if rows > 1 else max(t.stride(0), t.shape[1])
        g.base[i] = t.data_ptr()
        # a piece may be a view into a larger buffer: the bound is the storage behind the view's first element
        room = t.untyped_storage().nbytes() // t.element_size() - t.storage_offset()
        if _span(rows, t.shape[1], int(g.ld[i])) > room:
            raise _lib.HapmiError(f"{what}: piece {i} reaches beyond its storage")
        pos += t.shape[1]
    g.begin[len(pieces)] = pos
    return g


def gemm(A: Optional[torch.Tensor], B: Optional[torch.Tensor], C: Optional[torch.Tensor], M: int, N: int, K: int, *, transA=False, transB=False,
         lda=None, ldb=None, ldc=None, bias: Optional[torch.Tensor] = None, accumulate=False, act=None, alpha=1.0,
         batch1=1, batch2=1, strideA=(0, 0), strideB=(0, 0), strideC=(0, 0),
         offA=0, offB=0, offC=0, workspace: Optional[torch.Tensor] = None,
         a_rowsum: Optional[torch.Tensor] = None, relu_mask: Optional[torch.Tensor] = None,
         addend: Optional[torch.Tensor] = None, a_segments=None, b_segments=None, c_segments=None,
         mask_segments=None, a_relu=False, b_relu=False, drop=None):
    """C = alpha * op(A) @ op(B) (+bias)(act)(+C).  Offsets and strides are in elements.
    ``drop`` = (p, rng_state, stream_id): dropout behind the activation, with the decisions ``dropout`` takes for C
    (one contiguous problem).  ``workspace`` (or
    the buffer installed with ``set_gemm_workspace``) lets the library split a long reduction over K.
    ``a_rowsum`` (float32[M], transA only): the sums over k of op(A)'s rows are added into it.
    ``relu_mask`` ([M, ldc] like C): result elements whose mask is <= 0 are zero (relu backward).
    ``addend`` ([M, ldc] like C, with ``accumulate``): C = addend + result; C itself is only written.
    ``a_segments`` / ``b_segments`` / ``c_segments`` / ``mask_segments``: the operand / result / relu mask as a list
    of pieces along K (A, stored [M, K]) or N (B stored [K, N], C, mask) instead of one tensor (pass None for it);
    ``a_relu`` / ``b_relu``: relu applied to that operand as it is loaded."""
    if a_segments is not None or b_segments is not None or c_segments is not None or a_relu or b_relu:
        if drop is not None:
            raise ValueError("gemm: dropout in the epilogue does not combine with operands in pieces")
        return _gemm_segmented(A, B, C, M, N, K, transA, transB, lda, ldb, ldc, bias, act, alpha, workspace, a_rowsum,
                               a_segments, b_segments, c_segments, mask_segments, a_relu, b_relu, accumulate)
    _dev(A, B, C, bias, a_rowsum, relu_mask, addend)
    if A.dtype != B.dtype:
        raise TypeError("gemm operands must share a dtype")
    a = GemmArgs()
    a.A = A.data_ptr() + offA * A.element_size()
    a.B = B.data_ptr() + offB * B.element_size()
    a.C = C.data_ptr() + offC * C.element_size()
    a.bias = bias.data_ptr() if bias is not None else 0
    if bias is not None and bias.dtype != torch.float32:
        raise TypeError("gemm bias must be float32")
    a.M, a.N, a.K = M, N, K
    a.lda = lda if lda is not None else (M if transA else K)
    a.ldb = ldb if ldb is not None else (K if transB else N)
    a.ldc = ldc if ldc is not None else N
    a.transA, a.transB = int(transA), int(transB)
    a.in_dtype, a.out_dtype = dtype_code(A), dtype_code(C)
    a.accumulate, a.act, a.alpha = int(accumulate), _ACT[act], float(alpha)
    a.batch1, a.batch2 = batch1, batch2
    a.strideA1, a.strideA2 = strideA
    a.strideB1, a.strideB2 = strideB
    a.strideC1, a.strideC2 = strideC
    ws = workspace if workspace is not None else _gemm_ws
    if ws is None and a_rowsum is not None:
        ws = _workspace(A.device)                      # the row sums' partial sums need one
    if ws is not None and ws.is_cuda and ws.device == A.device:
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    else:
        a.workspace, a.workspace_bytes = 0, 0
    zb = lambda st: (batch1 - 1) * st[0] + (batch2 - 1) * st[1]
    epv = 16 // A.element_size()
    up = lambda n: (n + epv - 1) // epv * epv          # the kernel reads whole 16-byte vectors along a row
    _need(A, _span(K if transA else M, up(M) if transA else K, a.lda) + zb(strideA), "gemm A", offA)
    _need(B, _span(N if transB else K, K if transB else up(N), a.ldb) + zb(strideB), "gemm B", offB)
    _need(C, _span(M, N, a.ldc) + zb(strideC), "gemm C", offC)
    _need(bias, N, "gemm bias")
    if a_rowsum is not None:
        if a_rowsum.dtype != torch.float32 or not transA or batch1 * batch2 != 1:
            raise TypeError("gemm a_rowsum: float32 vector, transA and a single problem expected")
        _need(a_rowsum, M, "gemm a_rowsum")
    a.a_rowsum = a_rowsum.data_ptr() if a_rowsum is not None else 0
    if relu_mask is not None:
        if relu_mask.dtype != C.dtype:
            raise TypeError("gemm relu_mask: C's element type expected")
        _need(relu_mask, _span(M, N, a.ldc) + zb(strideC), "gemm relu_mask")
    a.c_relu_mask = relu_mask.data_ptr() if relu_mask is not None else 0
    if addend is not None:
        if addend.dtype != C.dtype or not accumulate or batch1 * batch2 != 1:
            raise TypeError("gemm addend: C's element type, accumulate and a single problem expected")
        _need(addend, _span(M, N, a.ldc), "gemm addend")
    a.c_addend = addend.data_ptr() if addend is not None else 0
    if drop is not None:
        p_, rng_state, stream_id = drop
        _dev(rng_state)
        _check_rng(rng_state, "gemm")
        a.drop_state, a.drop_stream_id, a.drop_p = rng_state.data_ptr(), int(stream_id), float(p_)
    if min(strideA + strideB + strideC) < 0:
        raise _lib.HapmiError("gemm: negative batch stride")
    if _gemm_log is not None:
        _gemm_log.append((a, (A, B, C, bias, ws, a_rowsum, relu_mask, addend, drop)))  # the tensors keep the recorded pointers alive
    check(lib().hapmi_gemm(ctypes.byref(a), _stream()))
    return C


def _gemm_segmented(A, B, C, M, N, K, transA, transB, lda, ldb, ldc, bias, act, alpha, workspace, a_rowsum,
                    a_segments, b_segments, c_segments, mask_segments, a_relu, b_relu, accumulate):
    """The forms of ``gemm`` with an operand or the result in pieces (one problem, bf16 operands)."""
    _dev(A, B, C, bias, a_rowsum)
    a = GemmArgs()
    keep = []
    first = lambda *ts: next(t for t in ts if t is not None)
    in_t = first(A, a_segments[0] if a_segments else None, B, b_segments[0] if b_segments else None)
    out_t = first(C, c_segments[0] if c_segments else None)
    epv = 16 // in_t.element_size()
    up = lambda n: (n + epv - 1) // epv * epv
    a.M, a.N, a.K = M, N, K
    a.lda = lda if lda is not None else (M if transA else K)
    a.ldb = ldb if ldb is not None else (K if transB else N)
    a.ldc = ldc if ldc is not None else N
    a.transA, a.transB = int(transA), int(transB)
    a.in_dtype, a.out_dtype = dtype_code(in_t), dtype_code(out_t)
    a.accumulate, a.act, a.alpha = int(accumulate), _ACT[act], float(alpha)
    a.batch1 = a.batch2 = 1
    if a_segments is not None:
        g = _segments(a_segments, M, "gemm a_segments")
        if int(g.begin[g.n]) != K:
            raise ValueError("gemm a_segments: the pieces must add up to K")
        keep.append(g)
        a.A_segments = ctypes.addressof(g)
    else:
        _need(A, _span(K if transA else M, up(M) if transA else K, a.lda), "gemm A")
        a.A = A.data_ptr()
    if b_segments is not None:
        g = _segments(b_segments, K, "gemm b_segments")
        if int(g.begin[g.n]) != N:
            raise ValueError("gemm b_segments: the pieces must add up to N")
        keep.append(g)
        a.B_segments = ctypes.addressof(g)
    else:
        _need(B, _span(N if transB else K, K if transB else up(N), a.ldb), "gemm B")
        a.B = B.data_ptr()
    if c_segments is not None:
        g = _segments(c_segments, M, "gemm c_segments")
        if int(g.begin[g.n]) != N:
            raise ValueError("gemm c_segments: the pieces must add up to N")
        keep.append(g)
        a.C_segments = ctypes.addressof(g)
        if mask_segments is not None:
            gm = _segments(mask_segments, M, "gemm mask_segments")
            keep.append(gm)
            a.c_mask_segments = ctypes.addressof(gm)
    else:
        _need(C, _span(M, N, a.ldc), "gemm C")
        a.C = C.data_ptr()
    a.a_relu, a.b_relu = int(bool(a_relu)), int(bool(b_relu))
    if bias is not None:
        if bias.dtype != torch.float32:
            raise TypeError("gemm bias must be float32")
        _need(bias, N, "gemm bias")
        a.bias = bias.data_ptr()
    if a_rowsum is not None:
        if a_rowsum.dtype != torch.float32 or not transA:
            raise TypeError("gemm a_rowsum: float32 vector and transA expected")
        _need(a_rowsum, M, "gemm a_rowsum")
        a.a_rowsum = a_rowsum.data_ptr()
    ws = workspace if workspace is not None else _gemm_ws
    if ws is None and a_rowsum is not None:
        ws = _workspace(in_t.device)
    if ws is not None and ws.is_cuda:
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    a._keep = tuple(keep)                              # the argument block points into these host structures
    if _gemm_log is not None:
        _gemm_log.append((a, (A, B, C, bias, a_segments, b_segments, c_segments, mask_segments)))
    check(lib().hapmi_gemm(ctypes.byref(a), _stream()))
    return C


def gemm_group(As: Sequence[torch.Tensor], Bs: Sequence[torch.Tensor], Cs: Sequence[torch.Tensor], M: int, N: int,
               K: int, *, transA=False, transB=False, lda=None, ldb=None, ldc=None, accumulate=False, alpha=1.0,
               a_rowsums: Optional[Sequence[Optional[torch.Tensor]]] = None, b_relu=False):
    """``Cs[z] = alpha * op(As[z]) @ op(Bs[z]) (+ Cs[z])`` for up to 16 problems of one shape in one launch
    (pointer lists of the C ABI; no K split).  ``a_rowsums[z]`` as ``a_rowsum`` of ``gemm``.  An entry of ``Bs`` may
    be a list of pieces along N (``b_segments`` of ``gemm``; then every entry must be, with equal piece shapes);
    ``b_relu``: relu applied to op(B) as it is loaded."""
    n = len(As)
    if not (1 <= n <= _lib.GEMM_MAX_LIST and len(Bs) == n and len(Cs) == n and (a_rowsums is None or len(a_rowsums) == n)):
        raise ValueError(f"gemm_group: 1..{_lib.GEMM_MAX_LIST} problems with one entry per list expected")
    pieces = isinstance(Bs[0], (list, tuple))
    seg_structs = None
    if pieces:
        if not all(isinstance(b, (list, tuple)) for b in Bs) or transB:
            raise ValueError("gemm_group: either every B is a list of pieces (transB = False) or none")
        seg_structs = [_segments(b, K, "gemm_group b_segments") for b in Bs]
        Bs = [b[0] for b in Bs]                           # stands for the operand in the checks below
    _dev(*As, *Bs, *Cs, *(a_rowsums or ()))
    a = GemmArgs()
    a.M, a.N, a.K = M, N, K
    a.lda = lda if lda is not None else (M if transA else K)
    a.ldb = ldb if ldb is not None else (K if transB else N)
    a.ldc = ldc if ldc is not None else N
    a.transA, a.transB = int(transA), int(transB)
    a.in_dtype, a.out_dtype = dtype_code(As[0]), dtype_code(Cs[0])
    a.accumulate, a.act, a.alpha = int(accumulate), 0, float(alpha)
    a.batch1, a.batch2 = n, 1
    epv = 16 // As[0].element_size()
    up = lambda v: (v + epv - 1) // epv * epv
    for A, B, C in zip(As, Bs, Cs):
        if A.dtype != As[0].dtype or B.dtype != As[0].dtype or C.dtype != Cs[0].dtype:
            raise TypeError("gemm_group: every problem must have the element types of the first")
        _need(A, _span(K if transA else M, up(M) if transA else K, a.lda), "gemm_group A")
        if not pieces:
            _need(B, _span(N if transB else K, K if transB else up(N), a.ldb), "gemm_group B")
        _need(C, _span(M, N, a.ldc), "gemm_group C")
    for r in a_rowsums or ():
        if r is not None:
            if r.dtype != torch.float32 or not transA:
                raise TypeError("gemm_group a_rowsums: float32 vectors and transA expected")
            _need(r, M, "gemm_group a_rowsum")
    arr = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() if t is not None else None for t in ts])
    la, lb, lc = arr(As), arr(Bs), arr(Cs)
    lr = arr(a_rowsums) if a_rowsums is not None else None
    a.A_list, a.B_list, a.C_list = ctypes.addressof(la), ctypes.addressof(lb), ctypes.addressof(lc)
    a.a_rowsum_list = ctypes.addressof(lr) if lr is not None else 0
    a._keep = (la, lb, lc, lr)                       # the argument block points into these host arrays
    a.b_relu = int(bool(b_relu))
    if seg_structs is not None:
        if any(int(g.begin[g.n]) != N for g in seg_structs):
            raise ValueError("gemm_group b_segments: the pieces must add up to N")
        ls = (ctypes.c_void_p * n)(*[ctypes.addressof(g) for g in seg_structs])
        a.B_segments_list = ctypes.addressof(ls)
        a._keep = a._keep + (ls, tuple(seg_structs))
    if lr is not None:
        ws = _workspace(As[0].device)                  # partial row sums
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
    if _gemm_log is not None:
        _gemm_log.append((a, (tuple(As), tuple(Bs), tuple(Cs), tuple(a_rowsums or ()))))
    check(lib().hapmi_gemm(ctypes.byref(a), _stream()))
    return Cs


_gemm_log = None
_SPLIT_MENU = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16)
_BF16_TILE_CONFIGS = tuple(range(10))
_F32_TILE_CONFIGS = (0, 10, 11)
_THREE_STAGE_CONFIGS = (5, 6, 7, 8, 9)
_TILE_N = {0: 128, 1: 256, 2: 192, 3: 256, 4: 192, 5: 128, 6: 256, 7: 128, 8: 128, 9: 192, 10: 64, 11: 128}


def record_gemms(on: bool):
    """Start (True) or stop (False) recording the argument blocks of every ``gemm`` call; stopping returns
    the list recorded so far."""
    global _gemm_log
    log, _gemm_log = _gemm_log, ([] if on else None)
    return log or []


def autotune_gemm(a: "GemmArgs", flush: Optional[torch.Tensor] = None, repeats: int = 3):
    """Time every tile configuration / K split that is legal for the recorded call ``a`` on its own operands
    and pin the fastest in the library's plan table (``hapmi_gemm_plan_set``).  Each sample is one launch
    bracketed by events after ``flush`` (a buffer larger than the caches) has been overwritten, so operands
    and output start as cold as they are inside a training step.  Returns (config, splits, microseconds)."""
    L = lib()
    batch = a.batch1 * a.batch2
    bf16_in = a.in_dtype == 1
    nk = -(-a.K // (64 if bf16_in else 32))
    per_split = a.M * ((a.N + 3) // 4 * 4) * 4
    max_splits = a.workspace_bytes // per_split if (a.workspace and per_split) else 0
    # calls with an operand or the result in pieces: three-stage configurations only for A in pieces / relu on A,
    # tiles whose N extent divides every piece boundary for B / C in pieces, and no K split
    need3 = bool(a.A_segments) or bool(a.a_relu)
    n_align = 0
    seg_ptrs = [a.B_segments, a.C_segments]
    if a.B_segments_list:
        seg_ptrs.append(ctypes.cast(a.B_segments_list, ctypes.POINTER(ctypes.c_void_p))[0])
    for ptr in seg_ptrs:
        if ptr:
            g = ctypes.cast(ptr, ctypes.POINTER(GemmSegments)).contents
            for i in range(1, g.n):
                n_align = math.gcd(n_align, int(g.begin[i]))
    segmented = need3 or any(seg_ptrs)
    cands = []
    for cfg in (_BF16_TILE_CONFIGS if bf16_in else _F32_TILE_CONFIGS):
        if (need3 and cfg not in _THREE_STAGE_CONFIGS) or (n_align and n_align % _TILE_N[cfg]):
            continue
        for s in _SPLIT_MENU:
            if s > 1 and (segmented or s > max_splits or batch != 1 or nk // s < 4):
                continue
            cands.append((cfg, s))
    stream = _stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = None
    try:
        for cfg, s in cands:
            check(L.hapmi_gemm_tuning(cfg, s))
            check(L.hapmi_gemm(ctypes.byref(a), stream))            # warm-up: code objects, LDS limit
            samples = []
            for _ in range(repeats):
                if flush is not None:
                    flush.add_(1)
                e0.record()
                check(L.hapmi_gemm(ctypes.byref(a), stream))
                e1.record()
                e1.synchronize()
                samples.append(e0.elapsed_time(e1) * 1e3)
            t = sorted(samples)[len(samples) // 2]
            if best is None or t < best[2]:
                best = (cfg, s, t)
    finally:
        check(L.hapmi_gemm_tuning(-1, 0))
    check(L.hapmi_gemm_plan_set(a.M, a.N, a.K, batch, a.transA, a.transB, a.in_dtype, a.out_dtype, best[0], best[1]))
    _pinned_plans[(a.M, a.N, a.K, batch, a.transA, a.transB, a.in_dtype, a.out_dtype)] = (best[0], best[1])
    return best


_pinned_plans = {}      # problem signature -> (tile configuration, K splits), as pinned in the library's plan table


def clear_gemm_plans():
    check(lib().hapmi_gemm_plan_clear())
    _pinned_plans.clear()


def pinned_gemm_plans() -> dict:
    """The plans pinned in this process: (M, N, K, batch, transA, transB, in, out) -> (tile configuration, K splits)."""
    return dict(_pinned_plans)


def save_gemm_plans(path: str) -> int:
    """Write the plans pinned by autotuning in this process as JSON; returns their number."""
    import json
    with open(path, "w") as f:
        json.dump([list(k) + list(v) for k, v in sorted(_pinned_plans.items())], f)
    return len(_pinned_plans)


def load_gemm_plans(path: str) -> int:
    """Pin the plans of a file written by ``save_gemm_plans`` (a tuning run on the same device)."""
    import json
    with open(path) as f:
        rows = json.load(f)
    for row in rows:
        if len(row) != 10:
            raise ValueError(f"{path}: a plan row has {len(row)} fields, 10 expected")
        check(lib().hapmi_gemm_plan_set(*[int(v) for v in row]))
        _pinned_plans[tuple(int(v) for v in row[:8])] = (int(row[8]), int(row[9]))
    return len(rows)


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, out_dtype=None, act=None) -> torch.Tensor:
    """F.linear on a [..., K] input with a [N, K] weight."""
    K = x.shape[-1]
    M = x.numel() // K
    N = w.shape[0]
    out = torch.empty(x.shape[:-1] + (N,), dtype=out_dtype or x.dtype, device=x.device)
    gemm(x, w, out, M, N, K, transB=True, bias=bias, act=act)
    return out


# ---------------------------------------------------------------------------
# row-wise
# ---------------------------------------------------------------------------

def _check_rng(rng_state, what):
    if rng_state is None or rng_state.dtype != torch.int64 or rng_state.numel() < 2:
        raise TypeError(f"{what}: rng_state must hold two int64 (seed, step)")


def add_layernorm_fwd(x, res, y, rstd, eps=1e-5, drop=None):
    """y = LN(x + res); ``drop`` = (p, rng_state, stream_id): y = LN(dropout(x) + res) with the decisions that
    ``dropout`` takes for x under the same three."""
    _dev(x, res, y, rstd)
    width = x.shape[-1]
    rows = x.numel() // width
    for t_ in (x, res, y):
        _need(t_, rows * width, "add_layernorm_fwd")
        if t_ is not None and t_.dtype != x.dtype:
            raise TypeError("add_layernorm_fwd: dtype mismatch")
    _need(rstd, rows, "add_layernorm_fwd rstd")
    if drop is None:
        check(lib().hapmi_add_layernorm_fwd(_ptr(x), _ptr(res), _ptr(y), _ptr(rstd), rows, width,
                                            ctypes.c_float(eps), dtype_code(x), _stream()))
        return
    p, rng_state, stream_id = drop
    _dev(rng_state)
    _check_rng(rng_state, "add_layernorm_fwd")
    check(lib().hapmi_dropout_add_layernorm_fwd(_ptr(x), _ptr(res), _ptr(y), _ptr(rstd), rows, width,
                                                ctypes.c_float(eps), ctypes.c_float(p), _ptr(rng_state),
                                                int(stream_id), dtype_code(x), _stream()))


def layernorm_bwd(dy, y, rstd, dx_add, dx, dx_drop=None, drop=None):
    """``dx_drop`` with ``drop`` = (p, rng_state, stream_id): also the gradient of the operand that went through
    dropout before the add (dropout's backward of dx)."""
    _dev(dy, y, rstd, dx_add, dx, dx_drop)
    width = y.shape[-1]
    rows = y.numel() // width
    for t_ in (dy, y, dx_add, dx, dx_drop):
        _need(t_, rows * width, "layernorm_bwd")
        if t_ is not None and t_.dtype != y.dtype:
            raise TypeError("layernorm_bwd: dtype mismatch")
    _need(rstd, rows, "layernorm_bwd rstd")
    if (dx_drop is None) != (drop is None):
        raise ValueError("layernorm_bwd: dx_drop and drop come together")
    if drop is None:
        check(lib().hapmi_layernorm_bwd(_ptr(dy), _ptr(y), _ptr(rstd), _ptr(dx_add), _ptr(dx), rows, width,
                                        dtype_code(y), _stream()))
        return
    if dx_drop.data_ptr() == dx.data_ptr():
        raise ValueError("layernorm_bwd: dx_drop must not alias dx")
    p, rng_state, stream_id = drop
    _dev(rng_state)
    _check_rng(rng_state, "layernorm_bwd")
    check(lib().hapmi_layernorm_bwd_dropout(_ptr(dy), _ptr(y), _ptr(rstd), _ptr(dx_add), _ptr(dx), _ptr(dx_drop),
                                            rows, width, ctypes.c_float(p), _ptr(rng_state), int(stream_id),
                                            dtype_code(y), _stream()))


def softmax_fwd(x, mask, p, rows, width, ld, mask_rows=1):
    _dev(x, mask, p)
    _need(x, _span(rows, width, ld), "softmax_fwd x")
    _need(p, _span(rows, width, ld), "softmax_fwd p")
    _need(mask, mask_rows * width, "softmax_fwd mask")
    if p.dtype != x.dtype or (mask is not None and mask.dtype != torch.float32):
        raise TypeError("softmax_fwd: dtype mismatch")
    check(lib().hapmi_softmax_fwd(_ptr(x), _ptr(mask), _ptr(p), rows, width, ld, mask_rows, dtype_code(x), _stream()))


def softmax_bwd(dp, p, ds, rows, width, ld):
    _dev(dp, p, ds)
    for t_ in (dp, p, ds):
        _need(t_, _span(rows, width, ld), "softmax_bwd")
        if t_.dtype != p.dtype:
            raise TypeError("softmax_bwd: dtype mismatch")
    check(lib().hapmi_softmax_bwd(_ptr(dp), _ptr(p), _ptr(ds), rows, width, ld, dtype_code(p), _stream()))


def _check_attn(qkv, out, lse, mask, b, S, H):
    E = H * 64
    _need(qkv, b * S * 3 * E, "attention qkv")
    _need(out, b * S * E, "attention out")
    _need(lse, b * H * S, "attention lse")
    _need(mask, S * S, "attention mask")
    if qkv.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or lse.dtype != torch.float32:
        raise TypeError("attention: bf16 qkv / out and float32 lse expected")
    if mask is not None and mask.dtype != torch.float32:
        raise TypeError("attention: float32 mask expected")


def attention_keep_words(b, S, H) -> int:
    """Number of uint32 in each of the two keep-word buffers of attention with dropout."""
    return b * H * S * 2 * ((S + 63) // 64)


def _check_keep(t, b, S, H, what):
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"attention {what}: contiguous int32 words expected")
    _need(t, attention_keep_words(b, S, H), f"attention {what}")


def attention_keep_bits(keep_rows, keep_cols, b, S, H, row_len, p, rng_state, stream_id):
    """The keep decisions of the probabilities' dropout as bit words (int32 tensors of attention_keep_words
    elements): those ``dropout`` takes for a [b*H, S, row_len] tensor under the same (p, rng_state, stream_id)."""
    _dev(keep_rows, keep_cols, rng_state)
    _check_keep(keep_rows, b, S, H, "keep_rows")
    _check_keep(keep_cols, b, S, H, "keep_cols")
    if rng_state.dtype != torch.int64 or rng_state.numel() < 2:
        raise TypeError("attention_keep_bits: rng_state must hold two int64")
    check(lib().hapmi_attention_keep_bits(_ptr(keep_rows), _ptr(keep_cols), b, S, H, row_len, ctypes.c_float(p),
                                          _ptr(rng_state), stream_id, _stream()))


def attention_fwd(qkv, mask, out, lse, b, S, H, scale, causal=False, keep_rows=None, p=0.0):
    """``causal``: the mask is torch.triu(full(-inf), 1); pass ``mask=None`` with it.  ``keep_rows`` (from
    attention_keep_bits) with ``p``: dropout of the probabilities."""
    _dev(qkv, mask, out, lse, keep_rows)
    _check_attn(qkv, out, lse, mask, b, S, H)
    if keep_rows is None:
        check(lib().hapmi_attention_fwd(_ptr(qkv), _ptr(mask), int(causal), _ptr(out), _ptr(lse), b, S, H,
                                        ctypes.c_float(scale), _stream()))
        return
    _check_keep(keep_rows, b, S, H, "keep_rows")
    check(lib().hapmi_attention_fwd_dropout(_ptr(qkv), _ptr(mask), int(causal), _ptr(out), _ptr(lse), b, S, H,
                                            ctypes.c_float(scale), _ptr(keep_rows), ctypes.c_float(p), _stream()))


def attention_bwd(qkv, out, dout, lse, mask, dqkv, delta_ws, b, S, H, scale, causal=False, keep_rows=None,
                  keep_cols=None, p=0.0):
    _dev(qkv, out, dout, lse, mask, dqkv, delta_ws, keep_rows, keep_cols)
    _check_attn(qkv, out, lse, mask, b, S, H)
    _need(dout, b * S * H * 64, "attention dout")
    _need(dqkv, b * S * 3 * H * 64, "attention dqkv")
    _need(delta_ws, b * H * S, "attention delta")
    if dout.dtype != torch.bfloat16 or dqkv.dtype != torch.bfloat16 or delta_ws.dtype != torch.float32:
        raise TypeError("attention_bwd: dtype mismatch")
    if keep_rows is None and keep_cols is None:
        check(lib().hapmi_attention_bwd(_ptr(qkv), _ptr(out), _ptr(dout), _ptr(lse), _ptr(mask), int(causal),
                                        _ptr(dqkv), _ptr(delta_ws), b, S, H, ctypes.c_float(scale), _stream()))
        return
    if keep_rows is None or keep_cols is None:
        raise ValueError("attention_bwd: keep_rows and keep_cols come together")
    _check_keep(keep_rows, b, S, H, "keep_rows")
    _check_keep(keep_cols, b, S, H, "keep_cols")
    check(lib().hapmi_attention_bwd_dropout(_ptr(qkv), _ptr(out), _ptr(dout), _ptr(lse), _ptr(mask), int(causal),
                                            _ptr(dqkv), _ptr(delta_ws), b, S, H, ctypes.c_float(scale),
                                            _ptr(keep_rows), _ptr(keep_cols), ctypes.c_float(p), _stream()))


def head_parallel_attention(x, w_in, b_in, w_out, num_heads, mask=None):
    """Forward of models.head_parallel_attention on GPU tensors: qkv projection of the given heads, softmax
    attention per head, partial output projection (no bias)."""
    _dev(x, w_in, b_in, w_out, mask)
    b, S, d = x.shape
    Ea = w_in.shape[0] // 3
    H = int(num_heads)
    if tuple(w_in.shape) != (3 * Ea, d) or w_out.shape[1] != Ea or H < 1 or Ea % H:
        raise ValueError("head_parallel_attention: projection shapes do not fit the heads")
    hd = Ea // H
    epv = 8 if x.dtype == torch.bfloat16 else 4
    if hd % epv:
        raise ValueError(f"head_parallel_attention: head_dim {hd} must be a multiple of {epv}")
    if mask is not None and (tuple(mask.shape) != (S, S) or mask.dtype != torch.float32):
        raise TypeError("head_parallel_attention: the mask must be a float32 [S, S] additive mask")
    x = x.contiguous()
    wi, wo = w_in.contiguous().to(x.dtype), w_out.contiguous().to(x.dtype)
    Sp = (S + epv - 1) // epv * epv
    M, scale = b * S, 1.0 / math.sqrt(hd)
    qkv = torch.empty(b, S, 3 * Ea, dtype=x.dtype, device=x.device)
    P = torch.empty(b, H, S, Sp, dtype=x.dtype, device=x.device)
    ctx = torch.empty(b, S, Ea, dtype=x.dtype, device=x.device)
    out = torch.empty(b, S, w_out.shape[0], dtype=x.dtype, device=x.device)
    sQ, sP = (S * 3 * Ea, hd), (H * S * Sp, S * Sp)
    gemm(x, wi, qkv, M, 3 * Ea, d, transB=True, bias=b_in.float().contiguous())
    gemm(qkv, qkv, P, S, S, hd, transB=True, lda=3 * Ea, ldb=3 * Ea, ldc=Sp, alpha=scale, batch1=b, batch2=H,
         strideA=sQ, strideB=sQ, strideC=sP, offB=Ea)
    softmax_fwd(P, mask, P, b * H * S, S, Sp, S)
    gemm(P, qkv, ctx, S, hd, S, lda=Sp, ldb=3 * Ea, ldc=Ea, batch1=b, batch2=H, strideA=sP, strideB=sQ,
         strideC=(S * Ea, hd), offB=2 * Ea)
    gemm(ctx, wo, out, M, w_out.shape[0], Ea, transB=True)
    return out


def logsoftmax_nll(logits, targets, row_loss, dlogits, rows, width, ld, ignore_index=-100, grad_scale=1.0):
    _dev(logits, targets, row_loss, dlogits)
    if targets.dtype != torch.int64:
        raise TypeError("targets must be int64")
    _need(logits, _span(rows, width, ld), "logsoftmax_nll logits")
    _need(dlogits, _span(rows, width, ld), "logsoftmax_nll dlogits")
    _need(targets, rows, "logsoftmax_nll targets")
    _need(row_loss, rows, "logsoftmax_nll row_loss")
    if row_loss.dtype != torch.float32 or (dlogits is not None and dlogits.dtype != logits.dtype):
        raise TypeError("logsoftmax_nll: dtype mismatch")
    check(lib().hapmi_logsoftmax_nll(_ptr(logits), _ptr(targets), ignore_index, _ptr(row_loss), _ptr(dlogits), rows,
                                     width, ld, ctypes.c_float(grad_scale), dtype_code(logits), _stream()))


def sum_f32(x, out):
    _dev(x, out)
    if x.dtype != torch.float32 or out.dtype != torch.float32 or out.numel() < 1:
        raise TypeError("sum_f32: float32 buffers expected")
    check(lib().hapmi_sum_f32(_ptr(x), x.numel(), _ptr(out), _stream()))


# ---------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------

def fill_value(t, value: float):
    _dev(t)
    if not t.is_contiguous():
        raise TypeError("fill_value: contiguous tensor expected")
    check(lib().hapmi_fill_value(_ptr(t), ctypes.c_float(value), t.numel(), dtype_code(t), _stream()))


def act_fwd(x, y, act):
    _dev(x, y)
    _need(y, x.numel(), "act_fwd")
    if y.dtype != x.dtype or not x.is_contiguous():
        raise TypeError("act_fwd: dtype / layout mismatch")
    check(lib().hapmi_act_fwd(_ptr(x), _ptr(y), x.numel(), _ACT[act], dtype_code(x), _stream()))


def act_bwd(dy, ref, dx, act):
    _dev(dy, ref, dx)
    _need(ref, dy.numel(), "act_bwd")
    _need(dx, dy.numel(), "act_bwd")
    if ref.dtype != dy.dtype or dx.dtype != dy.dtype:
        raise TypeError("act_bwd: dtype mismatch")
    check(lib().hapmi_act_bwd(_ptr(dy), _ptr(ref), _ptr(dx), dy.numel(), _ACT[act], dtype_code(dy), _stream()))


def add(a, b, out):
    _dev(a, b, out)
    _need(b, a.numel(), "add")
    _need(out, a.numel(), "add")
    if b.dtype != a.dtype or out.dtype != a.dtype:
        raise TypeError("add: dtype mismatch")
    check(lib().hapmi_add(_ptr(a), _ptr(b), _ptr(out), a.numel(), dtype_code(a), _stream()))


def scale(a, s, out):
    _dev(a, out)
    _need(out, a.numel(), "scale")
    if out.dtype != a.dtype:
        raise TypeError("scale: dtype mismatch")
    check(lib().hapmi_scale(_ptr(a), ctypes.c_float(s), _ptr(out), a.numel(), dtype_code(a), _stream()))


def add_bcast_rows(a, b, out, rows, b_rows, width):
    _dev(a, b, out)
    _need(a, rows * width, "add_bcast_rows")
    _need(out, rows * width, "add_bcast_rows")
    _need(b, b_rows * width, "add_bcast_rows")
    if b.dtype != a.dtype or out.dtype != a.dtype:
        raise TypeError("add_bcast_rows: dtype mismatch")
    check(lib().hapmi_add_bcast_rows(_ptr(a), _ptr(b), _ptr(out), rows, b_rows, width, dtype_code(a), _stream()))


def colsum(x, out, M, N, ldx=None, accumulate=False):
    _dev(x, out)
    _need(x, _span(M, N, ldx if ldx is not None else N), "colsum x")
    _need(out, N, "colsum out")
    if out.dtype != torch.float32:
        raise TypeError("colsum: float32 output expected")
    ws = _workspace(x.device)
    check(lib().hapmi_colsum(_ptr(x), _ptr(out), M, N, ldx if ldx is not None else N, int(accumulate),
                             dtype_code(x), _ptr(ws), ws.numel(), _stream()))


def dropout(x, y, p: float, rng_state, stream_id: int):
    """y = x * keep / (1 - p) (F.dropout in training mode); keep = f(rng_state = [seed, step], stream_id, index)."""
    _dev(x, y, rng_state)
    _need(y, x.numel(), "dropout y")
    if x.dtype != y.dtype or rng_state.dtype != torch.int64 or rng_state.numel() < 2:
        raise TypeError("dropout: x and y of one type and an int64[2] state expected")
    check(lib().hapmi_dropout(_ptr(x), _ptr(y), x.numel(), ctypes.c_float(p), _ptr(rng_state), int(stream_id),
                              dtype_code(x), _stream()))


def dropout_mask(n: int, p: float, rng_state, stream_id: int) -> torch.Tensor:
    """The keep decisions (uint8, 1 = kept) that ``dropout`` takes for n elements with this state and stream id."""
    _dev(rng_state)
    mask = torch.empty(n, dtype=torch.uint8, device=rng_state.device)
    check(lib().hapmi_dropout_mask(_ptr(mask), n, ctypes.c_float(p), _ptr(rng_state), int(stream_id), _stream()))
    return mask


def rng_advance(rng_state):
    _dev(rng_state)
    check(lib().hapmi_rng_advance(_ptr(rng_state), _stream()))


def fill_zero(t):
    _dev(t)
    check(lib().hapmi_fill_zero(_ptr(t), t.numel() * t.element_size(), _stream()))


def cast(src, dst):
    _dev(src, dst)
    _need(dst, src.numel(), "cast")
    check(lib().hapmi_cast(_ptr(src), dtype_code(src), _ptr(dst), dtype_code(dst), src.numel(), _stream()))


def embedding_fwd(ids, table, pe, out, S, scale_=1.0):
    _dev(ids, table, pe, out)
    _need(out, ids.numel() * table.shape[1], "embedding_fwd out")
    _need(pe, S * table.shape[1], "embedding_fwd pe")
    if ids.dtype != torch.int64 or out.dtype != table.dtype or (pe is not None and pe.dtype != table.dtype):
        raise TypeError("embedding_fwd: dtype mismatch")
    check(lib().hapmi_embedding_fwd(_ptr(ids), _ptr(table), _ptr(pe), _ptr(out), ids.numel(), table.shape[1], S,
                                    table.shape[0], ctypes.c_float(scale_), dtype_code(table), _stream()))


def embedding_bwd(ids, dout, dtable, scale_=1.0):
    _dev(ids, dout, dtable)
    _need(dout, ids.numel() * dtable.shape[1], "embedding_bwd dout")
    if ids.dtype != torch.int64 or dtable.dtype != torch.float32 or not dtable.is_contiguous():
        raise TypeError("embedding_bwd: dtype mismatch")
    check(lib().hapmi_embedding_bwd(_ptr(ids), _ptr(dout), _ptr(dtable), ids.numel(), dtable.shape[1],
                                    dtable.shape[0], ctypes.c_float(scale_), dtype_code(dout), _stream()))


def patchify(x, cols, b, C, gh, gw, ph, pw):
    _dev(x, cols)
    _need(x, b * C * gh * ph * gw * pw, "patchify x")
    _need(cols, b * C * gh * ph * gw * pw, "patchify cols")
    if x.dtype != torch.float32:
        raise TypeError("patchify: float32 images expected")
    check(lib().hapmi_patchify(_ptr(x), _ptr(cols), b, C, gh, gw, ph, pw, dtype_code(cols), _stream()))


def append_cls_pos(patches, cls, pos, out, b, T, d):
    """``pos`` None: the bare append_cls_token."""
    _dev(patches, cls, pos, out)
    _need(patches, b * T * d, "append_cls_pos patches")
    _need(cls, d, "append_cls_pos cls")
    _need(pos, (T + 1) * d, "append_cls_pos pos")
    _need(out, b * (T + 1) * d, "append_cls_pos out")
    if not (patches.dtype == cls.dtype == out.dtype) or (pos is not None and pos.dtype != out.dtype):
        raise TypeError("append_cls_pos: dtype mismatch")
    check(lib().hapmi_append_cls_pos(_ptr(patches), _ptr(cls), _ptr(pos) if pos is not None else None, _ptr(out), b, T, d,
                                     dtype_code(out), _stream()))


# ---------------------------------------------------------------------------
# optimizer
# ---------------------------------------------------------------------------

def sgd_step(param, grad, shadow, lr, grad_scale=None):
    _dev(param, grad, shadow, grad_scale)
    _need(grad, param.numel(), "sgd_step grad")
    _need(shadow, param.numel(), "sgd_step shadow")
    if param.dtype != torch.float32 or grad.dtype != torch.float32 or (shadow is not None and shadow.dtype != torch.bfloat16):
        raise TypeError("sgd_step: dtype mismatch")
    check(lib().hapmi_sgd_step(_ptr(param), _ptr(grad), _ptr(shadow), param.numel(), ctypes.c_float(lr),
                               _ptr(grad_scale), _stream()))


def adam_step(param, grad, exp_avg, exp_avg_sq, shadow, lr, beta1, beta2, eps, step, grad_scale=None):
    _dev(param, grad, exp_avg, exp_avg_sq, shadow, grad_scale)
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    for t_ in (grad, exp_avg, exp_avg_sq):
        _need(t_, param.numel(), "adam_step")
        if t_.dtype != torch.float32:
            raise TypeError("adam_step: float32 state expected")
    _need(shadow, param.numel(), "adam_step shadow")
    if param.dtype != torch.float32 or (shadow is not None and shadow.dtype != torch.bfloat16):
        raise TypeError("adam_step: dtype mismatch")
    check(lib().hapmi_adam_step(_ptr(param), _ptr(grad), _ptr(exp_avg), _ptr(exp_avg_sq), _ptr(shadow), param.numel(),
                                ctypes.c_float(lr), ctypes.c_float(beta1), ctypes.c_float(beta2), ctypes.c_float(eps),
                                ctypes.c_float(bc1), ctypes.c_float(bc2), _ptr(grad_scale), _stream()))


def adam_step_dev(param, grad, exp_avg, exp_avg_sq, shadow, lr, beta1, beta2, eps, state, grad_scale=None):
    """Adam with the step count / bias corrections in ``state`` (float32[4] on the device, zero at start)."""
    _dev(param, grad, exp_avg, exp_avg_sq, shadow, grad_scale, state)
    for t_ in (grad, exp_avg, exp_avg_sq):
        _need(t_, param.numel(), "adam_step_dev")
        if t_.dtype != torch.float32:
            raise TypeError("adam_step_dev: float32 state expected")
    _need(shadow, param.numel(), "adam_step_dev shadow")
    _need(state, 3, "adam_step_dev state")
    if param.dtype != torch.float32 or state.dtype != torch.float32 or (shadow is not None and shadow.dtype != torch.bfloat16):
        raise TypeError("adam_step_dev: dtype mismatch")
    check(lib().hapmi_adam_step_dev(_ptr(param), _ptr(grad), _ptr(exp_avg), _ptr(exp_avg_sq), _ptr(shadow), param.numel(),
                                    ctypes.c_float(lr), ctypes.c_float(beta1), ctypes.c_float(beta2), ctypes.c_float(eps),
                                    _ptr(state), _ptr(grad_scale), _stream()))


def adam_advance(state, beta1, beta2):
    """Advance the device-side step count / bias corrections once (see ``adam_apply_dev``)."""
    _dev(state)
    _need(state, 3, "adam_advance state")
    check(lib().hapmi_adam_advance(_ptr(state), ctypes.c_float(beta1), ctypes.c_float(beta2), _stream()))


def adam_apply_dev(param, grad, exp_avg, exp_avg_sq, shadow, lr, beta1, beta2, eps, state, grad_scale=None):
    """Adam on one piece of the parameters with the device-side state as it is (``adam_advance`` once per step)."""
    _dev(param, grad, exp_avg, exp_avg_sq, shadow, grad_scale, state)
    for t_ in (grad, exp_avg, exp_avg_sq):
        _need(t_, param.numel(), "adam_apply_dev")
        if t_.dtype != torch.float32:
            raise TypeError("adam_apply_dev: float32 state expected")
    _need(shadow, param.numel(), "adam_apply_dev shadow")
    _need(state, 3, "adam_apply_dev state")
    if param.dtype != torch.float32 or state.dtype != torch.float32 or (shadow is not None and shadow.dtype != torch.bfloat16):
        raise TypeError("adam_apply_dev: dtype mismatch")
    check(lib().hapmi_adam_apply_dev(_ptr(param), _ptr(grad), _ptr(exp_avg), _ptr(exp_avg_sq), _ptr(shadow), param.numel(),
                                     ctypes.c_float(lr), ctypes.c_float(beta1), ctypes.c_float(beta2), ctypes.c_float(eps),
                                     _ptr(state), _ptr(grad_scale), _stream()))


def sumsq_workspace_elems(n: int) -> int:
    need = ctypes.c_int64()
    check(lib().hapmi_sumsq_workspace_elems(n, ctypes.byref(need)))
    return need.value


def sumsq(g, out, workspace=None):
    """out[0] = sum of g^2 (deterministic; ``workspace``: float32 scratch of ``sumsq_workspace_elems(n)``)."""
    ws = workspace if workspace is not None else _workspace(g.device)
    _dev(g, out, ws)
    if ws.dtype != torch.float32 or g.dtype != torch.float32 or out.dtype != torch.float32:
        raise TypeError("sumsq: float32 tensors expected")
    check(lib().hapmi_sumsq(_ptr(g), g.numel(), _ptr(out), _ptr(ws), ws.numel(), _stream()))


def clip_coef(sumsq_t, max_norm, coef):
    _dev(sumsq_t, coef)
    check(lib().hapmi_clip_coef(_ptr(sumsq_t), ctypes.c_float(max_norm), _ptr(coef), _stream()))


# ---------------------------------------------------------------------------
# MoE
# ---------------------------------------------------------------------------

def top2_gate(logits, capacity):
    """logits [B,S,E] float32 -> dict(probs, index, slot, gate, token_of_slot)."""
    _dev(logits)
    B, S, E = logits.shape
    dev = logits.device
    r = dict(probs=torch.empty(B, S, E, dtype=torch.float32, device=dev),
             index=torch.empty(B, S, 2, dtype=torch.int32, device=dev),
             slot=torch.empty(B, S, 2, dtype=torch.int32, device=dev),
             gate=torch.empty(B, S, 2, dtype=torch.float32, device=dev),
             token_of_slot=torch.empty(B, E, capacity, dtype=torch.int32, device=dev))
    top2_gate_into(logits, capacity, r)
    return r


def _check_routing(r, B, S, E=None, C=None):
    _dev(*r.values())
    _need(r["index"], B * S * 2, "routing index")
    _need(r["slot"], B * S * 2, "routing slot")
    _need(r["gate"], B * S * 2, "routing gate")
    if r["index"].dtype != torch.int32 or r["slot"].dtype != torch.int32 or r["gate"].dtype != torch.float32:
        raise TypeError("routing tensors must be int32 / int32 / float32")
    if E is not None:
        _need(r["probs"], B * S * E, "routing probs")
        if C is not None:
            _need(r["token_of_slot"], B * E * C, "routing token_of_slot")
            if r["token_of_slot"].dtype != torch.int32:
                raise TypeError("token_of_slot must be int32")


def top2_gate_into(logits, capacity, r):
    B, S, E = logits.shape
    _dev(logits)
    if logits.dtype != torch.float32 or not logits.is_contiguous():
        raise TypeError("top2_gate: contiguous float32 logits expected")
    _check_routing(r, B, S, E, capacity)
    check(lib().hapmi_top2_gate(_ptr(logits), _ptr(r["probs"]), _ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]),
                                _ptr(r["token_of_slot"]), B, S, E, capacity, _stream()))


def switch_gate_into(logits, capacity, r):
    """Switch (top-1) gating into top-2-shaped routing records: the second choice of every token is dropped."""
    B, S, E = logits.shape
    _dev(logits)
    if logits.dtype != torch.float32 or not logits.is_contiguous():
        raise TypeError("switch_gate: contiguous float32 logits expected")
    _check_routing(r, B, S, E, capacity)
    check(lib().hapmi_switch_gate(_ptr(logits), _ptr(r["probs"]), _ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]),
                                  _ptr(r["token_of_slot"]), B, S, E, capacity, _stream()))


def switch_gate(logits, capacity):
    """logits [B,S,E] float32 -> dict(probs, index, slot, gate, token_of_slot), one kept choice per token at most."""
    _dev(logits)
    B, S, E = logits.shape
    dev = logits.device
    r = dict(probs=torch.empty(B, S, E, dtype=torch.float32, device=dev),
             index=torch.empty(B, S, 2, dtype=torch.int32, device=dev),
             slot=torch.empty(B, S, 2, dtype=torch.int32, device=dev),
             gate=torch.empty(B, S, 2, dtype=torch.float32, device=dev),
             token_of_slot=torch.empty(B, E, capacity, dtype=torch.int32, device=dev))
    switch_gate_into(logits, capacity, r)
    return r


def top2_gate_bwd(r, dgate, dlogits):
    B, S, E = r["probs"].shape
    _check_routing(r, B, S, E)
    _dev(dgate, dlogits)
    _need(dgate, B * S * 2, "top2_gate_bwd dgate")
    _need(dlogits, B * S * E, "top2_gate_bwd dlogits")
    if dgate.dtype != torch.float32 or dlogits.dtype != torch.float32:
        raise TypeError("top2_gate_bwd: float32 expected")
    check(lib().hapmi_top2_gate_bwd(_ptr(r["probs"]), _ptr(r["index"]), _ptr(r["slot"]), _ptr(dgate), _ptr(dlogits),
                                    B, S, E, _stream()))


def top2_densify(r, E, C):
    B, S, _ = r["index"].shape
    dev = r["index"].device
    dispatch = torch.empty(B, S, E, C, dtype=torch.float32, device=dev)
    combine = torch.empty(B, S, E, C, dtype=torch.float32, device=dev)
    _check_routing(r, B, S)
    check(lib().hapmi_top2_densify(_ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]), _ptr(dispatch), _ptr(combine),
                                   B, S, E, C, _stream()))
    return dispatch, combine


def _capacity_window(C, c_lo, C_loc):
    """(c_lo, C_loc) of the device's capacity slots; None = all of them."""
    c_lo = 0 if c_lo is None else int(c_lo)
    C_loc = C - c_lo if C_loc is None else int(C_loc)
    if c_lo < 0 or C_loc < 0 or c_lo + C_loc > C:
        raise _lib.HapmiError(f"capacity window [{c_lo}, {c_lo + C_loc}) outside [0, {C})")
    return c_lo, C_loc


def _position_window(r, tokens, s_lo):
    """(B, S, S_loc, s_lo, d): the routing ``r`` covers S positions, the token tensor [B, S_loc, d] holds those from
    s_lo on (None: it must hold all of them)."""
    B, S_loc, d = tokens.shape
    S = r["index"].shape[1]
    if s_lo is None:
        if S_loc != S:
            raise _lib.HapmiError(f"a token tensor of {S_loc} positions next to a routing of {S} needs s_lo")
        s_lo = 0
    s_lo = int(s_lo)
    if r["index"].shape[0] != B or s_lo < 0 or s_lo + S_loc > S:
        raise _lib.HapmiError(f"positions [{s_lo}, {s_lo + S_loc}) outside [0, {S}), or batch {B} against {r['index'].shape[0]}")
    return B, S, S_loc, s_lo, d


def moe_dispatch(x, r, expert_in, E, C, e_lo, E_loc, c_lo=None, C_loc=None, s_lo=None):
    """einsum "bsd,bsec->becd" on the experts [e_lo, e_lo + E_loc), capacity slots [c_lo, c_lo + C_loc) and positions
    [s_lo, s_lo + x.shape[1]) of the routing ``r``: expert_in[E_loc, B, C_loc, d]."""
    B, S, S_loc, s_lo, d = _position_window(r, x, s_lo)
    _dev(x, expert_in)
    _check_routing(r, B, S, E, C)
    c_lo, C_loc = _capacity_window(C, c_lo, C_loc)
    _need(expert_in, E_loc * B * C_loc * d, "moe_dispatch expert_in")
    if expert_in.dtype != x.dtype or not x.is_contiguous():
        raise TypeError("moe_dispatch: dtype / layout mismatch")
    check(lib().hapmi_moe_dispatch(_ptr(x), _ptr(r["token_of_slot"]), _ptr(expert_in), B, S, E, C, d, e_lo, E_loc,
                                   c_lo, C_loc, s_lo, S_loc, dtype_code(x), _stream()))


def moe_combine(expert_out, r, out, C, e_lo, E_loc, c_lo=None, C_loc=None, s_lo=None):
    B, S, S_loc, s_lo, d = _position_window(r, out, s_lo)
    _dev(expert_out, out)
    _check_routing(r, B, S)
    c_lo, C_loc = _capacity_window(C, c_lo, C_loc)
    _need(expert_out, E_loc * B * C_loc * d, "moe_combine expert_out")
    if expert_out.dtype != out.dtype or not out.is_contiguous():
        raise TypeError("moe_combine: dtype / layout mismatch")
    check(lib().hapmi_moe_combine(_ptr(expert_out), _ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]), _ptr(out),
                                  B, S, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, dtype_code(out), _stream()))


def moe_combine_bwd(dout, expert_out, r, d_expert_out, dgate, E, C, e_lo, E_loc, c_lo=None, C_loc=None, s_lo=None):
    B, S, S_loc, s_lo, d = _position_window(r, dout, s_lo)
    if not dout.is_contiguous():
        raise TypeError("moe_combine_bwd: dout must be contiguous")
    _dev(dout, expert_out, d_expert_out, dgate)
    _check_routing(r, B, S, E, C)
    c_lo, C_loc = _capacity_window(C, c_lo, C_loc)
    _need(expert_out, E_loc * B * C_loc * d, "moe_combine_bwd expert_out")
    _need(d_expert_out, E_loc * B * C_loc * d, "moe_combine_bwd d_expert_out")
    _need(dgate, B * S * 2, "moe_combine_bwd dgate")
    if not (expert_out.dtype == d_expert_out.dtype == dout.dtype) or dgate.dtype != torch.float32:
        raise TypeError("moe_combine_bwd: dtype mismatch")
    check(lib().hapmi_moe_combine_bwd(_ptr(dout), _ptr(expert_out), _ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]),
                                      _ptr(r["token_of_slot"]), _ptr(d_expert_out), _ptr(dgate), B, S, E, C, d, e_lo,
                                      E_loc, c_lo, C_loc, s_lo, S_loc, dtype_code(dout), _stream()))


def moe_dispatch_bwd(d_expert_in, r, dx, C, e_lo, E_loc, accumulate, c_lo=None, C_loc=None, s_lo=None):
    B, S, S_loc, s_lo, d = _position_window(r, dx, s_lo)
    _dev(d_expert_in, dx)
    _check_routing(r, B, S)
    c_lo, C_loc = _capacity_window(C, c_lo, C_loc)
    _need(d_expert_in, E_loc * B * C_loc * d, "moe_dispatch_bwd d_expert_in")
    if d_expert_in.dtype != dx.dtype or not dx.is_contiguous():
        raise TypeError("moe_dispatch_bwd: dtype / layout mismatch")
    check(lib().hapmi_moe_dispatch_bwd(_ptr(d_expert_in), _ptr(r["index"]), _ptr(r["slot"]), _ptr(r["gate"]), _ptr(dx),
                                       B, S, C, d, e_lo, E_loc, c_lo, C_loc, s_lo, S_loc, int(accumulate), dtype_code(dx),
                                       _stream()))


# ---------------------------------------------------------------------------
# leaf ops with autograd, for direct (eager) use of the emitted graph's callables
# ---------------------------------------------------------------------------

class _AppendCls(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cls_token):
        _dev(x, cls_token)
        b, T, d = x.shape
        out = torch.empty(b, T + 1, d, dtype=x.dtype, device=x.device)
        zeros = torch.zeros(T + 1, d, dtype=x.dtype, device=x.device)
        append_cls_pos(x.contiguous(), cls_token.contiguous(), zeros, out, b, T, d)
        return out

    @staticmethod
    def backward(ctx, g):
        g = g.contiguous()
        b, T1, d = g.shape
        dx = slice_rows(g, 1, 1, T1 - 1)
        dcls = torch.empty(d, dtype=torch.float32, device=g.device)
        colsum(g, dcls, b, d, ldx=T1 * d)
        return dx, dcls.to(g.dtype).view(1, 1, d)


def append_cls_token(x, cls_token):
    return _AppendCls.apply(x, cls_token)


class _GetCls(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        _dev(x)
        ctx.shape = x.shape
        b, T, d = x.shape
        return slice_rows(x.contiguous().view(b, T, d), 1, 0, 1).view(b, d)

    @staticmethod
    def backward(ctx, g):
        b, T, d = ctx.shape
        dx = torch.empty(b, T, d, dtype=g.dtype, device=g.device)
        fill_zero(dx)
        place_rows(g.contiguous().view(b, 1, d), dx, 1, 0)
        return dx


def get_cls_token(x):
    return _GetCls.apply(x)


def top_2_gating_dense(gate_input, n_expert, capacity, gate_weight):
    """Dense (dispatch, combine) [B,S,E,C] from the index-form gate kernel (forward only)."""
    _dev(gate_input, gate_weight)
    B, S, d = gate_input.shape
    x = gate_input.contiguous()
    w = gate_weight.contiguous().to(x.dtype)
    logits = torch.empty(B, S, n_expert, dtype=torch.float32, device=x.device)
    if n_expert % 4 != 0:
        raise _lib.HapmiError("top_2_gating: n_expert must be a multiple of 4")
    gemm(x, w, logits, B * S, n_expert, d)
    r = top2_gate(logits, capacity)
    return top2_densify(r, n_expert, capacity)


def switch_gating_dense(gate_input, n_expert, capacity, gate_weight):
    """Dense (dispatch, combine) [B,S,E,C] of switch gating from the index-form kernel (forward only)."""
    _dev(gate_input, gate_weight)
    B, S, d = gate_input.shape
    x = gate_input.contiguous()
    w = gate_weight.contiguous().to(x.dtype)
    if n_expert % 4 != 0:
        raise _lib.HapmiError("switch_gating: n_expert must be a multiple of 4")
    logits = torch.empty(B, S, n_expert, dtype=torch.float32, device=x.device)
    gemm(x, w, logits, B * S, n_expert, d)
    return top2_densify(switch_gate(logits, capacity), n_expert, capacity)
