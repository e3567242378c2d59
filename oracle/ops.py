"""CPU restatements of the reference leaf functions.  TEST INFRASTRUCTURE ONLY.

Everything here runs on the CPU with stock PyTorch / numpy and is used solely
as the checker for the HIP path (tests/, smoke(), bench.py's cpu_baseline).

Functions and the reference lines they follow:

* ``sharding_round``       -- /root/reference/hap.rs:3536-3559 (C restatement in
  oracle/sharding_round.c, loaded through ctypes).
* ``positional_encoding``  -- /root/reference/models.py:504-509.
* ``top_2_gating``         -- /root/reference/models.py:477-502.
* ``switch_gating``        -- /root/reference/models.py:452-475.
* ``gating_slots``         -- the integer part of both (models.py:483-491, 458-466) in index form, in C
  (oracle/gating_slots.c).
* ``attention_with_dropped_probabilities`` -- F.multi_head_attention_forward's explicit path
  (torch:nn/functional.py:6435-6612, the call emitted at hap.rs:1301-1321) with a given dropout mask.
* ``head_parallel_attention`` -- no reference counterpart (the reference shards
  attention over the batch only): softmax attention of a subset of heads.
* ``JointWorld`` collectives -- /root/reference/collectives.py:6-29 (padded,
  AllGather), 73-84 (AllReduce), 88-103 (ReduceScatter), 146-148
  (dynamic_slice), 152-166 (AllToAll), 171-180 (Replicate).

The reference's arithmetic lives in PyTorch (environment.yml pins 1.13.1); the
oracle calls the same public PyTorch routines on the CPU.

Pins (see tests/test_oracle_*.py): sharding_round -- hand-derived known
answers + invariants; positional_encoding -- closed form at chosen points;
top_2_gating -- hand-worked routing vector, per-token brute force, slot
invariants; switch_gating -- hand-worked routing vector, per-token brute force,
slot invariants, agreement with the first choices of top_2_gating; collectives -- the ones-tensor expectations the reference keeps in
collectives.py:195-323, round-trip identities.  Tie order of equal gate
probabilities inside torch.topk is unspecified by PyTorch: parity unpinned for
exact ties (they do not occur for the seeded continuous inputs used).
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import List, Sequence

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_liboracle = None


def _lib():
    global _liboracle
    if _liboracle is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            import subprocess
            subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])
        _liboracle = ctypes.CDLL(path)
        _liboracle.oracle_sharding_round.restype = ctypes.c_int
        _liboracle.oracle_sharding_round.argtypes = [
            ctypes.c_int64, ctypes.POINTER(ctypes.c_double), ctypes.c_int64,
            ctypes.POINTER(ctypes.c_int64)]
        i64p = ctypes.POINTER(ctypes.c_int64)
        _liboracle.oracle_gating_slots.restype = ctypes.c_int
        _liboracle.oracle_gating_slots.argtypes = [i64p] + [ctypes.c_int64] * 5 + [i64p, i64p]
    return _liboracle


def sharding_round(full_length: int, ratios: Sequence[float]) -> List[int]:
    """hap.rs:3536-3559.  Returns the integer lengths (does not mutate)."""
    n = len(ratios)
    r = (ctypes.c_double * n)(*[float(x) for x in ratios])
    out = (ctypes.c_int64 * n)()
    rc = _lib().oracle_sharding_round(int(full_length), r, n, out)
    if rc != 0:
        raise AssertionError("truncated lengths exceed full_length (hap.rs:3543)")
    return [int(v) for v in out]


def positional_encoding(seqlen: int, emsize: int) -> np.ndarray:
    """models.py:504-509: angle = pos / 10000^(2*(j//2)/emsize); even columns
    take sin, odd columns cos; float64."""
    pos = np.arange(seqlen, dtype=np.float64)[:, None]
    j = np.arange(emsize)[None, :]
    angle = pos / np.power(10000.0, 2.0 * (j // 2) / emsize)
    out = np.empty_like(angle)
    out[:, 0::2] = np.sin(angle[:, 0::2])
    out[:, 1::2] = np.cos(angle[:, 1::2])
    return out


def densify_vectorised(index, slot, gate, n_expert: int, capacity: int):
    """``densify`` without Python loops (any number of choices per token): combine[b, s, index_k, slot_k] = gate_k
    for every kept choice, dispatch = combine > 0."""
    B, S, k = index.shape
    combine = torch.zeros(B, S, n_expert, capacity, dtype=gate.dtype)
    b, s, j = (slot > 0).nonzero(as_tuple=True)
    combine.index_put_((b, s, index[b, s, j], slot[b, s, j]), gate[b, s, j], accumulate=True)
    return (combine > 0).to(torch.float32), combine


# --------------------------------------------------------------------------
# top-2 gating
# --------------------------------------------------------------------------

def top_2_gating(gate_input, n_expert: int, capacity: int, gate_weight, train: bool = True, index=None):
    """models.py:477-502, dense form: returns (dispatch, combine), each
    [B, S, E, C]; dispatch is float32, combine carries the gate dtype.
    ``index`` (not in the reference): expert choices [B, S, 2] to use instead of topk's own, for a run that must
    share its discrete decisions with another run; the gates are still this run's probabilities of those experts."""
    logits = gate_input @ gate_weight                                  # :478
    probs = torch.softmax(logits, dim=2)                               # :479
    if index is None:
        gate, index = probs.topk(2, dim=2)                             # :481  [B,S,2]
    else:
        gate = probs.gather(2, index)
    chosen = F.one_hot(index, n_expert)                                # :483  [B,S,2,E] int64
    pos = chosen.cumsum(dim=1) * chosen                                # :485  1-based, per choice
    first_sum = pos[:, :, 0, :].sum(dim=1, keepdim=True)               # :486  sum of positions (n(n+1)/2)
    pos = torch.stack([pos[:, :, 0, :], pos[:, :, 1, :] + first_sum], dim=2) * chosen   # :487-488
    fits = pos < capacity                                              # :490-491
    kept = chosen * fits
    pos = pos * fits
    kept_flag = kept.sum(dim=3)                                        # :493  [B,S,2]
    weight = (gate * kept_flag)[:, :, :, None, None]                   # :496
    combine = (weight * F.one_hot(index, n_expert)[..., None]          # :497
               * F.one_hot(pos, capacity)).sum(dim=2)                  # :498
    dispatch = (combine > 0).to(torch.float32)                         # :500
    return dispatch, combine


def gating_slots(index: torch.Tensor, n_expert: int, capacity: int):
    """The integer part of models.py:483-491 (top-2) / 458-466 (switch) in index form, in C
    (oracle/gating_slots.c): ``index`` [B, S, k] int64 -> (slot [B, S, k] with 0 = dropped, token_of_slot [B, E, C]
    with -1 = empty)."""
    index = index.to(torch.int64).contiguous()
    B, S, k = index.shape
    slot = torch.zeros(B, S, k, dtype=torch.int64)
    tos = torch.empty(B, n_expert, capacity, dtype=torch.int64)
    i64p = ctypes.POINTER(ctypes.c_int64)
    rc = _lib().oracle_gating_slots(ctypes.cast(index.data_ptr(), i64p), B, S, n_expert, capacity, k,
                                    ctypes.cast(slot.data_ptr(), i64p), ctypes.cast(tos.data_ptr(), i64p))
    if rc != 0:
        raise ValueError("gating_slots: an expert index lies outside [0, n_expert)")
    return slot, tos


def head_parallel_attention(x, in_proj_weight, in_proj_bias, out_proj_weight, num_heads: int, attn_mask=None):
    """Self-attention over a subset of a layer's heads, written out with plain tensor operations: the rows of
    the packed in-projection are [q; k; v] of those heads, the out-projection holds their columns, and the
    result is the partial output without the output bias.  (No reference counterpart; pinned by the identity
    that the partial outputs of a partition of the heads plus the bias add up to
    F.multi_head_attention_forward of the whole layer.)"""
    b, S, _d = x.shape
    Ea = in_proj_weight.shape[0] // 3
    hd = Ea // num_heads
    qkv = x @ in_proj_weight.t() + in_proj_bias
    q, k, v = (t.reshape(b, S, num_heads, hd).transpose(1, 2) for t in qkv.split(Ea, dim=2))
    scores = (q @ k.transpose(2, 3)) / math.sqrt(hd)
    if attn_mask is not None:
        scores = scores + attn_mask.to(scores.dtype)
    ctx = (torch.softmax(scores.float(), dim=3).to(v.dtype) @ v).transpose(1, 2).reshape(b, S, Ea)
    return ctx @ out_proj_weight.t()


def attention_with_dropped_probabilities(query, in_proj_weight, in_proj_bias, out_proj_weight, out_proj_bias,
                                         num_heads: int, attn_mask, keep, p: float):
    """The explicit path of F.multi_head_attention_forward for self-attention (packed in-projection, baddbmm /
    softmax / dropout / bmm, out-projection: torch:nn/functional.py:6435, 6504-6519, 6576-6612) with the dropout
    of the probabilities written as a multiplication with a GIVEN keep mask: ``keep`` [N, H, L, S] (bool) and
    the probability ``p`` it was drawn with, so P becomes P * keep / (1 - p).  ``query`` is (L, N, E) as in the
    emitted node (hap.rs:1301-1321); returns the attention output (L, N, E).  Pinned by: with keep all ones and
    p = 0 it is F.multi_head_attention_forward(dropout_p = 0); a dropped probability removes exactly that key's
    value from that query's output (tests/test_oracle_attention.py)."""
    L, N, E = query.shape
    hd = E // num_heads
    qkv = F.linear(query, in_proj_weight, in_proj_bias)
    q, k, v = qkv.split(E, dim=2)
    heads = lambda t: t.reshape(L, N * num_heads, hd).transpose(0, 1)          # [N*H, L, hd]
    q, k, v = heads(q), heads(k), heads(v)
    scores = (q * (1.0 / math.sqrt(hd))) @ k.transpose(1, 2)
    if attn_mask is not None:
        scores = scores + attn_mask.to(scores.dtype)
    probs = torch.softmax(scores.float(), dim=2).to(v.dtype)
    scale = 1.0 / (1.0 - p) if p < 1.0 else 0.0
    probs = (probs.float() * (keep.reshape(N * num_heads, L, -1).float() * scale)).to(v.dtype)
    ctx = (probs @ v).transpose(0, 1).reshape(L * N, E)
    return F.linear(ctx, out_proj_weight, out_proj_bias).view(L, N, E)


# --------------------------------------------------------------------------
# dropout keep decisions (this build's own counter-based definition; the reference draws from torch's generator,
# hap.rs:1464, whose stream a GPU kernel cannot reproduce)
# --------------------------------------------------------------------------

def _mix32(x):
    """numpy uint32 restatement of the multiply-xorshift mixer (wrapping arithmetic)."""
    x = np.asarray(x, dtype=np.uint64) & 0xFFFFFFFF
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7feb352d)) & np.uint64(0xFFFFFFFF)
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846ca68b)) & np.uint64(0xFFFFFFFF)
    x ^= x >> np.uint64(16)
    return x


def dropout_keep(seed: int, step: int, stream_id: int, p: float, n: int) -> torch.Tensor:
    """Keep decisions (bool[n]) of the product's dropout for elements 0..n-1: element i is kept iff the 16 random
    bits that the pair i // 2 yields for it (low half: even element, high half: odd element) are >= round(p * 65536);
    the pair's 32 bits are two rounds of mixing of (pair index, key) and the key is a mix of seed, step and stream id.
    Pinned by the statistics any dropout mask must have (keep rate within the binomial bound, no correlation
    between neighbours, between steps, between streams: tests/test_oracle_dropout.py); the GPU kernels must give
    exactly these bits (tests/test_gpu_dropout.py)."""
    M = 0xFFFFFFFF
    seed, step, stream_id = seed & 0xFFFFFFFFFFFFFFFF, step & 0xFFFFFFFFFFFFFFFF, stream_id & 0xFFFFFFFFFFFFFFFF
    k = int(_mix32((seed & M) ^ 0x9e3779b9))
    k = int(_mix32(k ^ (seed >> 32)))
    k = int(_mix32(k ^ (step & M)))
    k = int(_mix32(k ^ (step >> 32) ^ 0x85ebca6b))
    k = int(_mix32(k ^ (stream_id & M)))
    k0 = k
    k1 = int(_mix32(k ^ 0xc2b2ae35 ^ (stream_id >> 32)))
    t = float(np.float32(p) * np.float32(65536.0) + np.float32(0.5))
    thr = 0 if t <= 0 else (65536 if t >= 65536.0 else int(t))
    j = np.arange((n + 1) // 2, dtype=np.uint64)
    inner = _mix32(((j & np.uint64(M)) + np.uint64(k0)) & np.uint64(M))
    hi = (((j >> np.uint64(32)) * np.uint64(0x9e3779b9)) + np.uint64(k1)) & np.uint64(M)
    bits = _mix32(inner ^ hi)
    halves = np.stack([bits & np.uint64(0xFFFF), bits >> np.uint64(16)], axis=1).reshape(-1)[:n]
    return torch.from_numpy(halves >= np.uint64(thr))


def switch_gating(gate_input, n_expert: int, capacity: int, gate_weight, train: bool = True):
    """models.py:452-475, dense form: returns (dispatch, combine), each
    [B, S, E, C]; one expert per token, kept while its 1-based position among
    the earlier tokens of that expert is below the capacity."""
    logits = gate_input @ gate_weight                                  # :453
    probs = torch.softmax(logits, dim=2)                               # :454
    gate, index = probs.topk(1, dim=2)                                 # :456
    gate, index = gate.squeeze(2), index.squeeze(2)                    # :457-458  [B,S]
    chosen = F.one_hot(index, n_expert)                                # :460  [B,S,E] int64
    pos = chosen.cumsum(dim=1) * chosen                                # :462  1-based
    fits = pos < capacity                                              # :463-464
    kept = chosen * fits
    pos = pos * fits
    kept_flag = kept.sum(dim=2)                                        # :466  [B,S]
    combine = ((gate * kept_flag)[:, :, None, None]                    # :469
               * F.one_hot(index, n_expert)[..., None]                 # :470
               * F.one_hot(pos, capacity))                             # :471  one_hot over [B,S,E] -> [B,S,E,C]
    dispatch = (combine > 0).to(torch.float32)                         # :473
    return dispatch, combine


def switch_gating_sparse(logits: torch.Tensor, capacity: int):
    """Per-token brute force over fp32 logits [B,S,E] (pure Python loops; small
    inputs only).  Returns (index[B,S] int64, slot[B,S] int64 with 0 =
    dropped, gate[B,S] float)."""
    B, S, E = logits.shape
    probs = torch.softmax(logits, dim=2)
    index = torch.zeros(B, S, dtype=torch.int64)
    slot = torch.zeros(B, S, dtype=torch.int64)
    gate = torch.zeros(B, S, dtype=probs.dtype)
    for b in range(B):
        seen = [0] * E
        for s in range(S):
            row = probs[b, s].tolist()
            e = min(range(E), key=lambda i: (-row[i], i))
            index[b, s], gate[b, s] = e, probs[b, s, e]
            seen[e] += 1
            slot[b, s] = seen[e] if seen[e] < capacity else 0
    return index, slot, gate


def top_2_gating_sparse(logits: torch.Tensor, capacity: int):
    """Per-token brute force over fp32 logits [B,S,E] (pure Python loops; small
    inputs only).  Returns (index[B,S,2] int64, slot[B,S,2] int64 with 0 =
    dropped, gate[B,S,2] float)."""
    B, S, E = logits.shape
    probs = torch.softmax(logits, dim=2)
    index = torch.zeros(B, S, 2, dtype=torch.int64)
    slot = torch.zeros(B, S, 2, dtype=torch.int64)
    gate = torch.zeros(B, S, 2, dtype=probs.dtype)
    for b in range(B):
        seen0 = [0] * E
        for s in range(S):
            row = probs[b, s].tolist()
            order = sorted(range(E), key=lambda e: (-row[e], e))
            index[b, s, 0], index[b, s, 1] = order[0], order[1]
            gate[b, s, 0], gate[b, s, 1] = probs[b, s, order[0]], probs[b, s, order[1]]
            seen0[order[0]] += 1
            p = seen0[order[0]]
            slot[b, s, 0] = p if p < capacity else 0
        offset = [n * (n + 1) // 2 for n in seen0]
        seen1 = [0] * E
        for s in range(S):
            e = int(index[b, s, 1])
            seen1[e] += 1
            p = seen1[e] + offset[e]
            slot[b, s, 1] = p if p < capacity else 0
    return index, slot, gate


def densify(index, slot, gate, n_expert: int, capacity: int):
    """Sparse routing -> dense (dispatch, combine) as the reference lays them out."""
    B, S, _ = index.shape
    combine = torch.zeros(B, S, n_expert, capacity, dtype=gate.dtype)
    for b in range(B):
        for s in range(S):
            for k in range(2):
                c = int(slot[b, s, k])
                if c > 0:
                    combine[b, s, int(index[b, s, k]), c] += gate[b, s, k]
    return (combine > 0).to(torch.float32), combine


# --------------------------------------------------------------------------
# uneven collectives over an in-memory world of W ranks
# --------------------------------------------------------------------------

def _padded(t: torch.Tensor, dim: int, length: int) -> torch.Tensor:
    """collectives.py:9-12.  The reference leaves the tail uninitialised
    (torch.empty); the oracle poisons it with NaN so that any read of it shows."""
    if t.shape[dim] == length:
        return t
    shape = list(t.shape)
    shape[dim] = length - t.shape[dim]
    tail = torch.full(shape, float("nan"), dtype=t.dtype)
    return torch.cat([t, tail], dim=dim)


def _accumulate(parts: Sequence[torch.Tensor]) -> torch.Tensor:
    """Elementwise sum over ranks in rank order with float32 accumulation."""
    acc = parts[0].float().clone()
    for p in parts[1:]:
        acc = acc + p.float()
    return acc.to(parts[0].dtype)


def _snapshot(messages):
    """Detached copies for the wire log: a message that needed no padding or splitting is the sender's own tensor
    (a parameter, when parameters are gathered), which a later optimizer step would change under the log."""
    if isinstance(messages, torch.Tensor):
        return messages.detach().clone()
    return [_snapshot(m) for m in messages]


class JointWorld:
    """All W ranks of the SPMD program live in one process; each collective is
    one autograd node over the W per-rank tensors, so one backward pass yields
    every rank's gradients.  ``log[(tag, 'fwd'|'bwd')]`` records what went over
    the wire: ``log[key][src][dst]`` is the message rank ``src`` sent to ``dst``."""

    def __init__(self, world_size: int):
        self.W = world_size
        self.log = {}

    # -- all_gather: collectives.py:14-29 --------------------------------
    def all_gather(self, tag, xs, dim, L):
        world = self

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *xs):
                m = max(L)
                sent = [_padded(x, dim, m).contiguous() for x in xs]                    # :19
                world.log[(tag, "fwd")] = _snapshot([[sent[src] for _ in range(world.W)] for src in range(world.W)])
                out = torch.cat([s.split([l, m - l], dim=dim)[0] for s, l in zip(sent, L)], dim=dim)  # :20
                return tuple(out.clone() for _ in range(world.W))

            @staticmethod
            def backward(ctx, *gs):
                m = max(L)
                sent = [[_padded(p, dim, m).contiguous() for p in torch.split(g.contiguous(), L, dim=dim)]
                        for g in gs]                                                       # :24-25
                world.log[(tag, "bwd")] = _snapshot(sent)
                outs = []
                for r in range(world.W):
                    red = _accumulate([sent[src][r] for src in range(world.W)])            # :27
                    outs.append(red.split([L[r], m - L[r]], dim=dim)[0])                   # :28
                return tuple(outs)

        return list(Fn.apply(*xs))

    # -- reduce_scatter: collectives.py:88-103 ---------------------------
    def reduce_scatter(self, tag, xs, dim, L):
        world = self

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *xs):
                m = max(L)
                sent = [[_padded(p, dim, m).contiguous() for p in torch.split(x.contiguous(), L, dim=dim)]
                        for x in xs]                                                       # :92-93
                world.log[(tag, "fwd")] = _snapshot(sent)
                outs = []
                for r in range(world.W):
                    red = _accumulate([sent[src][r] for src in range(world.W)])            # :95
                    outs.append(red.split([L[r], m - L[r]], dim=dim)[0].clone())           # :96
                return tuple(outs)

            @staticmethod
            def backward(ctx, *gs):
                m = max(L)
                sent = [_padded(g.contiguous(), dim, m).contiguous() for g in gs]          # :101
                world.log[(tag, "bwd")] = _snapshot([[sent[src] for _ in range(world.W)] for src in range(world.W)])
                grad = torch.cat([s.split([l, m - l], dim=dim)[0] for s, l in zip(sent, L)], dim=dim)  # :102
                return tuple(grad.clone() for _ in range(world.W))

        return list(Fn.apply(*xs))

    # -- all_to_all: collectives.py:152-166 ------------------------------
    def all_to_all(self, tag, xs, split_dim, cat_dim, split_L, cat_L):
        world = self

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *xs):
                sent = [[p.contiguous() for p in torch.split(x.contiguous(), split_L, dim=split_dim)]
                        for x in xs]                                                       # :156-158
                world.log[(tag, "fwd")] = _snapshot(sent)
                return tuple(torch.cat([sent[src][r] for src in range(world.W)], dim=cat_dim)  # :159
                             for r in range(world.W))

            @staticmethod
            def backward(ctx, *gs):
                sent = [[p.contiguous() for p in torch.split(g.contiguous(), cat_L, dim=cat_dim)]
                        for g in gs]                                                       # :163-165
                world.log[(tag, "bwd")] = _snapshot(sent)
                return tuple(torch.cat([sent[src][r] for src in range(world.W)], dim=split_dim)  # :166
                             for r in range(world.W))

        return list(Fn.apply(*xs))

    # -- all_reduce: collectives.py:73-84 --------------------------------
    def all_reduce(self, tag, xs):
        world = self

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *xs):
                sent = [x.contiguous() for x in xs]
                world.log[(tag, "fwd")] = _snapshot([[sent[src] for _ in range(world.W)] for src in range(world.W)])
                total = _accumulate(sent)
                return tuple(total.clone() for _ in range(world.W))

            @staticmethod
            def backward(ctx, *gs):
                sent = [g.clone() for g in gs]
                world.log[(tag, "bwd")] = _snapshot([[sent[src] for _ in range(world.W)] for src in range(world.W)])
                total = _accumulate(sent)
                return tuple(total.clone() for _ in range(world.W))

        return list(Fn.apply(*xs))

    # -- replicate: collectives.py:171-180 -------------------------------
    def replicate(self, tag, xs):
        world = self

        class Fn(torch.autograd.Function):
            @staticmethod
            def forward(ctx, *xs):
                return tuple(x.view_as(x) for x in xs)

            @staticmethod
            def backward(ctx, *gs):
                sent = [g.contiguous() for g in gs]
                world.log[(tag, "bwd")] = _snapshot([[sent[src] for _ in range(world.W)] for src in range(world.W)])
                total = _accumulate(sent)
                return tuple(total.clone() for _ in range(world.W))

        return list(Fn.apply(*xs))

    # -- dynamic_slice: collectives.py:146-148 (local, no wire) ----------
    @staticmethod
    def dynamic_slice(x, dim, L, rank):
        return torch.split(x, L, dim=dim)[rank].contiguous()
