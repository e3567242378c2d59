"""Executor of one device's SPMD program on MI355X.

``compile_program(graph_module, ...)`` walks the ``torch.fx`` graph that HAP's
synthesizer emits (node forms: /root/reference/hap.rs:991-2324, 2466-2746) ONCE
and turns it into two static lists of kernel launches -- forward and backward
-- over buffers that are allocated up front.  A training step is then a fixed
sequence of HIP kernel launches through the C ABI of libhapmi.so (no autograd
graph, no allocation, no host synchronisation), which is also what a HIP graph
can capture.  The reference runs the same graph through PyTorch eager +
autograd (/root/reference/worker.py:44-76).

Fusions done while walking the graph (results equal the unfused program):
``operator.add`` + ``F.layer_norm`` -> one kernel; ``transpose`` around
``F.multi_head_attention_forward`` -> folded into strides; ``F.dropout(p=0)``
-> alias; ``all_to_all`` + ``F.relu`` -> activation inside the concat;
``torch.log_softmax`` + ``transpose`` + ``F.nll_loss`` -> one kernel that also
writes d(logits); ``top_2_gating`` + ``dynamic_slice`` + the four einsums ->
index-form gather / grouped GEMM / weighted gather; ``conv2d`` (kernel = stride)
+ ``flatten`` + ``transpose`` -> patch rows + GEMM; ``append_cls_token`` +
``operator.add(pos_embed)`` -> one kernel.

bf16 mode: float32 master parameters in one flat buffer, a bf16 shadow of it
that the GEMMs read, bf16 activations and activation gradients, float32
parameter gradients / statistics / loss / gate probabilities.
"""
from __future__ import annotations

import math
import operator
from typing import Callable, Dict, List, Optional

import torch
import torch.fx
import torch.nn.functional as F

from . import collectives, models, ops
from .wire import SilentWire, Wire

_EPS = 1e-5


class Val:
    """Compile-time description of a program value."""

    def __init__(self, kind: str, t: Optional[torch.Tensor] = None, shape=None, **kw):
        self.kind = kind            # 'tensor' | 'param' | 'input' | lazy kinds
        self.t = t                  # storage (static buffer) for materialised values
        self.shape = tuple(shape) if shape is not None else (tuple(t.shape) if t is not None else None)
        self.ld = kw.pop("ld", None)        # row stride when the last dim is padded in storage
        self.grad: Optional[torch.Tensor] = None
        self.needs_grad = kw.pop("needs_grad", False)
        self.meta = kw


def _round_up(n, m):
    return (n + m - 1) // m * m


class ShardExecutor:
    def __init__(self, gm: torch.fx.GraphModule, example_inputs, dtype: str = "fp32", wire: Optional[Wire] = None,
                 rank: int = 0, world_size: int = 1, device: str = "cuda:0", fused_attention: bool = True,
                 overlap_wgrad: bool = False, launch_lists: bool = True, relu_mask_in_dgrad: bool = True,
                 overlap_optimizer: bool = False, optimizer_chunk_min: int = 1 << 20,
                 relu_bwd_in_split: bool = True, wgrad_group: int = 8, receive_in_place: bool = True,
                 dropout_seed: int = 0, exchange_in_pieces: bool = True, fuse_dropout: bool = True):
        """``example_inputs``: the program's inputs (global batch) as tensors or shapes; activations are
        sized from them.  ``rank`` / ``world_size`` are only needed by all_reduce / replicate, whose node
        forms do not carry them (collectives.py:86, 182)."""
        if dtype not in ("fp32", "bf16"):
            raise ValueError("dtype must be 'fp32' or 'bf16'")
        if not torch.cuda.is_available():
            raise ops._lib.HapmiError("no GPU visible: the shard executor has no CPU path")
        ops.init()
        self.gm = gm
        self.dev = torch.device(device)
        self.cdt = torch.float32 if dtype == "fp32" else torch.bfloat16
        self.dtype = dtype
        self.epv = 4 if dtype == "fp32" else 8
        self.wire = wire if wire is not None else SilentWire()
        self.fwd: List[Callable[[], None]] = []
        self.bwd: List[Callable[[], None]] = []
        self._tape: List[Callable[[], None]] = []      # backward emitters, run in reverse at compile time
        self.env: Dict[torch.fx.Node, object] = {}
        self.inputs: List[dict] = []
        self.loss: Optional[torch.Tensor] = None
        self._opt = None
        self._step_count = 0
        self._shadow_stale = False
        self._example_inputs = [a if isinstance(a, torch.Tensor) else torch.empty(tuple(a), device="meta")
                                for a in example_inputs]
        self.rank_hint, self.world_hint = rank, world_size
        self._param_reduce: List[Callable[[], None]] = []
        self._scratch_pool: Dict[tuple, torch.Tensor] = {}
        self.fused_attention = fused_attention
        # Optional: weight-gradient GEMMs (and bias column sums) feed nothing but the optimizer, so they can be
        # launched on a second stream of the same priority, next to the activation-gradient chain on the main
        # stream; the side stream joins before the gradients of replicated parameters are reduced.  Measured on
        # the BERT-large shard this hides host launch latency of eager steps (about 6 %), but adds nothing to a
        # step replayed from a HIP graph, so it is off by default.
        self.overlap_wgrad = overlap_wgrad
        self.relu_mask_in_dgrad = relu_mask_in_dgrad
        # relu's backward behind an all_to_all rides on the copying split of the backward exchange (one pass over
        # the gradient less per layer); False keeps the separate pass, for comparison
        self.relu_bwd_in_split = relu_bwd_in_split
        self.fuse_dropout = fuse_dropout               # F.dropout inside the kernel next to it where one can take it
        # the backward all_to_all of the column-sharded FFN concatenates along dim 0: every peer's piece is a
        # contiguous row range of the result, so it is received there (Wire.recv(into=...)) instead of into a
        # buffer of its own that a copy kernel then moves; False keeps the copy
        self.receive_in_place = receive_in_place
        # all_to_all -> relu -> linear (the column-sharded FFN, bf16): the linear reads the exchanged pieces where
        # they were received (relu applied as the operand is loaded) and its backward writes the pieces of the backward
        # exchange directly, so neither the concatenating copy forward nor the splitting copy backward runs; False
        # keeps the copies (which then carry the relu), for comparison
        self.exchange_in_pieces = exchange_in_pieces
        # Optional: train_step() applies the optimizer to each stretch of the flat parameter buffer as soon as
        # backward has finished with it, on a second stream.  Measured on the BERT-large shard the step takes the
        # same time either way (27.1 against 27.0 ms): the GEMMs that run next to the update slow down by what the
        # update saves (they are bound by the memory system too), so it is off by default.
        self.overlap_optimizer = overlap_optimizer and not overlap_wgrad
        self._opt_stream = torch.cuda.Stream(device=self.dev) if self.overlap_optimizer else None
        self._opt_join = torch.cuda.Event() if self.overlap_optimizer else None
        self._opt_chunks: Optional[list] = None
        self.optimizer_chunk_min = int(optimizer_chunk_min)      # smallest stretch (elements) worth a launch of its own
        self._touched: Optional[list] = None
        self._grad_final_idx: Dict[str, int] = {}
        # The weight gradient of one linear has a small output and a long reduction (BERT-large shard: [1024, 1024]
        # to [1024, 4096] outputs over 6144-16384 tokens): alone it fills the chip only with its reduction split
        # 2-8 ways through float32 partial sums.  The same linear's weight gradients of `wgrad_group` consecutive
        # layers go into ONE launch instead (pointer lists, no split): measured 153 us against 247 us per layer.
        # They are held back until the group is full (or backward ends); their operands are per-layer buffers
        # that nothing overwrites before (see _grad_slot / _guard_write).  1 = every weight gradient at once.
        self.wgrad_group = 1 if (overlap_wgrad or self.overlap_optimizer) else max(1, min(int(wgrad_group), ops._lib.GEMM_MAX_LIST))
        self._send_hooks = 0                               # callables the wire asked to run after every message is complete
        self._grad_sharers: Dict[int, list] = {}           # gradient storage -> values whose gradient aliases it
        self._emit_pos = -1                                # index of the backward emitter that is running
        self.shared_gradient_copies = 0                    # times a contribution went to a new buffer because of sharing
        self._param_vals: Dict[str, Val] = {}
        self._wire_backed: set = set()                     # storages that peers' messages are received into in place
        self._pending_wgrads: Dict[tuple, list] = {}
        self._deferred_reads: Dict[int, int] = {}          # storage -> launches held back that read it
        self._side_stream = torch.cuda.Stream(device=self.dev) if overlap_wgrad else None
        self._side_join = torch.cuda.Event() if overlap_wgrad else None
        self._side_used = False
        self._side_readers: Dict[int, torch.cuda.Event] = {}   # storage -> event after its last side-stream reader
        self.side_workspace = torch.empty(64 << 20, dtype=torch.float32, device=self.dev) if overlap_wgrad else None
        self._single_use_params = self._find_single_use_params(gm)
        # F.dropout with p > 0: keep decisions are a function of (seed, step, node, element); the step count lives on
        # the device and is advanced by the first launch of every forward pass, so replayed steps draw new masks
        self.rng_state = torch.tensor([int(dropout_seed), 0], dtype=torch.int64, device=self.dev)
        self._node_ids = {node: i for i, node in enumerate(gm.graph.nodes)}
        self._uses_rng = False
        # Every launch of a step is a library call on static buffers with constant arguments, so the calls of
        # the first forward / backward / optimizer phase are recorded and later phases replay the recorded
        # calls directly (no per-call argument marshalling or host-side checks: about 10 us of interpreter
        # time per launch otherwise).  Keyed by stream; not used together with the side stream.
        self.launch_lists = launch_lists and not overlap_wgrad
        self._lists: Dict[tuple, list] = {}
        self.gemm_workspace = torch.empty(64 << 20, dtype=torch.float32, device=self.dev)   # 256 MiB of split-K scratch
        ops.set_gemm_workspace(self.gemm_workspace)
        self._prepare_params()
        self._compile()
        self._finish_param_reduce()

    # ------------------------------------------------------------------ parameters
    def _prepare_params(self):
        """Parameters the program reads go into one flat float32 master buffer (views replace
        ``p.data``), with flat float32 gradients and, in bf16 mode, a flat bf16 shadow."""
        used = []
        for node in self.gm.graph.nodes:
            if node.op == "get_attr" and node.target not in used:
                used.append(node.target)
        self.param_names, self.buffers = [], {}
        metas = []
        off = 0
        found = []
        for name in used:
            obj = self._fetch(name)
            if isinstance(obj, torch.nn.Parameter):
                found.append((name, obj))
            else:
                self.buffers[name] = obj
        # vectors (biases) first and contiguous: their gradients are column sums accumulated with atomics, so
        # one fill per step clears all of them
        found.sort(key=lambda kv: 0 if kv[1].dim() == 1 else 1)
        self.n_vector_region = 0
        for name, obj in found:
            n = obj.numel()
            metas.append((name, obj, off, n))
            off += _round_up(n, 64)            # keep every view 256-byte aligned
            if obj.dim() == 1:
                self.n_vector_region = off
            self.param_names.append(name)
        self.n_flat = off
        self.master = torch.zeros(max(off, 4), dtype=torch.float32, device=self.dev)
        self.flat_grad = torch.zeros_like(self.master)
        self.shadow = torch.zeros(max(off, 4), dtype=torch.bfloat16, device=self.dev) if self.dtype == "bf16" else None
        self.params: Dict[str, dict] = {}
        for name, p, o, n in metas:
            view = self.master[o:o + n].view(p.shape)
            view.copy_(p.data.to(self.dev, torch.float32))
            p.data = view
            g = self.flat_grad[o:o + n].view(p.shape)
            p.grad = g
            sh = self.shadow[o:o + n].view(p.shape) if self.shadow is not None else None
            self.params[name] = dict(param=p, master=view, grad=g, shadow=sh, offset=o, numel=n)
        if self.shadow is not None:
            ops.cast(self.master, self.shadow)
        # whole-shape float32 gradients of parameters that are stored as shards and gathered at use; vectors
        # first, as in the flat gradient buffer, so that one fill clears them
        gathered = []
        for node in self.gm.graph.nodes:
            if (node.op == "call_function" and node.target is collectives.all_gather
                    and node.args[0].op == "get_attr" and node.args[0].target in self.params):
                shape = (sum(node.args[2]),) + tuple(self.params[node.args[0].target]["param"].shape[1:])
                gathered.append((node.args[0].target, shape))
        gathered.sort(key=lambda kv: 0 if len(kv[1]) == 1 else 1)
        off, spans = 0, []
        self.n_gathered_vector_region = 0
        for name, shape in gathered:
            n = 1
            for v in shape:
                n *= v
            spans.append((name, shape, off, n))
            off += _round_up(n, 64)
            if len(shape) == 1:
                self.n_gathered_vector_region = off
        self.gathered_grad = torch.zeros(max(off, 4), dtype=torch.float32, device=self.dev) if gathered else None
        self._gathered_grads = {name: self.gathered_grad[o:o + n].view(shape) for name, shape, o, n in spans}

    def _fetch(self, target: str):
        obj = self.gm
        for atom in target.split("."):
            obj = getattr(obj, atom)
        return obj

    # ------------------------------------------------------------------ small helpers
    def _new(self, shape, dtype=None):
        return torch.empty(tuple(shape), dtype=dtype or self.cdt, device=self.dev)

    def _val(self, x):
        return self.env[x] if isinstance(x, torch.fx.Node) else x

    def _place_gather_inputs(self):
        """Which nodes write their result straight into the rows of an all_gather's result.  The gather along dim 0
        concatenates the ranks' shards; when the shard's producer allocates the whole result and writes its rows of
        it, the gather has no copy of the own shard left to make (the peers' shards are received at their rows).
        Producers that do this: layer_norm (the input of the column-sharded FFN's gather)."""
        self._gather_of: Dict[torch.fx.Node, torch.fx.Node] = {}
        self._gather_results: Dict[torch.fx.Node, torch.Tensor] = {}
        if not self.receive_in_place:
            return
        for node in self.gm.graph.nodes:
            if node.op != "call_function" or node.target is not collectives.all_gather or len(node.args) < 4:
                continue
            src, dim, L, rank = node.args[0], node.args[1], list(node.args[2]), node.args[3]
            if (dim == 0 and isinstance(src, torch.fx.Node) and src.op == "call_function" and src.target is F.layer_norm
                    and src not in self._gather_of and L[rank] > 0):
                self._gather_of[src] = node

    def _placed_output(self, node, shape):
        """The buffer for ``node``'s result: new, or its rows of the all_gather result that it feeds."""
        g = self._gather_of.get(node)
        if g is None or len(shape) < 1:
            return self._new(shape)
        L, rank = list(g.args[2]), g.args[3]
        if shape[0] != L[rank]:
            return self._new(shape)
        full = self._new((sum(L),) + tuple(shape[1:]))
        self._gather_results[g] = full
        return full.narrow(0, sum(L[:rank]), L[rank])

    def _scratch(self, key, shape, dtype=None):
        """Backward-only temporaries that live inside one node's backward closure are shared between
        nodes of the same shape (the launches of a step are serialised on one stream)."""
        k = (key, tuple(shape), dtype or self.cdt)
        if k not in self._scratch_pool:
            self._scratch_pool[k] = self._new(shape, dtype)
        return self._scratch_pool[k]

    def _grad_slot(self, v: Val):
        """Buffer that the next contribution to d(v) goes into and whether it must accumulate."""
        if v.grad is None:
            v.grad = self._new(v.t.shape if v.t is not None else v.shape)
            return v.grad, False
        if self._shared_with_pending(v):
            # another value's gradient aliases this buffer and its producer has not read it yet: continue in a copy
            old = v.grad
            v.grad = self._new(old.shape, old.dtype)
            new = v.grad
            self.bwd.append(lambda: ops.scale(old, 1.0, new))
            return v.grad, True
        self._guard_write(v.grad)
        return v.grad, True

    def _grad_slot_addend(self, v: Val):
        """``_grad_slot`` for a GEMM: (buffer, accumulate, addend).  When the gradient exists but weight-gradient
        launches that are held back still read its buffer, the sum goes to a new buffer (C = addend + A B) and
        the old one stays as it is."""
        if v.grad is not None and (self._is_read_later(v.grad) or self._shared_with_pending(v)):
            old = v.grad
            v.grad = self._new(old.shape, old.dtype)
            return v.grad, True, old
        g, acc = self._grad_slot(v)
        return g, acc, None

    def _is_read_later(self, t: Optional[torch.Tensor]) -> bool:
        return t is not None and self._deferred_reads.get(t.untyped_storage().data_ptr(), 0) > 0

    def _emit_wgrad(self, dy, xt, gw, gb, n_out, n_in, rows, ld_dy, ld_x, acc, params, x_relu=False):
        """dW[n_out, n_in] (+)= dy[rows, n_out]^T x[rows, n_in], the bias gradient gb (column sums of dy) taken by
        the same kernel.  Launched at once, or held back to share a launch with the same linear of the next
        layers (only for parameters with a single use: their gradient is written once, order does not matter).
        ``xt`` may be a list of pieces [rows, len] along n_in (with ``x_relu``: relu applied as they are loaded)."""
        pieces = isinstance(xt, (list, tuple))
        if not self._holds_back_wgrad(params):
            if pieces:
                self.bwd.append(lambda: ops.gemm(dy, None, gw, n_out, n_in, rows, transA=True, lda=ld_dy, accumulate=acc,
                                                 a_rowsum=gb, b_segments=list(xt), b_relu=x_relu))
            else:
                self.bwd.append(lambda: ops.gemm(dy, xt, gw, n_out, n_in, rows, transA=True, lda=ld_dy, ldb=ld_x,
                                                 accumulate=acc, a_rowsum=gb))
            return
        layout = tuple((t.shape[1], t.stride(0)) for t in xt) if pieces else None
        sig = (n_out, n_in, rows, ld_dy, ld_x, bool(acc), dy.dtype, gw.dtype, layout, bool(x_relu))
        q = self._pending_wgrads.setdefault(sig, [])
        q.append((dy, xt, gw, gb, [v.meta.get("name") or v.meta.get("shard_of") for v in params if v is not None], []))
        for t in (dy,) + (tuple(xt) if pieces else (xt,)):
            k = t.untyped_storage().data_ptr()
            self._deferred_reads[k] = self._deferred_reads.get(k, 0) + 1
        if len(q) >= self.wgrad_group:
            self._flush_wgrads(sig)

    def _holds_back_wgrad(self, params) -> bool:
        """Whether the weight gradient of these parameters (weight, bias) is held back for a shared launch: only when
        each is used once in the program, so that its gradient is written once and the order does not matter."""
        return self.wgrad_group > 1 and all(
            v is None or v.meta.get("name") in self._single_use_params or v.meta.get("single_use") for v in params)

    def _flush_wgrads(self, sig=None):
        """Append the launches of the weight gradients held back (of one signature, or all)."""
        for key in ([sig] if sig is not None else list(self._pending_wgrads)):
            q = self._pending_wgrads.pop(key, [])
            if not q:
                continue
            n_out, n_in, rows, ld_dy, ld_x, acc = key[:6]
            for dy, xt, _, _, _, _ in q:
                for t in (dy,) + (tuple(xt) if isinstance(xt, (list, tuple)) else (xt,)):
                    self._deferred_reads[t.untyped_storage().data_ptr()] -= 1
            self.bwd.append(self._wgrad_launch(q, n_out, n_in, rows, ld_dy, ld_x, acc, key[9]))
            for e in q:
                for hook in e[5]:
                    hook()                               # launches that wait for this weight gradient
            for e in q:
                for name in e[4]:
                    self._grad_final_idx[name] = len(self.bwd)

    def _after_wgrad(self, grad_t: torch.Tensor, fn: Callable[[], None]):
        """Run ``fn`` (which appends launches that read the gradient buffer ``grad_t``) once the weight gradient
        that writes ``grad_t`` has been appended: now, or when the group that holds it back is launched."""
        key = grad_t.data_ptr()                          # gradient buffers are views of one flat buffer
        for q in self._pending_wgrads.values():
            for e in q:
                if any(t is not None and t.data_ptr() == key for t in (e[2], e[3])):
                    e[5].append(fn)
                    return
        fn()

    @staticmethod
    def _wgrad_launch(q, n_out, n_in, rows, ld_dy, ld_x, acc, x_relu=False):
        pieces = isinstance(q[0][1], (list, tuple))
        if len(q) == 1:
            dy, xt, gw, gb = q[0][:4]
            if pieces:
                return lambda: ops.gemm(dy, None, gw, n_out, n_in, rows, transA=True, lda=ld_dy, accumulate=acc, a_rowsum=gb,
                                        b_segments=list(xt), b_relu=x_relu)
            return lambda: ops.gemm(dy, xt, gw, n_out, n_in, rows, transA=True, lda=ld_dy, ldb=ld_x, accumulate=acc,
                                    a_rowsum=gb)
        dys, xts, gws = [e[0] for e in q], [e[1] for e in q], [e[2] for e in q]
        gbs = [e[3] for e in q] if any(e[3] is not None for e in q) else None
        return lambda: ops.gemm_group(dys, xts, gws, n_out, n_in, rows, transA=True, lda=ld_dy, ldb=None if pieces else ld_x,
                                      accumulate=acc, a_rowsums=gbs, b_relu=x_relu)

    def _param_grad_slot(self, v: Val):
        if self._touched is not None and v.meta.get("name") is not None:
            self._touched.append(v.meta["name"])
        first = not v.meta.get("grad_written", False)
        v.meta["grad_written"] = True
        if v.meta["grad"].dim() == 1:
            return v.meta["grad"], True       # the vector region is cleared once at the start of backward
        return v.meta["grad"], not first

    @staticmethod
    def _find_single_use_params(gm):
        """Names of parameters with exactly one consumer in the program (through replicate / all_gather
        wrappers): only their gradients can be produced off the main stream without ordering against another
        contribution."""
        names = set()
        for node in gm.graph.nodes:
            if node.op != "get_attr":
                continue
            n, ok = node, True
            while ok:
                users = list(n.users)
                if len(users) != 1:
                    ok = False
                elif users[0].op == "call_function" and users[0].target in (collectives.replicate, collectives.all_gather,
                                                                             models.new_segment):
                    n = users[0]
                else:
                    break
            if ok:
                names.add(node.target)
        return names

    def _side_ok(self, *vals) -> bool:
        return self.overlap_wgrad and all(v is None or v.meta.get("name") in self._single_use_params for v in vals)

    def _emit_side(self, fn: Callable[[], None], reads):
        """Append ``fn`` to the backward list so that its launches run on the side stream, ordered after
        everything the main stream has enqueued so far.  ``reads`` are the buffers ``fn`` reads: gradient
        buffers alias each other through residual adds and are accumulated into in place later in the
        backward list, so a later main-stream writer of one of them first waits for ``fn``
        (see _guard_write)."""
        fork, done = torch.cuda.Event(), torch.cuda.Event()
        side = self._side_stream
        for t in reads:
            self._side_readers[t.untyped_storage().data_ptr()] = done

        def run():
            fork.record(torch.cuda.current_stream())
            side.wait_event(fork)
            with torch.cuda.stream(side):
                fn()
            done.record(side)
            self._side_used = True
        self.bwd.append(run)

    def _guard_write(self, t: Optional[torch.Tensor]):
        """Called while the backward list is built, right before a launch that writes into ``t`` is appended:
        when a side-stream launch appended earlier reads ``t``'s storage, the main stream waits for it first;
        when weight-gradient launches that are held back read it, they are appended first."""
        if t is not None and t.untyped_storage().data_ptr() in self._wire_backed:
            raise RuntimeError("internal: a launch would write into a buffer that peers' messages are received into")
        if self._is_read_later(t):
            self._flush_wgrads()             # weight gradients held back read t: they go first
        if t is None or not self._side_readers:
            return
        done = self._side_readers.pop(t.untyped_storage().data_ptr(), None)
        if done is not None:
            self.bwd.append(lambda: torch.cuda.current_stream().wait_event(done))

    def _join_side(self):
        if self._side_used:
            self._side_join.record(self._side_stream)
            torch.cuda.current_stream().wait_event(self._side_join)
            self._side_used = False

    def _unsupported(self, node, why):
        raise ValueError(f"node {node.name} ({node.target}): {why}")

    # ------------------------------------------------------------------ compile
    def _compile(self):
        handlers = {
            F.embedding: self._embedding, operator.mul: self._mul, operator.add: self._add,
            torch.transpose: self._transpose, F.multi_head_attention_forward: self._mha,
            operator.getitem: self._getitem, F.dropout: self._dropout, F.layer_norm: self._layer_norm,
            F.linear: self._linear, F.relu: self._activation, F.gelu: self._activation,
            torch.sigmoid: self._activation, torch.sum: self._sum,
            torch.log_softmax: self._log_softmax, F.nll_loss: self._nll_loss,
            F.conv2d: self._conv2d, torch.flatten: self._flatten,
            models.append_cls_token: self._append_cls, models.get_cls_token: self._get_cls,
            models.new_segment: self._alias, models.top_2_gating: self._gating, models.switch_gating: self._gating,
            models.head_parallel_attention: self._head_parallel_attention,
            torch.einsum: self._einsum,
            collectives.replicate: self._replicate, collectives.all_gather: self._all_gather,
            collectives.reduce_scatter: self._reduce_scatter, collectives.all_to_all: self._all_to_all,
            collectives.all_reduce: self._all_reduce, collectives.dynamic_slice: self._dynamic_slice,
        }
        self._place_gather_inputs()
        for node in self.gm.graph.nodes:
            if node.op == "placeholder":
                self.env[node] = Val("input", name=node.name, index=len(self.inputs))
                self.inputs.append(dict(name=node.name, buf=None, offset=None, length=None))
            elif node.op == "get_attr":
                self.env[node] = self._get_attr(node)
            elif node.op == "call_method":
                if node.target != "split":
                    self._unsupported(node, "only Tensor.split is emitted for inputs")
                src = self._val(node.args[0])
                if src.kind != "input" or len(node.args) != 3:
                    self._unsupported(node, "split(lengths, dim) is only supported on a program input")
                self.env[node] = Val("input_split", src=src, lengths=list(node.args[1]), dim=int(node.args[2]))
            elif node.op == "call_function":
                h = handlers.get(node.target)
                if h is None:
                    self._unsupported(node, "this op has no handler")
                val = self.env[node] = h(node)
                # which backward emitter belongs to the producer of this value (see _shared_with_pending)
                if isinstance(val, Val) and "tape_idx" not in val.meta:
                    val.meta["tape_idx"] = len(self._tape) - 1
            elif node.op == "output":
                out = self._val(node.args[0])
                if out.kind != "loss":
                    self._unsupported(node, "the program output must be the scalar of nll_loss or torch.sum")
                self.loss = out.t
        # backward list: the tape in reverse.  For every parameter remember how many backward launches must have
        # been enqueued before nothing reads its value or writes its gradient any more (all of them are made by
        # the emit of a node that consumes the parameter)
        for idx in range(len(self._tape) - 1, -1, -1):
            self._touched = []
            self._emit_pos = idx
            self._tape[idx]()
            for name in self._touched:
                self._grad_final_idx[name] = len(self.bwd)
        self._flush_wgrads()
        self._touched = None
        self._tape = []
        if self._uses_rng:
            self.fwd.insert(0, lambda: ops.rng_advance(self.rng_state))

    # ------------------------------------------------------------------ leaves
    def _get_attr(self, node):
        name = node.target
        if name in self.params:
            # one value per parameter, however many get_attr nodes name it: whether its gradient has had its first
            # contribution (which overwrites; later ones accumulate) is kept on the value
            if name not in self._param_vals:
                rec = self.params[name]
                t = rec["shadow"] if self.dtype == "bf16" else rec["master"]
                self._param_vals[name] = Val("param", t, name=name, master=rec["master"], grad=rec["grad"], needs_grad=True)
            return self._param_vals[name]
        buf = self.buffers[name]
        keep_f32 = name.endswith("src_mask")
        t = buf.detach().to(self.dev, torch.float32 if keep_f32 else self.cdt).contiguous()
        return Val("tensor", t, name=name)

    def _alias(self, node):
        return self._val(node.args[0])

    def _replicate(self, node):
        v = self._val(node.args[0])
        if v.kind == "param":
            v.meta["replicated_tag"] = node.name
        return v

    def _getitem(self, node):
        src, idx = self._val(node.args[0]), node.args[1]
        if src.kind == "input_split":
            L = src.meta["lengths"]
            return Val("input_slice", src=src.meta["src"], offset=sum(L[:idx]), length=L[idx], dim=src.meta["dim"])
        if src.kind == "mha":
            if idx == 0:
                return src.meta["out"]
            return Val("dead", why="head-averaged attention probabilities are never consumed by the program")
        if src.kind == "gating":
            return Val("routing", which="dispatch" if idx == 0 else "combine", gating=src, e_lo=0, E_loc=src.meta["E"],
                       c_lo=0, C_loc=src.meta["C"], s_lo=0, S_loc=src.meta["x"].t.shape[1])
        self._unsupported(node, f"getitem on a {src.kind} value")

    # ------------------------------------------------------------------ ops
    def _embedding(self, node):
        ids_v, table = self._val(node.args[0]), self._val(node.args[1])
        ids = self._input_buffer(ids_v, torch.int64)
        d = table.t.shape[1]
        out = Val("tensor", self._new(tuple(ids.shape) + (d,)), needs_grad=True)
        self.fwd.append(lambda: ops.embedding_fwd(ids, table.t, None, out.t, 1, 1.0))

        def emit():
            if out.grad is None:
                return
            g, acc = self._param_grad_slot(table)
            if not acc:
                self.bwd.append(lambda: ops.fill_zero(g))
            self.bwd.append(lambda: ops.embedding_bwd(ids, out.grad, g, 1.0))
        self._tape.append(emit)
        return out

    def _input_buffer(self, v: Val, dtype) -> torch.Tensor:
        if v.kind not in ("input", "input_slice"):
            raise ValueError("expected a program input")
        src = v if v.kind == "input" else v.meta["src"]
        rec = self.inputs[src.meta["index"]]
        full = self._example_inputs[src.meta["index"]]
        off = v.meta.get("offset") if v.kind == "input_slice" else None
        dim = v.meta.get("dim", 0) if v.kind == "input_slice" else 0
        if dim < 0:
            dim += full.dim()
        length = v.meta.get("length") if v.kind == "input_slice" else full.shape[0]
        if rec["buf"] is None:
            rec.update(offset=off, length=length, dim=dim)
            shape = list(full.shape)
            shape[dim] = length
            rec["buf"] = torch.empty(tuple(shape), dtype=dtype, device=self.dev)
        elif (rec["offset"], rec["length"], rec.get("dim", 0)) != (off, length, dim) or rec["buf"].dtype != dtype:
            raise ValueError(f"program input {rec['name']!r} is used as two different slices / types")
        return rec["buf"]

    def _mul(self, node):
        a, s = self._val(node.args[0]), node.args[1]
        if not isinstance(s, (int, float)):
            self._unsupported(node, "only multiplication by a number is supported")
        out = Val("tensor", self._new(a.t.shape), needs_grad=a.needs_grad)
        self.fwd.append(lambda: ops.scale(a.t, float(s), out.t))

        def emit():
            if out.grad is None or not a.needs_grad:
                return
            g, acc = self._grad_slot(a)
            if acc:
                tmp = self._new(a.t.shape)
                self.bwd.append(lambda: (ops.scale(out.grad, float(s), tmp), ops.add(g, tmp, g)))
            else:
                self.bwd.append(lambda: ops.scale(out.grad, float(s), g))
        self._tape.append(emit)
        return out

    def _add(self, node):
        a, b = self._val(node.args[0]), self._val(node.args[1])
        users = list(node.users)
        if a.kind == "cls_appended" or b.kind == "cls_appended":
            ac, other = (a, b) if a.kind == "cls_appended" else (b, a)
            n, T, d = ac.meta["x"].t.shape
            if other.t is not None and tuple(other.t.shape) == (1, T + 1, d):
                return self._append_cls_pos(node, ac, other)       # the position embedding's add (models.py:167)
            done = self._append_cls_pos(node, ac, None)             # some other add: the bare append first
            a, b = (done, b) if a is ac else (a, done)
        if a.kind == "dropped" or b.kind == "dropped":
            # _dropout has checked the form: the other operand is a tensor of this shape and layer_norm reads the sum
            return Val("sum", None, shape=a.shape, a=a, b=b, needs_grad=True)
        if a.t is None or b.t is None:
            self._unsupported(node, "operands must be materialised tensors")
        if tuple(a.t.shape) == tuple(b.t.shape):
            if len(users) == 1 and users[0].target is F.layer_norm:
                return Val("sum", None, shape=a.t.shape, a=a, b=b, needs_grad=True)
            out = Val("tensor", self._new(a.t.shape), needs_grad=a.needs_grad or b.needs_grad)
            self.fwd.append(lambda: ops.add(a.t, b.t, out.t))

            def emit():
                if out.grad is None:
                    return
                for v in (a, b):
                    if v.needs_grad:
                        self._accumulate_into(v, out.grad)
            self._tape.append(emit)
            return out
        # broadcast over the leading dimension(s): [b, S, d] + [1, S, d], or [b, S, d] + [d] (a bias)
        big, small = (a, b) if a.t.numel() >= b.t.numel() else (b, a)
        vector = small.t.dim() == 1 and small.t.shape[0] == big.t.shape[-1]
        if not vector and (small.t.shape[0] != 1 or tuple(small.t.shape[1:]) != tuple(big.t.shape[1:])):
            self._unsupported(node, f"broadcast of {tuple(small.t.shape)} onto {tuple(big.t.shape)} is not supported")
        width = big.t.shape[-1]
        b_rows = small.t.numel() // width
        rows = big.t.numel() // width
        out = Val("tensor", self._new(big.t.shape), needs_grad=big.needs_grad or small.needs_grad)
        self.fwd.append(lambda: ops.add_bcast_rows(big.t, small.t, out.t, rows, b_rows, width))

        def emit():
            if out.grad is None:
                return
            if big.needs_grad:
                self._accumulate_into(big, out.grad)
            if small.kind == "param":
                g, acc = self._param_grad_slot(small)
                n = small.t.numel()
                self.bwd.append(lambda: ops.colsum(out.grad, g, rows // b_rows, n, n, acc))
        self._tape.append(emit)
        return out

    def _accumulate_into(self, v: Val, src: torch.Tensor):
        """d(v) += src; when d(v) does not exist yet it ALIASES src (the residual add hands one buffer to both of
        its operands).  A later contribution is added in place only if no other value still needs the buffer as
        it is (_shared_with_pending, weight gradients held back); otherwise the sum goes to a new buffer."""
        if v.grad is None:
            v.grad = src
            self._grad_sharers.setdefault(src.untyped_storage().data_ptr(), []).append(v)
        elif self._is_read_later(v.grad) or self._shared_with_pending(v):
            g = v.grad
            v.grad = self._new(g.shape, g.dtype)         # weight gradients held back, or another value, still read g
            out = v.grad
            self.bwd.append(lambda: ops.add(g, src, out))
        else:
            g = v.grad
            self._guard_write(g)
            self.bwd.append(lambda: ops.add(g, src, g))

    def _shared_with_pending(self, v: Val) -> bool:
        """True when d(v)'s buffer is also the gradient of another value whose producer has not been through its
        backward emitter yet: that emitter will read the buffer, so nothing may be added into it in place before.
        (Emitters run in reverse program order; a value's producer is pending while its index is below the
        running emitter's.  The generated programs never get here: between the residual add and the producer of
        its second operand they have no other consumer of the first.)"""
        if v.grad is None:
            return False
        for o in self._grad_sharers.get(v.grad.untyped_storage().data_ptr(), ()):
            if o is not v and o.grad is not None and o.grad.untyped_storage().data_ptr() == v.grad.untyped_storage().data_ptr() \
                    and 0 <= o.meta.get("tape_idx", -1) < self._emit_pos:
                self.shared_gradient_copies += 1
                return True
        return False

    def _transpose(self, node):
        v, d0, d1 = self._val(node.args[0]), node.args[1], node.args[2]
        dims = tuple(sorted((d0, d1)))
        if v.kind == "transposed" and v.meta["dims"] == dims:
            return v.meta["src"]
        if v.kind == "logprobs" and dims == (1, 2):
            return Val("logprobs", src=v.meta["src"], transposed=True)
        if v.kind == "conv_flat" and dims == (1, 2):
            return v.meta["tokens"]
        if v.t is None:
            self._unsupported(node, f"transpose of a {v.kind} value")
        return Val("transposed", None, src=v, dims=dims, needs_grad=v.needs_grad)

    def _dropout(self, node):
        """F.dropout(input, p) (hap.rs:1464: training mode).  p = 0 is the identity.  Otherwise one elementwise pass
        forward and the same pass on the gradient backward; the mask is regenerated, not stored."""
        p = float(node.args[1])
        if len(node.args) > 2 or node.kwargs:
            self._unsupported(node, "the program emits F.dropout(input, p) only")
        x = self._val(node.args[0])
        if p == 0.0:
            return x
        if not 0.0 < p <= 1.0:
            self._unsupported(node, f"dropout probability {p}")
        if x.kind == "pieces":
            return self._dropout_on_pieces(node, x, p)
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"dropout of a {x.kind} value")
        self._uses_rng = True
        sid = self._node_ids[node]
        if (self.fuse_dropout and x.meta.get("fused_act") == "relu" and x.meta.get("can_fuse_drop") and p < 1.0
                and "fused_drop" not in x.meta and self._only_reader(node, x)):
            # relu -> dropout, both applied by the kernel that produces the value (it reads fused_drop when it runs).
            # The stored value is the dropped one: positive exactly where relu passed and dropout kept, so every
            # form of relu's backward serves as the backward of both once its result is scaled by 1 / (1 - p).
            x.meta["fused_drop"] = (p, sid)
            x.meta["dropout"] = (p, sid)
            return x
        if self.fuse_dropout and self._feeds_residual_layer_norm(node, x):
            # dropout -> add -> layer_norm: the layer_norm kernels apply it to their operand (forward) and give its
            # backward as a second result; nothing is materialised here
            return Val("dropped", None, shape=x.t.shape, src=x, needs_grad=x.needs_grad, dropout=(p, sid))
        out = Val("tensor", self._new(x.t.shape), needs_grad=x.needs_grad, dropout=(p, sid))
        self.fwd.append(lambda: ops.dropout(x.t, out.t, p, self.rng_state, sid))

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            if x.grad is None:
                x.grad = self._new(x.t.shape)
                g = x.grad
                self.bwd.append(lambda: ops.dropout(out.grad, g, p, self.rng_state, sid))
            else:
                tmp = self._new(x.t.shape)
                g, _ = self._grad_slot(x)
                self.bwd.append(lambda: (ops.dropout(out.grad, tmp, p, self.rng_state, sid), ops.add(g, tmp, g)))
        self._tape.append(emit)
        return out

    def _dropout_on_pieces(self, node, x: Val, p: float):
        """relu -> dropout on the pieces of an all_to_all that a linear reads where they lie: one pass writes
        dropout(relu(piece)) for every piece (decisions by the element's place in the concatenation, which never
        exists); the linear then reads those, and its data gradient is masked with them and scaled by 1 / (1 - p),
        which is the backward of both."""
        if not (x.meta["relu"] and 0.0 < p < 1.0 and "mask_scale" not in x.meta):
            self._unsupported(node, "on the pieces of an exchange only relu -> one dropout is handled")
        self._uses_rng = True
        sid = self._node_ids[node]
        src = x.meta["pieces2d"]
        dst = [self._new(t.shape) for t in src]
        self.fwd.append(lambda: ops.relu_dropout_pieces(src, dst, p, self.rng_state, sid))
        lead = tuple(x.shape[:-1])
        return Val("pieces", None, shape=x.shape, needs_grad=x.needs_grad, relu=False, mask_scale=1.0 / (1.0 - p),
                   pieces=[t.view(lead + (t.shape[-1],)) for t in dst], pieces2d=dst, dropout=(p, sid),
                   backward_exchange=x.meta["backward_exchange"])

    def _feeds_residual_layer_norm(self, node, x: Val) -> bool:
        """node's only reader is an operator.add of it and an already materialised tensor of the same shape, whose
        only reader is F.layer_norm (the form _add hands to _layer_norm as a lazy sum)."""
        users = list(node.users)
        if len(users) != 1 or users[0].target is not operator.add or len(users[0].args) != 2:
            return False
        add = users[0]
        others = [a for a in add.args if a is not node]
        if len(others) != 1 or not isinstance(others[0], torch.fx.Node):
            return False
        other = self.env.get(others[0])
        if not isinstance(other, Val) or other.t is None or other.ld is not None or tuple(other.t.shape) != tuple(x.t.shape):
            return False
        ln = list(add.users)
        return len(ln) == 1 and ln[0].target is F.layer_norm and len(ln[0].args) == 2 and not ln[0].kwargs

    def dropout_masks(self) -> Dict[str, torch.Tensor]:
        """The keep decisions of the step that ran last, by node name: for an F.dropout node a bool tensor of its
        input's shape, for an attention node with dropout_p > 0 a bool tensor [batch, heads, L, S] over its
        probabilities.  (Tests hand them to the CPU oracle, which cannot share a random stream with the GPU.)"""
        out = {}
        for node, v in self.env.items():
            if not isinstance(node, torch.fx.Node) or node.op != "call_function":
                continue
            if isinstance(v, Val) and v.meta.get("dropout") and node.target is F.dropout and float(node.args[1]) > 0:
                p, sid = v.meta["dropout"]
                out[node.name] = ops.dropout_mask(math.prod(v.shape), p, self.rng_state, sid).view(v.shape).bool()
            elif isinstance(v, Val) and v.kind == "mha" and v.meta.get("dropout"):
                p, sid, shape, S = v.meta["dropout"]
                n = 1
                for d in shape:
                    n *= d
                out[node.name] = ops.dropout_mask(n, p, self.rng_state, sid).view(shape)[..., :S].bool()
        return out

    def _layer_norm(self, node):
        v, shape = self._val(node.args[0]), tuple(node.args[1])
        if len(node.args) > 2 or node.kwargs:
            self._unsupported(node, "the program emits layer_norm without affine parameters")
        drop = dropped = None
        if v.kind == "sum":
            a, b = v.meta["a"], v.meta["b"]
            if b.kind != "dropped" and a.kind == "dropped":
                a, b = b, a
            if b.kind == "dropped":            # LN(res + dropout(src)): the kernel's first operand is the dropped one
                dropped, b = b, b.meta["src"]
                drop = (dropped.meta["dropout"][0], self.rng_state, dropped.meta["dropout"][1])
                x, res, ref_shape = b.t, a.t, a.t.shape
            else:
                x, res, ref_shape = a.t, b.t, a.t.shape
        else:
            a, b, x, res, ref_shape = v, None, v.t, None, v.t.shape
        if len(shape) != 1 or shape[0] != ref_shape[-1]:
            self._unsupported(node, "layer_norm over the last dimension only")
        rows = x.numel() // shape[0]
        out = Val("tensor", self._placed_output(node, ref_shape), needs_grad=True)
        rstd = self._new((rows,), torch.float32)
        self.fwd.append(lambda: ops.add_layernorm_fwd(x, res, out.t, rstd, _EPS, drop))

        def emit():
            if out.grad is None:
                return
            targets = [v for v in (a, b) if v is not None and v.needs_grad]
            if not targets:
                return
            dx = self._new(ref_shape)
            if dropped is not None and b.needs_grad:
                dx_drop = self._new(ref_shape)
                self.bwd.append(lambda: ops.layernorm_bwd(out.grad, out.t, rstd, None, dx, dx_drop, drop))
                if a.needs_grad:
                    self._accumulate_into(a, dx)
                self._accumulate_into(b, dx_drop)
                return
            self.bwd.append(lambda: ops.layernorm_bwd(out.grad, out.t, rstd, None, dx))
            for v in targets:                   # the residual add passes the same gradient to both operands
                self._accumulate_into(v, dx)
        self._tape.append(emit)
        return out

    # ---- linear ---------------------------------------------------------------------------------
    def _linear_on_pieces(self, node, x: Val, w: Val, b: Optional[Val]):
        """F.linear whose input is relu(cat(pieces)) of an all_to_all (kind 'pieces'): forward reads the pieces as
        they lie, the weight gradient does the same, and the data gradient is written, masked with relu's derivative,
        as the pieces of the backward all_to_all."""
        pieces = x.meta["pieces2d"]
        lead = tuple(x.shape[:-1])
        N, K = w.t.shape
        M = pieces[0].shape[0]
        store = self._new(lead + (N,))
        out = Val("tensor", store, needs_grad=True)
        bias = b.meta["master"] if b is not None else None
        relu = bool(x.meta["relu"])
        # pieces that already hold dropout(relu(.)): they are their own mask, and the masked gradient takes the factor
        mask_scale = x.meta.get("mask_scale")
        self.fwd.append(lambda: ops.gemm(None, w.t, store, M, N, K, transB=True, bias=bias, a_segments=pieces, a_relu=relu))

        def emit():
            if out.grad is None:
                return
            dy = out.grad
            gw, accw = self._param_grad_slot(w)
            gb, accb = self._param_grad_slot(b) if b is not None else (None, False)
            self._emit_wgrad(dy, list(pieces), gw, gb, N, K, M, N, K, accw, (w, b), x_relu=relu)
            if x.needs_grad:
                back, finish = x.meta["backward_exchange"]()
                mask = pieces if (relu or mask_scale) else None
                self.bwd.append(lambda: ops.gemm(dy, w.t, None, M, K, N, c_segments=back, mask_segments=mask,
                                                 alpha=mask_scale or 1.0))
                finish()
        self._tape.append(emit)
        return out

    def _linear(self, node):
        x, w, b = self._val(node.args[0]), self._val(node.args[1]), self._val(node.args[2])
        if w.kind != "param" or (b is not None and b.kind != "param"):
            self._unsupported(node, "weight and bias must be parameters")
        if x.kind == "pieces":
            return self._linear_on_pieces(node, x, w, b)
        if x.kind in ("input", "input_slice"):
            # a floating-point program input used as an activation (the MLP models, models.py:19-24): its device
            # buffer in the compute type; load_inputs converts
            if "as_tensor" not in x.meta:
                x.meta["as_tensor"] = Val("tensor", self._input_buffer(x, self.cdt), needs_grad=False)
            x = x.meta["as_tensor"]
        if x.kind == "cls_view":
            xt, lda, lead = x.meta["src"].t, x.meta["row_stride"], (x.meta["src"].t.shape[0],)
        elif x.t is not None:
            xt, lda, lead = x.t, x.ld or x.t.shape[-1], tuple(x.t.shape[:-1])
        else:
            self._unsupported(node, f"linear on a {x.kind} value")
        N, K = w.t.shape
        M = 1
        for s in lead:
            M *= s
        ldc = _round_up(N, self.epv)
        store = self._new(lead + (ldc,))
        out = Val("tensor", store, shape=lead + (N,), ld=ldc if ldc != N else None, needs_grad=True)
        bias = b.meta["master"] if b is not None else None
        # a relu that is the only reader of the result is applied by the GEMM's epilogue; its backward masks the
        # incoming gradient with the stored (activated) output
        fuse = self._wants_fused_relu(node) and ldc == N
        if fuse:
            out.meta["fused_act"] = "relu"
            out.meta["can_fuse_drop"] = N % 2 == 0      # a dropout behind the relu rides on the epilogue as well

        def drop():
            fd = out.meta.get("fused_drop")
            return (fd[0], self.rng_state, fd[1]) if fd else None
        self.fwd.append(lambda: ops.gemm(xt, w.t, store, M, N, K, transB=True, lda=lda, ldc=ldc, bias=bias,
                                         act="relu" if fuse else None, drop=drop()))

        def emit():
            if out.grad is None:
                return
            if fuse:
                self._relu_backward_through(out)
            dy = out.grad
            gw, accw = self._param_grad_slot(w)
            gb, accb = self._param_grad_slot(b) if b is not None else (None, False)
            side = self._side_ok(w, b)

            def wgrad():
                # the bias gradient (column sums of dy) is taken by the same kernel as dy passes through it
                ops.gemm(dy, xt, gw, N, K, M, transA=True, lda=ldc, ldb=lda, accumulate=accw,
                         workspace=self.side_workspace if side else None, a_rowsum=gb)
            if side:
                self._emit_side(wgrad, (dy, xt))
            else:
                self._emit_wgrad(dy, xt, gw, gb, N, K, M, ldc, lda, accw, (w, b))
            if x.kind == "cls_view":
                src = x.meta["src"]
                if src.grad is None:
                    src.grad = self._new(src.t.shape)
                    g = src.grad
                    self.bwd.append(lambda: ops.fill_zero(g))
                g, _ = self._grad_slot(src)
                self.bwd.append(lambda: ops.gemm(dy, w.t, g, M, K, N, lda=ldc, ldc=lda, accumulate=True))
            elif x.needs_grad:
                g, acc, addend = self._grad_slot_addend(x)
                # x is the output of a producer that applied relu itself and this linear is its only reader:
                # the data gradient leaves the GEMM already masked and the separate relu-backward pass is skipped
                mask = None
                if (self.relu_mask_in_dgrad and x.meta.get("fused_act") == "relu" and not acc and x.ld is None and self._only_reader(node, x)
                        and not x.meta.get("relu_bwd_done") and not x.meta.get("relu_bwd_in_split")):
                    mask = x.t
                    x.meta["relu_bwd_done"] = True
                k = self._relu_grad_scale(x) if mask is not None else 1.0
                self.bwd.append(lambda: ops.gemm(dy, w.t, g, M, K, N, lda=ldc, ldc=lda, accumulate=acc, relu_mask=mask,
                                                 addend=addend, alpha=k))
        self._tape.append(emit)
        return out

    def _activation(self, node):
        x = self._val(node.args[0])
        kind = "relu" if node.target is F.relu else ("sigmoid" if node.target is torch.sigmoid else "gelu")
        if node.target is torch.sigmoid and (len(node.args) != 1 or node.kwargs):
            self._unsupported(node, "the program emits torch.sigmoid(input) only")
        if node.target is F.gelu and (len(node.args) > 1 or node.kwargs.get("approximate", "none") != "none"):
            self._unsupported(node, "only the erf form of gelu is implemented")
        if x.kind == "pieces":
            if kind != "relu" or x.meta["relu"]:
                self._unsupported(node, "only one relu is applied to the pieces of an exchange")
            x.meta["relu"] = True                       # applied by the consuming linear as it loads the pieces
            return x
        if x.meta.get("fused_act") == kind:
            return x                                    # already applied by the producer
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"activation on a {x.kind} value")
        out = Val(x.kind if x.kind == "expert" else "tensor", self._new(x.t.shape), shape=x.shape, needs_grad=x.needs_grad)
        self.fwd.append(lambda: ops.act_fwd(x.t, out.t, kind))

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            ref = x.t if kind == "gelu" else out.t      # relu and sigmoid differentiate through their output
            if x.grad is None:
                x.grad = self._new(x.t.shape)
                g = x.grad
                self.bwd.append(lambda: ops.act_bwd(out.grad, ref, g, kind))
            else:
                tmp = self._new(x.t.shape)
                g, _ = self._grad_slot(x)
                self.bwd.append(lambda: (ops.act_bwd(out.grad, ref, tmp, kind), ops.add(g, tmp, g)))
        self._tape.append(emit)
        return out

    def _only_reader(self, node, x: Val, arg: int = 0) -> bool:
        """True when ``node`` is the only consumer of the value ``x`` (its argument number ``arg``), followed back
        through the nodes that pass it on unchanged (the relu a producer already applied, dropout with p = 0)."""
        n = node.args[arg]
        if not (isinstance(n, torch.fx.Node) and self.env.get(n) is x):
            return False
        while isinstance(n, torch.fx.Node) and self.env.get(n) is x:
            if len(n.users) != 1:
                return False
            n = n.args[0] if n.args and isinstance(n.args[0], torch.fx.Node) else None
        return True

    def _wants_fused_relu(self, node):
        users = list(node.users)
        return len(users) == 1 and users[0].target is F.relu

    @staticmethod
    def _relu_grad_scale(out: Val) -> float:
        """1 / (1 - p) of the dropout folded into the producer behind its relu (1 without one)."""
        fd = out.meta.get("fused_drop")
        return 1.0 / (1.0 - fd[0]) if fd else 1.0

    def _relu_backward_through(self, out: Val):
        """For a producer that applied relu itself: d(pre-activation) = d(out) * (out > 0), in place (times the
        factor of a dropout folded in behind the relu)."""
        if out.meta.get("relu_bwd_done"):
            return
        g = out.grad
        k = self._relu_grad_scale(out)
        if len(self._grad_sharers.get(g.untyped_storage().data_ptr(), ())) > 1 or self._is_read_later(g):
            # the buffer is also another value's gradient (or a launch that is held back reads it): mask into a new one
            self.shared_gradient_copies += 1
            out.grad = self._new(g.shape, g.dtype)
            masked = out.grad
            self.bwd.append(lambda: ops.act_bwd(g, out.t, masked, "relu"))
            if k != 1.0:
                self.bwd.append(lambda: ops.scale(masked, k, masked))
            return
        self._guard_write(g)
        self.bwd.append(lambda: ops.act_bwd(g, out.t, g, "relu"))
        if k != 1.0:
            self.bwd.append(lambda: ops.scale(g, k, g))

    # ---- attention ------------------------------------------------------------------------------
    def _mha(self, node):
        kw = {k: self._val(v) for k, v in node.kwargs.items()}
        q = kw["query"]
        if not (kw["key"] is q and kw["value"] is q):
            self._unsupported(node, "self-attention only (query, key and value must be one tensor)")
        if q.kind != "transposed" or q.meta["dims"] != (0, 1):
            self._unsupported(node, "expects the (L, N, E) view produced by transpose(0, 1) of a batch-first tensor")
        if kw.get("bias_k") is not None or kw.get("bias_v") is not None or kw.get("add_zero_attn"):
            self._unsupported(node, "bias_k / bias_v / add_zero_attn are not supported")
        p_drop = float(kw.get("dropout_p", 0.0))
        if not 0.0 <= p_drop <= 1.0:
            self._unsupported(node, f"attention dropout probability {p_drop}")
        x = q.meta["src"]
        E = x.t.shape[2]
        if kw["embed_dim_to_check"] != E or E % kw["num_heads"]:
            self._unsupported(node, "embed_dim mismatch")
        out_bsd = self._attention_core(node, x, kw["in_proj_weight"], kw["in_proj_bias"], kw["out_proj_weight"],
                                       kw["out_proj_bias"], kw["num_heads"], kw.get("attn_mask"), p_drop)
        out = Val("transposed", None, src=out_bsd, dims=(0, 1), needs_grad=True)
        return Val("mha", None, out=out, dropout=out_bsd.meta.get("prob_dropout"))

    def _head_parallel_attention(self, node):
        """models.head_parallel_attention(x, in_proj_weight, in_proj_bias, out_proj_weight, num_heads, attn_mask):
        the heads of this device on the whole batch; the output is the device's partial sum of the output
        projection (no bias), which the program reduce-scatters."""
        args = [self._val(a) for a in node.args]
        x, w_in, b_in, w_out, H = args[:5]
        mask = args[5] if len(args) > 5 else self._val(node.kwargs.get("attn_mask"))
        if x.t is None or x.ld is not None or x.t.dim() != 3:
            self._unsupported(node, "expects a materialised [batch, seq, d] tensor")
        return self._attention_core(node, x, w_in, b_in, w_out, None, H, mask)

    def _attention_core(self, node, x: Val, w_in: Val, b_in: Val, w_out: Val, b_out: Optional[Val], H: int, mask,
                        p_drop: float = 0.0):
        """qkv = x W_in^T + b_in over Ea = H * head_dim attention columns (all heads, or this device's heads),
        softmax attention per head, out = ctx W_out^T (+ b_out).  x is [b, S, d]; W_in [3 Ea, d]; W_out [d_out, Ea].
        ``p_drop`` > 0 (dropout of the probabilities, torch:nn/functional.py:6591): the fused kernels take the keep
        decisions as bit words, written once per step by a kernel of their own; the path that materialises the
        probabilities (float32, other head sizes) runs the dropout kernel over them.  Both take the same decisions."""
        for v in (w_in, b_in, w_out) + ((b_out,) if b_out is not None else ()):
            if v.kind != "param":
                self._unsupported(node, "attention weights must be parameters")
        b, S, d = x.t.shape
        Ea = w_in.t.shape[0] // 3
        d_out = w_out.t.shape[0]
        if tuple(w_in.t.shape) != (3 * Ea, d) or tuple(w_out.t.shape) != (d_out, Ea) or H < 1 or Ea % H:
            self._unsupported(node, f"projection shapes {tuple(w_in.t.shape)} / {tuple(w_out.t.shape)} do not fit "
                                    f"{H} heads on a width-{d} input")
        hd = Ea // H
        if hd % self.epv:
            self._unsupported(node, f"head_dim {hd} must be a multiple of {self.epv}")
        mask_t = None
        if mask is not None:
            if tuple(mask.t.shape) != (S, S) or mask.t.dtype != torch.float32:
                self._unsupported(node, "attn_mask must be a float32 [L, S] additive mask")
            mask_t = mask.t
        scale = 1.0 / math.sqrt(hd)
        fused = (self.fused_attention and self.dtype == "bf16" and hd == 64
                 and (p_drop == 0.0 or (self.fuse_dropout and p_drop < 1.0)))
        # a constant mask (a buffer of the module, not a gathered shard) that is exactly the causal one is
        # applied arithmetically by the fused kernels, which then also skip the key tiles above the diagonal
        causal = False
        if fused and mask is not None and mask.meta.get("name") is not None:
            causal = bool(torch.equal(mask.t.cpu(), torch.triu(torch.full((S, S), float("-inf")), diagonal=1)))
        fused_mask = None if causal else mask_t
        Sp = _round_up(S, self.epv)
        qkv = self._new((b, S, 3 * Ea))
        ctx = self._new((b, S, Ea))
        o = self._new((b, S, d_out))
        if fused:
            lse = self._new((b, H, S), torch.float32)
            P = None
        else:
            P = self._new((b, H, S, Sp))
        out_bsd = Val("tensor", o, needs_grad=True)
        sid = self._node_ids[node]
        if p_drop > 0.0:
            self._uses_rng = True
            out_bsd.meta["prob_dropout"] = (p_drop, sid, (b, H, S, Sp), S)
            if fused:
                # the step's keep decisions in the two bit orders the kernels read; backward takes the forward's
                n_words = ops.attention_keep_words(b, S, H)
                keep_rows, keep_cols = self._new((n_words,), torch.int32), self._new((n_words,), torch.int32)
            else:
                Pd = self._scratch("attn_Pd", (b, H, S, Sp))      # dropout(P): rebuilt from P wherever it is needed
        if not (fused and p_drop > 0.0):
            keep_rows = keep_cols = None
        M = b * S
        sQ, sP = (S * 3 * Ea, hd), (H * S * Sp, S * Sp)
        bias_out = b_out.meta["master"] if b_out is not None else None

        def forward():
            ops.gemm(x.t, w_in.t, qkv, M, 3 * Ea, d, transB=True, bias=b_in.meta["master"])
            if fused:
                if keep_rows is not None:
                    ops.attention_keep_bits(keep_rows, keep_cols, b, S, H, Sp, p_drop, self.rng_state, sid)
                ops.attention_fwd(qkv, fused_mask, ctx, lse, b, S, H, scale, causal, keep_rows, p_drop)
            else:
                ops.gemm(qkv, qkv, P, S, S, hd, transB=True, lda=3 * Ea, ldb=3 * Ea, ldc=Sp, alpha=scale, batch1=b,
                         batch2=H, strideA=sQ, strideB=sQ, strideC=sP, offB=Ea)
                ops.softmax_fwd(P, mask_t, P, b * H * S, S, Sp, S)
                Pv = P
                if p_drop > 0.0:
                    ops.dropout(P, Pd, p_drop, self.rng_state, sid)
                    Pv = Pd
                ops.gemm(Pv, qkv, ctx, S, hd, S, lda=Sp, ldb=3 * Ea, ldc=Ea, batch1=b, batch2=H, strideA=sP, strideB=sQ,
                         strideC=(S * Ea, hd), offB=2 * Ea)
            ops.gemm(ctx, w_out.t, o, M, d_out, Ea, transB=True, bias=bias_out)
        self.fwd.append(forward)

        def emit():
            if out_bsd.grad is None:
                return
            do = out_bsd.grad
            dctx = self._scratch("attn_dctx", (b, S, Ea))
            side = self._side_ok(w_out, b_out, w_in, b_in)
            held = not side and self._holds_back_wgrad((w_in, b_in))
            # the in-projection's weight gradient reads dqkv from the side stream, or later together with the next
            # layers' (wgrad_group), so it cannot be shared scratch then
            dqkv = self._new((b, S, 3 * Ea)) if (side or held) else self._scratch("attn_dqkv", (b, S, 3 * Ea))
            if fused:
                delta = self._scratch("attn_delta", (b, H, S), torch.float32)
            else:
                dP = self._scratch("attn_dP", (b, H, S, Sp))
            gwo, acc_wo = self._param_grad_slot(w_out)
            gbo, acc_bo = self._param_grad_slot(b_out) if b_out is not None else (None, False)
            gwi, acc_wi = self._param_grad_slot(w_in)
            gbi, acc_bi = self._param_grad_slot(b_in)
            if side:
                gx, acc_x = self._grad_slot(x) if x.needs_grad else (None, False)
                addend_x = None
            else:
                # first in the list (as before); held back, it keeps reading `do`, which d(x) usually aliases (the
                # residual add hands one buffer to both): the in-projection's data gradient then goes to a new buffer
                self._emit_wgrad(do, ctx, gwo, gbo, d_out, Ea, M, d_out, Ea, acc_wo, (w_out, b_out))
                gx, acc_x, addend_x = self._grad_slot_addend(x) if x.needs_grad else (None, False, None)

            ws = self.side_workspace if side else None

            def wgrad_out():
                ops.gemm(do, ctx, gwo, d_out, Ea, M, transA=True, accumulate=acc_wo, workspace=ws, a_rowsum=gbo)

            def wgrad_in():
                ops.gemm(dqkv, x.t, gwi, 3 * Ea, d, M, transA=True, accumulate=acc_wi, workspace=ws, a_rowsum=gbi)

            def backward():
                ops.gemm(do, w_out.t, dctx, M, Ea, d_out)
                if fused:
                    ops.attention_bwd(qkv, ctx, dctx, lse, fused_mask, dqkv, delta, b, S, H, scale, causal, keep_rows,
                                      keep_cols, p_drop)
                else:
                    # dP = dctx V^T ; dV = P^T dctx
                    ops.gemm(dctx, qkv, dP, S, S, hd, transB=True, lda=Ea, ldb=3 * Ea, ldc=Sp, batch1=b, batch2=H,
                             strideA=(S * Ea, hd), strideB=sQ, strideC=sP, offB=2 * Ea)
                    Pv = P
                    if p_drop > 0.0:
                        ops.dropout(P, Pd, p_drop, self.rng_state, sid)      # the forward's dropped probabilities again
                        ops.dropout(dP, dP, p_drop, self.rng_state, sid)     # d(P) = d(dropout(P)) * keep / (1 - p)
                        Pv = Pd
                    ops.gemm(Pv, dctx, dqkv, S, hd, S, transA=True, lda=Sp, ldb=Ea, ldc=3 * Ea, batch1=b, batch2=H,
                             strideA=sP, strideB=(S * Ea, hd), strideC=sQ, offC=2 * Ea)
                    ops.softmax_bwd(dP, P, dP, b * H * S, S, Sp)
                    # dQ = scale dS K ; dK = scale dS^T Q
                    ops.gemm(dP, qkv, dqkv, S, hd, S, lda=Sp, ldb=3 * Ea, ldc=3 * Ea, alpha=scale, batch1=b, batch2=H,
                             strideA=sP, strideB=sQ, strideC=sQ, offB=Ea)
                    ops.gemm(dP, qkv, dqkv, S, hd, S, transA=True, lda=Sp, ldb=3 * Ea, ldc=3 * Ea, alpha=scale, batch1=b,
                             batch2=H, strideA=sP, strideB=sQ, strideC=sQ, offC=Ea)

            def dgrad_in():
                ops.gemm(dqkv, w_in.t, gx, M, d, 3 * Ea, accumulate=acc_x, addend=addend_x)
            if side:
                # do is final here; dqkv is final once `backward` is enqueued.  d(x) usually aliases do (the
                # residual add hands one buffer to both), so the in-projection's data gradient, which
                # accumulates into it, is ordered after the out-projection's weight gradient.
                self._emit_side(wgrad_out, (do, ctx))
                self.bwd.append(backward)
                self._emit_side(wgrad_in, (dqkv, x.t))
            else:
                self.bwd.append(backward)
                self._emit_wgrad(dqkv, x.t, gwi, gbi, 3 * Ea, d, M, 3 * Ea, d, acc_wi, (w_in, b_in))
            if gx is not None:
                if acc_x and addend_x is None:
                    self._guard_write(gx)
                self.bwd.append(dgrad_in)
        self._tape.append(emit)
        return out_bsd

    # ---- loss -----------------------------------------------------------------------------------
    def _log_softmax(self, node):
        v, dim = self._val(node.args[0]), node.args[1]
        nd = len(v.shape)
        if dim < 0:
            dim += nd
        if v.t is None or dim != nd - 1:
            self._unsupported(node, "log_softmax over the last dimension of a materialised tensor only")
        for u in node.users:
            if u.target not in (torch.transpose, F.nll_loss):
                self._unsupported(node, "log-probabilities may only feed transpose / nll_loss")
        return Val("logprobs", src=v, transposed=False)

    def _nll_loss(self, node):
        lp, y = self._val(node.args[0]), self._val(node.args[1])
        if node.kwargs.get("reduction") != "sum" or lp.kind != "logprobs":
            self._unsupported(node, "expects nll_loss(log_softmax(...), target, reduction='sum')")
        logits = lp.meta["src"]
        nd = len(logits.shape)
        if (nd == 3) != bool(lp.meta["transposed"]):
            self._unsupported(node, "class dimension must be dim 1 of the nll_loss input")
        V = logits.shape[-1]
        ld = logits.ld or V
        rows = logits.t.numel() // ld
        tgt = self._input_buffer(y, torch.int64)
        row_loss = self._new((rows,), torch.float32)
        loss = self._new((1,), torch.float32)
        ignore = node.kwargs.get("ignore_index", -100)

        def forward():
            # writes d(loss)/d(logits) over the logits: the backward pass starts from it
            ops.logsoftmax_nll(logits.t, tgt, row_loss, logits.t, rows, V, ld, ignore, 1.0)
            ops.sum_f32(row_loss, loss)
        self.fwd.append(forward)
        logits.grad = logits.t
        return Val("loss", loss)

    def _sum(self, node):
        """torch.sum(input) (hap.rs:1133): the sum of all elements as the program's (partial) loss, the output of
        the reference's MLP models (models.py:24).  Backward starts from d(input) = 1."""
        if len(node.args) != 1 or node.kwargs:
            self._unsupported(node, "the program emits torch.sum(input) only")
        x = self._val(node.args[0])
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"sum of a {x.kind} value")
        if any(u.op != "output" for u in node.users):
            self._unsupported(node, "torch.sum is supported as the program's output")
        width = x.t.shape[-1]
        rows = x.t.numel() // width
        cols = self._new((width,), torch.float32)
        loss = self._new((1,), torch.float32)
        self.fwd.append(lambda: (ops.colsum(x.t, cols, rows, width), ops.sum_f32(cols, loss)))

        def emit():
            if not x.needs_grad:
                return
            g, acc = self._grad_slot(x)
            if acc:
                ones = self._new(x.t.shape)
                self.bwd.append(lambda: (ops.fill_value(ones, 1.0), ops.add(g, ones, g)))
            else:
                self.bwd.append(lambda: ops.fill_value(g, 1.0))
        self._tape.append(emit)
        return Val("loss", loss)

    # ---- ViT leaves -----------------------------------------------------------------------------
    def _conv2d(self, node):
        x, w, b = self._val(node.args[0]), self._val(node.args[1]), self._val(node.args[2])
        stride, padding, dilation, groups = node.args[3], node.args[4], node.args[5], node.args[6]
        d, C, ph, pw = w.t.shape
        if tuple(stride) != (ph, pw) or tuple(padding) != (0, 0) or tuple(dilation) != (1, 1) or groups != 1:
            self._unsupported(node, "only the patch-embedding form (kernel = stride, no padding) is supported")
        img = self._input_buffer(x, torch.float32)
        n, _, Hh, Ww = img.shape
        gh, gw = Hh // ph, Ww // pw
        Kc = C * ph * pw
        if Kc % self.epv:
            self._unsupported(node, "C*ph*pw must be a multiple of the vector width")
        cols = self._new((n * gh * gw, Kc))
        tokens = Val("tensor", self._new((n, gh * gw, d)), needs_grad=True)
        M = n * gh * gw

        def forward():
            ops.patchify(img, cols, n, C, gh, gw, ph, pw)
            ops.gemm(cols, w.t, tokens.t, M, d, Kc, transB=True, bias=b.meta["master"])
        self.fwd.append(forward)

        def emit():
            if tokens.grad is None:
                return
            gw_, accw = self._param_grad_slot(w)
            gb_, accb = self._param_grad_slot(b)
            dy = tokens.grad
            self.bwd.append(lambda: (ops.gemm(dy, cols, gw_, d, Kc, M, transA=True, accumulate=accw),
                                     ops.colsum(dy, gb_, M, d, d, accb)))
        self._tape.append(emit)
        return Val("conv_out", None, tokens=tokens, shape=(n, d, gh, gw))

    def _flatten(self, node):
        v = self._val(node.args[0])
        if v.kind != "conv_out" or node.args[1] != 2 or node.args[2] != -1:
            self._unsupported(node, "flatten(2, -1) of the patch convolution only")
        return Val("conv_flat", None, tokens=v.meta["tokens"])

    def _append_cls(self, node):
        x, cls = self._val(node.args[0]), self._val(node.args[1])
        users = list(node.users)
        if len(users) == 1 and users[0].target is operator.add:
            return Val("cls_appended", None, x=x, cls=cls)          # decided at the add: fused if it adds [1, T + 1, d]
        return self._append_cls_pos(node, Val("cls_appended", None, x=x, cls=cls), None)

    def _append_cls_pos(self, node, ac: Val, pos: Optional[Val]):
        """append_cls_token, fused with the position-embedding add that follows it in the reference's ViT
        (models.py:167) or, ``pos`` None, on its own."""
        x, cls = ac.meta["x"], ac.meta["cls"]
        n, T, d = x.t.shape
        if pos is not None and tuple(pos.t.shape) != (1, T + 1, d):
            self._unsupported(node, "position embedding must be [1, T+1, d]")
        out = Val("tensor", self._new((n, T + 1, d)), needs_grad=True)
        pos_t = pos.t if pos is not None else None
        self.fwd.append(lambda: ops.append_cls_pos(x.t, cls.t, pos_t, out.t, n, T, d))

        def emit():
            if out.grad is None:
                return
            g = out.grad
            if pos is not None and pos.kind == "param":
                gp, accp = self._param_grad_slot(pos)
                self.bwd.append(lambda: ops.colsum(g, gp, n, (T + 1) * d, (T + 1) * d, accp))
            if cls.kind == "param":
                gc, accc = self._param_grad_slot(cls)
                self.bwd.append(lambda: ops.colsum(g, gc, n, d, (T + 1) * d, accc))
            if x.needs_grad:
                if x.grad is None:
                    x.grad = self._new(x.t.shape)
                    gx = x.grad
                    self.bwd.append(lambda: ops.slice_rows(g, 1, 1, T, gx))
                else:
                    tmp = self._new(x.t.shape)
                    gx, _ = self._grad_slot(x)
                    self.bwd.append(lambda: (ops.slice_rows(g, 1, 1, T, tmp), ops.add(gx, tmp, gx)))
        self._tape.append(emit)
        return out

    def _get_cls(self, node):
        v = self._val(node.args[0])
        n, T, d = v.t.shape
        return Val("cls_view", None, src=v, row_stride=T * d, shape=(n, d), needs_grad=v.needs_grad)

    # ---- collectives (device-local halves + wire) ---------------------------------------------
    def _peers(self, tag, direction, rank, W, shape, reduction, dtype=None):
        out = {}
        for src in range(W):
            if src != rank:
                out[src] = self.wire.recv(tag, direction, src, shape, dtype or self.cdt, self.dev, reduction=reduction)
        return out

    def _announce(self, tag, direction, rank, W, buffer_for, sink: List[Callable]):
        """Tell the wire which static buffer holds the message for every peer; a callable it returns runs in
        every step right after the preparation kernels (enqueued just before this call) of the collective."""
        for dst in range(W):
            if dst != rank:
                hook = self.wire.send(tag, direction, dst, buffer_for(dst))
                if hook is not None:
                    # through host_call, so that the hook also sits in the recorded launch list that later steps replay
                    self._send_hooks += 1
                    sink.append(lambda hook=hook: ops._lib.host_call(hook))

    def _emit_gather(self, tag, direction, x_t, dim, L, rank, sink: List[Callable], full=None):
        """pad own shard -> [wire] -> cut pads and concatenate.  Returns the full tensor.  ``full``: the result's
        buffer when the producer of ``x_t`` already wrote the shard at its rows of it (_place_gather_inputs)."""
        m, W = max(L), len(L)
        pshape = ops._with_dim(x_t.shape, dim, m)
        # a shard of the longest length needs no padding: the tensor itself is the message
        unpadded = L[rank] == m and x_t.is_contiguous() and tuple(x_t.shape) == tuple(pshape)
        own = x_t if unpadded else self._new(pshape, x_t.dtype)
        if full is None:
            full = self._new(ops._with_dim(x_t.shape, dim, sum(L)), x_t.dtype)
        # Along dim 0 a peer's shard is received straight into its rows of the result (the payload rows of a shard that
        # was padded to the longest length).  Only in the forward direction, where the result is an activation that no
        # launch writes afterwards; a gathered gradient may be accumulated into in place by other consumers.
        into = {}
        if self.receive_in_place and dim == 0 and direction == "fwd":
            into = {s: full.narrow(0, sum(L[:s]), L[s]) for s in range(W) if s != rank and L[s] > 0}
            if into:
                self._wire_backed.add(full.untyped_storage().data_ptr())
        peers = {s: self.wire.recv(tag, direction, s, pshape, x_t.dtype, self.dev, reduction=False, into=into.get(s))
                 for s in range(W) if s != rank}
        row = full[0].numel() * full.element_size() if full.dim() > 0 and full.shape[0] > 0 else 0
        own_placed = dim == 0 and x_t.is_contiguous() and x_t.data_ptr() == full.data_ptr() + sum(L[:rank]) * row
        slices = [(x_t if (unpadded or own_placed) else own) if s == rank else peers[s] for s in range(W)]
        placed = all(L[s] == 0 or (dim == 0 and slices[s] is not None and slices[s].is_contiguous()
                                   and slices[s].data_ptr() == full.data_ptr() + sum(L[:s]) * row) for s in range(W))
        if not unpadded:
            sink.append(lambda: ops.pad_rows(x_t, dim, m, own))
        if not placed:
            sink.append(lambda: ops.unpad_concat(slices, L, dim, full))
        self._announce(tag, direction, rank, W, lambda dst: own, sink)        # the padded shard goes to every peer
        return full

    def _emit_scatter(self, tag, direction, full_t, dim, L, rank, sink: List[Callable], out_t=None, addend=None):
        """split + pad -> [wire] -> rank-ordered float32 sum of the pieces for this rank, pad cut off; ``addend``
        (the output's shape) is added to the sum in the same pass."""
        m, W = max(L), len(L)
        pshape = ops._with_dim(full_t.shape, dim, m)
        peers = self._peers(tag, direction, rank, W, pshape, True, full_t.dtype)
        out = out_t if out_t is not None else self._new(ops._with_dim(full_t.shape, dim, L[rank]), full_t.dtype)
        if dim == 0 and full_t.is_contiguous() and L[rank] > 0:
            # along dim 0 this rank's own piece is a contiguous row range of the full tensor: the sum reads it there
            # (and the first L[rank] rows of the peers' padded pieces), and no padded copy of it is made; a peer's
            # piece of the longest length needs no padding either: its rows of the full tensor are the message
            in_place = [s != rank and self.receive_in_place and L[s] == m for s in range(W)]
            sent = [None if (s == rank or in_place[s]) else self._new(pshape, full_t.dtype) for s in range(W)]
            messages = [full_t.narrow(0, sum(L[:s]), m) if in_place[s] else sent[s] for s in range(W)]
            own = full_t.narrow(0, sum(L[:rank]), L[rank])
            contribs = [own if s == rank else (peers[s].narrow(0, 0, L[rank]) if peers[s] is not None else None)
                        for s in range(W)]
        else:
            sent = [self._new(pshape, full_t.dtype) for _ in range(W)]
            messages = sent
            contribs = [sent[rank] if s == rank else peers[s] for s in range(W)]
        contribs = [c for c in contribs if c is not None]
        if any(t is not None for t in sent):
            sink.append(lambda: ops.split_pad(full_t, L, dim, m, sent))
        sink.append(lambda: ops.ragged_reduce(contribs, dim, 0, L[rank], out, addend=addend))
        self._announce(tag, direction, rank, W, lambda dst: messages[dst], sink)  # the padded piece that rank dst reduces
        return out

    def _all_gather(self, node):
        x, dim, L, rank = self._val(node.args[0]), node.args[1], list(node.args[2]), node.args[3]
        if x.kind == "param":
            return self._gathered_param(node, x, dim, L, rank)
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"all_gather of a {x.kind} value")
        full = self._emit_gather(node.name, "fwd", x.t, dim, L, rank, self.fwd, full=self._gather_results.pop(node, None))
        out = Val("tensor", full, needs_grad=x.needs_grad)

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            if x.grad is None:
                x.grad = self._emit_scatter(node.name, "bwd", out.grad, dim, L, rank, self.bwd)
            else:
                # d(x) += the reduced piece, in the reduction's own pass: in place, or into a new buffer while
                # weight gradients that are held back still read the old one
                g = x.grad
                if self._is_read_later(g) or self._shared_with_pending(x):
                    x.grad = self._new(g.shape, g.dtype)
                else:
                    self._guard_write(g)
                self._emit_scatter(node.name, "bwd", out.grad, dim, L, rank, self.bwd, out_t=x.grad, addend=g)
        self._tape.append(emit)
        return out

    def _gathered_param(self, node, x: Val, dim, L, rank):
        """A parameter stored as its dim-0 shard and gathered at use (get_attr_zero, hap.rs:2527-2547).  Forward:
        the shard (bf16 shadow for matrices, float32 master for vectors, which consumers add in float32) is
        gathered every step.  The consumers see a whole parameter whose float32 gradient is a buffer of the
        whole shape; once they have all written it, that gradient is reduce-scattered into the shard's slot
        of the flat gradient buffer (AllGather.backward, collectives.py:22-29)."""
        if dim != 0 or x.t.shape[0] != L[rank]:
            self._unsupported(node, "a gathered parameter must be a dim-0 shard of the plan's length")
        vector = x.t.dim() == 1
        src = x.meta["master"] if vector else x.t
        full = self._emit_gather(node.name, "fwd", src, 0, L, rank, self.fwd)
        full_grad = self._gathered_grads[x.meta["name"]]
        out = Val("param", full, master=full if vector else None, grad=full_grad, needs_grad=True, shard_of=x.meta["name"],
                  single_use=len(node.users) == 1)

        def emit():
            if not out.meta.get("grad_written"):
                return
            x.meta["grad_written"] = True
            if self._touched is not None:
                self._touched.append(x.meta["name"])
            # the consumer's weight gradient writes full_grad; it may be held back to share a launch with later layers
            self._after_wgrad(full_grad, lambda: self._emit_scatter(node.name, "bwd", full_grad, 0, L, rank, self.bwd,
                                                                    out_t=x.meta["grad"]))
        self._tape.append(emit)
        return out

    def _reduce_scatter(self, node):
        x, dim, L, rank = self._val(node.args[0]), node.args[1], list(node.args[2]), node.args[3]
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"reduce_scatter of a {x.kind} value")
        piece = self._emit_scatter(node.name, "fwd", x.t, dim, L, rank, self.fwd)
        out = Val("tensor", piece, needs_grad=x.needs_grad)

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            full = self._emit_gather(node.name, "bwd", out.grad, dim, L, rank, self.bwd)
            self._accumulate_into(x, full)
        self._tape.append(emit)
        return out

    def _emit_exchange(self, tag, direction, x_t, split_dim, cat_dim, split_L, cat_L, rank, sink, act=None,
                       relu_of=None, receive_in_place=False, presplit=False, drop_from: Optional[Val] = None,
                       relu_scale: float = 1.0):
        """The local half of an all_to_all.  ``act``: activation applied while concatenating.  ``relu_of``: forward
        output of a relu whose backward is applied to ``x_t`` while splitting (only for a split that copies).
        ``receive_in_place`` (concatenation along dim 0, no activation): the peers' pieces are received straight
        into their rows of the result, which nothing may write afterwards; no concat launch is left.
        ``presplit``: ``x_t`` is only a shape (a meta tensor); the caller writes the pieces itself (a GEMM whose result
        is laid out in pieces).  Returns (result, pieces, finish): nothing is launched until ``finish()`` appends
        what is left of the exchange (the concat, the wire's send hooks).
        ``drop_from``: the value this exchange produces; if a dropout behind the fused relu has been folded into it
        (meta fused_drop, set after this call), the concat applies it too.  ``relu_scale``: factor on ``relu_of``'s
        masked gradient (that dropout's 1 / (1 - p))."""
        W = len(split_L)
        # pieces along the slowest dimension are contiguous ranges of the input: views, as torch.split gives the
        # reference (collectives.py:156); any other dimension needs the strided copy
        views = split_dim == 0 and not presplit and x_t.is_contiguous()
        own_shape = ops._with_dim(x_t.shape, split_dim, split_L[rank])
        out = self._new(ops._with_dim(own_shape, cat_dim, sum(cat_L)))
        if views:
            pieces = list(torch.split(x_t, list(split_L), 0))
        else:
            pieces = [self._new(ops._with_dim(x_t.shape, split_dim, l)) for l in split_L]
            if cat_dim == 0:
                # the copying split writes this rank's own piece straight to its rows of the concatenation
                pieces[rank] = out.narrow(0, sum(cat_L[:rank]), cat_L[rank])
        own = pieces[rank]
        parts = []
        for src in range(W):
            if src == rank:
                parts.append(own)
            else:
                shape = ops._with_dim(own.shape, cat_dim, cat_L[src])
                into = None
                if receive_in_place and cat_dim == 0 and act is None and not views and cat_L[src] > 0:
                    into = out.narrow(0, sum(cat_L[:src]), cat_L[src])
                    self._wire_backed.add(out.untyped_storage().data_ptr())
                parts.append(self.wire.recv(tag, direction, src, shape, self.cdt, self.dev, reduction=False, into=into))

        def drop():
            fd = drop_from.meta.get("fused_drop") if drop_from is not None else None
            return (fd[0], self.rng_state, fd[1]) if fd else None

        def finish():
            if views or presplit:
                sink.append(lambda: ops.concat_rows(parts, cat_dim, out, act, drop()))
            else:
                sink.append(lambda: (ops.split_rows(x_t, split_L, split_dim, pieces, relu_of=relu_of, scale=relu_scale),
                                     ops.concat_rows(parts, cat_dim, out, act, drop())))
            self._announce(tag, direction, rank, W, lambda dst: pieces[dst], sink)
        if presplit:
            return out, pieces, finish
        finish()
        return out

    def _exchange_in_pieces(self, node, x: Val, sd, cd, sL, cL, rank):
        """all_to_all whose result only feeds relu -> linear: nothing is copied.  The value is the list of pieces
        (this rank's own rows of the input, the peers' messages where the wire delivered them); the linear reads
        them in place, and its backward writes the pieces of the backward exchange."""
        W = len(sL)
        x_t = x.t
        pieces = list(torch.split(x_t, list(sL), 0))
        own = pieces[rank]
        parts = []
        for src in range(W):
            shape = ops._with_dim(own.shape, cd, cL[src])
            parts.append(own if src == rank else
                         self.wire.recv(node.name, "fwd", src, shape, self.cdt, self.dev, reduction=False))
        self._announce(node.name, "fwd", rank, W, lambda dst: pieces[dst], self.fwd)
        live = [t for t, l in zip(parts, cL) if l > 0]
        out = Val("pieces", None, shape=ops._with_dim(own.shape, cd, sum(cL)), needs_grad=x.needs_grad, relu=False,
                  pieces=parts, pieces2d=[t.reshape(-1, t.shape[-1]) for t in live])

        def backward_exchange():
            # the gradient [own rows, sum(cL)] never exists as one tensor: the linear's data-gradient GEMM writes it
            # as the pieces of the backward exchange (split along cd by cL, concatenated along sd by sL)
            shape = torch.empty(out.shape, device="meta")
            # the result is d(x); when x is a linear's output that only this exchange reads, d(x) is read by that
            # linear's two gradient GEMMs and written by nobody: the peers' pieces can be received in place
            producer = node.args[0]
            in_place = (self.receive_in_place and x.grad is None and isinstance(producer, torch.fx.Node)
                        and producer.target is F.linear and len(producer.users) == 1 and not x.meta.get("fused_act"))
            g, back, finish = self._emit_exchange(node.name, "bwd", shape, cd, sd, cL, sL, rank, self.bwd,
                                                  receive_in_place=in_place, presplit=True)

            def done():
                finish()
                self._accumulate_into(x, g)
            return [t.reshape(-1, t.shape[-1]) for t, l in zip(back, cL) if l > 0], done
        out.meta["backward_exchange"] = backward_exchange
        return out

    def _feeds_only_relu_linear(self, node) -> bool:
        """node -> F.relu -> [F.dropout]* -> F.linear (as its input), every link the only user; of the dropouts at
        most one has p > 0 (it gets a pass of its own over the pieces)."""
        users = list(node.users)
        if len(users) != 1 or users[0].target is not F.relu:
            return False
        n = users[0]
        live = 0
        while True:
            users = list(n.users)
            if len(users) != 1:
                return False
            u = users[0]
            if u.target is F.dropout and u.args[0] is n and len(u.args) == 2 and not u.kwargs:
                p = float(u.args[1])
                live += p > 0.0
                if p >= 1.0 or live > 1 or (p > 0.0 and not self.fuse_dropout):
                    return False
                n = u
                continue
            return u.target is F.linear and u.args[0] is n and u.args[1] is not n and u.args[2] is not n

    @staticmethod
    def _split_can_mask(grad, fwd_out, dim, lengths):
        """The masked split works on 16-byte vectors: every piece's rows and both base addresses must be aligned."""
        if not (grad.is_contiguous() and fwd_out.is_contiguous() and grad.shape == fwd_out.shape and grad.dtype == fwd_out.dtype):
            return False
        inner = 1
        for d in grad.shape[dim + 1:]:
            inner *= d
        es = grad.element_size()
        return (grad.data_ptr() % 16 == 0 and fwd_out.data_ptr() % 16 == 0
                and all((l * inner * es) % 16 == 0 for l in lengths))

    def _all_to_all(self, node):
        x, sd, cd = self._val(node.args[0]), node.args[1], node.args[2]
        sL, cL, rank = list(node.args[3]), list(node.args[4]), node.args[5]
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"all_to_all of a {x.kind} value")
        if any(u.target is torch.log_softmax for u in node.users):
            # ShardingPlan(decoder="vocabulary"): the generator emits it and the CPU tests pin it against the
            # single-device model; the logits' exchange (pieces whose widths are no multiple of the 16-byte vector,
            # e.g. 11446 of 30522 columns) has no GPU parity test yet, so the executor does not run it
            self._unsupported(node, "an all_to_all in front of log_softmax (the vocabulary-split output projection) is "
                                    "not built in this executor")
        # piece boundaries: multiples of 64 for the k-tiles of the forward GEMM and of 128, the narrowest bf16 tile,
        # for the N tiles of the two backward GEMMs
        bounds = [sum(cL[:i]) for i in range(1, len(cL))]
        if (self.exchange_in_pieces and self.dtype == "bf16" and sd == 0 and cd == x.t.dim() - 1 and x.t.is_contiguous()
                and self._feeds_only_relu_linear(node) and all(v % 128 == 0 for v in bounds) and sum(cL) % 64 == 0
                and sum(1 for l in cL if l > 0) <= ops._lib.GEMM_MAX_SEGMENTS and sL[rank] > 0 and x.t.shape[-1] % 8 == 0):
            return self._exchange_in_pieces(node, x, sd, cd, sL, cL, rank)
        fuse = self._wants_fused_relu(node)
        out = Val("tensor", None, needs_grad=x.needs_grad)
        out.t = self._emit_exchange(node.name, "fwd", x.t, sd, cd, sL, cL, rank, self.fwd, "relu" if fuse else None,
                                    drop_from=out)
        out.shape = tuple(out.t.shape)
        if fuse:
            out.meta["fused_act"] = "relu"
            # a dropout behind the relu can ride on the same copy (16-byte vectors of the result)
            out.meta["can_fuse_drop"] = self._split_can_mask(out.t, out.t, cd, cL)
            # the backward exchange splits along the forward's concat dimension; where that split copies, relu's
            # backward rides on the copy instead of a pass of its own over the gradient (or a mask read in the
            # next linear's data-gradient GEMM)
            out.meta["relu_bwd_in_split"] = self.relu_bwd_in_split and cd != 0 and self._split_can_mask(out.t, out.t, cd, cL)

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            in_split = (fuse and out.meta["relu_bwd_in_split"] and not out.meta.get("relu_bwd_done")
                        and self._split_can_mask(out.grad, out.t, cd, cL))
            if fuse and not in_split:
                self._relu_backward_through(out)
            # The result is d(x).  When x is a linear's output that only this exchange reads, d(x) is read by that
            # linear's two gradient GEMMs and written by nobody: the peers' pieces can be received in place.
            producer = node.args[0]
            in_place = (self.receive_in_place and x.grad is None and isinstance(producer, torch.fx.Node)
                        and producer.target is F.linear and len(producer.users) == 1 and not x.meta.get("fused_act"))
            g = self._emit_exchange(node.name, "bwd", out.grad, cd, sd, cL, sL, rank, self.bwd,
                                    relu_of=out.t if in_split else None, receive_in_place=in_place,
                                    relu_scale=self._relu_grad_scale(out) if in_split else 1.0)
            self._accumulate_into(x, g)
        self._tape.append(emit)
        return out

    def _emit_sum(self, tag, direction, x_t, rank, W, sink, out_t=None):
        peers = self._peers(tag, direction, rank, W, x_t.shape, True)
        contribs = [x_t if s == rank else peers[s] for s in range(W)]
        contribs = [c.view(1, -1) for c in contribs if c is not None]
        out = out_t if out_t is not None else self._new(x_t.shape, x_t.dtype)
        n = x_t.numel()
        self._announce(tag, direction, rank, W, lambda dst: x_t, sink)         # before the sum (it may run in place)
        sink.append(lambda: ops.ragged_reduce(contribs, 1, 0, n, out.view(1, -1)))
        return out

    def _all_reduce(self, node):
        x = self._val(node.args[0])
        if x.t is None or x.ld is not None:
            self._unsupported(node, f"all_reduce of a {x.kind} value")
        rank, W = self.rank_hint, self.world_hint
        if x.kind == "expert":
            return self._all_reduce_expert(node, x, rank, W)
        t = self._emit_sum(node.name, "fwd", x.t, rank, W, self.fwd)
        out = Val("tensor", t, needs_grad=x.needs_grad)

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            g = self._emit_sum(node.name, "bwd", out.grad, rank, W, self.bwd)
            self._accumulate_into(x, g)
        self._tape.append(emit)
        return out

    def _all_reduce_expert(self, node, x: Val, rank, W):
        """all_reduce of expert-major activations (the partial sums of an expert product over a split model
        dimension, hap.rs:3331-3335, or the dispatched tokens of a split over positions, hap.rs:3300-3304).  The
        program's tensor is [B, E, C, N] and that is what crosses the wire; the
        storage here is [E, B, C, N], so the value is brought into the program's order before the sum and back
        behind it (two strided copies per direction)."""
        El, B, C, N = x.t.shape
        each = [1] * El

        def to_program_order(src, dst):          # [E, B, C, N] -> [B, E, C, N]
            ops.concat_rows([src[e].view(B, 1, C * N) for e in range(El)], 1, dst.view(B, El, C * N))

        def to_expert_major(src, dst):           # [B, E, C, N] -> [E, B, C, N]
            ops.split_rows(src.view(B, El, C * N), each, 1, [dst[e].view(B, 1, C * N) for e in range(El)])

        mine = self._new((B, El, C, N))
        self.fwd.append(lambda: to_program_order(x.t, mine))
        total = self._emit_sum(node.name, "fwd", mine, rank, W, self.fwd)
        out = Val("expert", self._new(x.t.shape), shape=x.shape, needs_grad=x.needs_grad)
        self.fwd.append(lambda: to_expert_major(total, out.t))

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            g_mine = self._new((B, El, C, N))
            dy = out.grad
            self.bwd.append(lambda: to_program_order(dy, g_mine))
            g_total = self._emit_sum(node.name, "bwd", g_mine, rank, W, self.bwd)
            g = self._new(x.t.shape)
            self.bwd.append(lambda: to_expert_major(g_total, g))
            self._accumulate_into(x, g)
        self._tape.append(emit)
        return out

    def _dynamic_slice(self, node):
        v, dim, L, rank = self._val(node.args[0]), node.args[1], list(node.args[2]), node.args[3]
        if v.kind == "routing" and dim in (1, 2, 3):
            # the device's window of the dense [B, S, E, C] tensor: positions (dim 1), experts (dim 2), capacity slots (dim 3)
            m = dict(which=v.meta["which"], gating=v.meta["gating"], e_lo=v.meta["e_lo"], E_loc=v.meta["E_loc"],
                     c_lo=v.meta["c_lo"], C_loc=v.meta["C_loc"], s_lo=v.meta["s_lo"], S_loc=v.meta["S_loc"])
            lo, n = {1: ("s_lo", "S_loc"), 2: ("e_lo", "E_loc"), 3: ("c_lo", "C_loc")}[dim]
            if sum(L) != m[n]:
                self._unsupported(node, f"the lengths {L} do not add up to the extent {m[n]} of dimension {dim}")
            m[lo], m[n] = m[lo] + sum(L[:rank]), L[rank]
            return Val("routing", **m)
        if v.t is None or v.ld is not None:
            self._unsupported(node, f"dynamic_slice of a {v.kind} value")
        off = sum(L[:rank])
        out = Val("tensor", self._new(ops._with_dim(v.t.shape, dim, L[rank])), needs_grad=v.needs_grad)
        self.fwd.append(lambda: ops.slice_rows(v.t, dim, off, L[rank], out.t))

        def emit():
            if out.grad is None or not v.needs_grad:
                return
            full = self._new(v.t.shape)
            self.bwd.append(lambda: (ops.fill_zero(full), ops.place_rows(out.grad, full, dim, off)))
            self._accumulate_into(v, full)
        self._tape.append(emit)
        return out

    # ---- mixture of experts -----------------------------------------------------------------------
    def _gating(self, node):
        x, E, C, wg = self._val(node.args[0]), node.args[1], node.args[2], self._val(node.args[3])
        if x.t is None or wg.kind != "param":
            self._unsupported(node, "gating expects a materialised input and a parameter")
        B, S, d = x.t.shape
        if E % self.epv:
            self._unsupported(node, f"n_expert must be a multiple of {self.epv}")
        logits = self._new((B, S, E), torch.float32)
        r = dict(probs=self._new((B, S, E), torch.float32), index=self._new((B, S, 2), torch.int32),
                 slot=self._new((B, S, 2), torch.int32), gate=self._new((B, S, 2), torch.float32),
                 token_of_slot=self._new((B, E, C), torch.int32))
        dgate = self._new((B, S, 2), torch.float32)
        route = ops.switch_gate_into if node.target is models.switch_gating else ops.top2_gate_into
        self.fwd.append(lambda: (ops.gemm(x.t, wg.t, logits, B * S, E, d), route(logits, C, r)))
        v = Val("gating", None, x=x, E=E, C=C, r=r, dgate=dgate, dgate_used=False, logits=logits)

        def emit():
            if not v.meta["dgate_used"]:
                return
            dlogits = self._new((B, S, E), torch.float32)
            dl = self._new((B, S, E)) if self.cdt != torch.float32 else dlogits
            gw, accw = self._param_grad_slot(wg)
            gx, accx = self._grad_slot(x) if x.needs_grad else (None, False)

            def backward():
                ops.top2_gate_bwd(r, dgate, dlogits)
                if dl is not dlogits:
                    ops.cast(dlogits, dl)
                ops.gemm(x.t, dl, gw, d, E, B * S, transA=True, accumulate=accw)
                if gx is not None:
                    ops.gemm(dl, wg.t, gx, B * S, d, E, transB=True, accumulate=accx)
            self.bwd.append(backward)
        self._tape.append(emit)
        return v

    def _einsum(self, node):
        code, a, b = node.args[0], self._val(node.args[1]), self._val(node.args[2])
        if code == "bsd,bsec->becd":
            return self._moe_dispatch(node, a, b)
        if code == "edh,becd->bech":
            return self._expert_gemm(node, a, b, first=True)
        if code == "ehd,bech->becd":
            return self._expert_gemm(node, a, b, first=False)
        if code == "becd,bsec->bsd":
            return self._moe_combine(node, a, b)
        self._unsupported(node, f"einsum code {code!r} has no handler")

    def _moe_dispatch(self, node, x: Val, route: Val):
        if route.kind != "routing" or route.meta["which"] != "dispatch" or x.t is None:
            self._unsupported(node, "expects (tokens, dispatch tensor of top_2_gating)")
        gv = route.meta["gating"]
        r, E, C = gv.meta["r"], gv.meta["E"], gv.meta["C"]
        e_lo, E_loc, c_lo, C_loc = route.meta["e_lo"], route.meta["E_loc"], route.meta["c_lo"], route.meta["C_loc"]
        s_lo, S_loc = route.meta["s_lo"], route.meta["S_loc"]
        B, S, d = x.t.shape
        if S != S_loc:
            self._unsupported(node, f"tokens of {S} positions against a dispatch tensor of {S_loc}")
        out = Val("expert", self._new((E_loc, B, C_loc, d)), shape=(B, E_loc, C_loc, d), needs_grad=True)
        self.fwd.append(lambda: ops.moe_dispatch(x.t, r, out.t, E, C, e_lo, E_loc, c_lo, C_loc, s_lo))

        def emit():
            if out.grad is None or not x.needs_grad:
                return
            gx, acc = self._grad_slot(x)
            self.bwd.append(lambda: ops.moe_dispatch_bwd(out.grad, r, gx, C, e_lo, E_loc, acc, c_lo, C_loc, s_lo))
        self._tape.append(emit)
        return out

    def _expert_gemm(self, node, w: Val, x: Val, first: bool):
        if w.kind != "param" or x.kind != "expert":
            self._unsupported(node, "expects (expert weights, expert-major activations)")
        E_loc, K, N = w.t.shape
        El, B, C, Kx = x.t.shape
        if El != E_loc or Kx != K:
            self._unsupported(node, "expert weight / activation shapes do not match")
        if K % self.epv or N % self.epv:
            self._unsupported(node, f"expert weight [{K}, {N}]: both extents must be multiples of {self.epv} "
                                    f"(rows of 16-byte vectors); pick shard widths accordingly")
        M = B * C
        fuse = self._wants_fused_relu(node)
        out = Val("expert", self._new((E_loc, B, C, N)), shape=(B, E_loc, C, N), needs_grad=True)
        if fuse:
            out.meta["fused_act"] = "relu"
        self.fwd.append(lambda: ops.gemm(x.t, w.t, out.t, M, N, K, batch1=E_loc, strideA=(M * K, 0), strideB=(K * N, 0),
                                         strideC=(M * N, 0), act="relu" if fuse else None))

        def emit():
            if out.grad is None:
                return
            if fuse:
                self._relu_backward_through(out)
            dy = out.grad
            gw, accw = self._param_grad_slot(w)
            self.bwd.append(lambda: ops.gemm(x.t, dy, gw, K, N, M, transA=True, lda=K, ldb=N, batch1=E_loc,
                                             strideA=(M * K, 0), strideB=(M * N, 0), strideC=(K * N, 0),
                                             accumulate=accw))
            if x.needs_grad:
                gx, accx = self._grad_slot(x)
                # the first expert GEMM applied relu itself and this one is its only reader: the data gradient
                # leaves the GEMM masked (every expert's mask lies at its output's offset)
                mask = None
                if (self.relu_mask_in_dgrad and x.meta.get("fused_act") == "relu" and not accx and self._only_reader(node, x, arg=2)
                        and not x.meta.get("relu_bwd_done")):
                    mask = x.t
                    x.meta["relu_bwd_done"] = True
                self.bwd.append(lambda: ops.gemm(dy, w.t, gx, M, K, N, transB=True, batch1=E_loc, strideA=(M * N, 0),
                                                 strideB=(K * N, 0), strideC=(M * K, 0), accumulate=accx, relu_mask=mask))
        self._tape.append(emit)
        return out

    def _moe_combine(self, node, eo: Val, route: Val):
        if route.kind != "routing" or route.meta["which"] != "combine" or eo.kind != "expert":
            self._unsupported(node, "expects (expert outputs, combine tensor of top_2_gating)")
        gv = route.meta["gating"]
        r, E, C = gv.meta["r"], gv.meta["E"], gv.meta["C"]
        e_lo, E_loc, c_lo, C_loc = route.meta["e_lo"], route.meta["E_loc"], route.meta["c_lo"], route.meta["C_loc"]
        El, B, Cl, d = eo.t.shape
        if (El, Cl) != (E_loc, C_loc):
            self._unsupported(node, f"expert outputs [{El} experts, {Cl} slots] do not match the combine tensor's "
                                    f"window [{E_loc}, {C_loc}]")
        s_lo, S_loc = route.meta["s_lo"], route.meta["S_loc"]       # the output covers the combine tensor's positions
        out = Val("tensor", self._new((B, S_loc, d)), needs_grad=True)
        self.fwd.append(lambda: ops.moe_combine(eo.t, r, out.t, C, e_lo, E_loc, c_lo, C_loc, s_lo))

        def emit():
            if out.grad is None:
                return
            if eo.grad is not None:
                self._unsupported(node, "expert outputs feed one combine only")
            eo.grad = self._new(eo.t.shape)
            gv.meta["dgate_used"] = True
            g, dgate = eo.grad, gv.meta["dgate"]
            self.bwd.append(lambda: ops.moe_combine_bwd(out.grad, eo.t, r, g, dgate, E, C, e_lo, E_loc, c_lo, C_loc, s_lo))
        self._tape.append(emit)
        return out

    # ------------------------------------------------------------------ running
    def load_inputs(self, *args):
        for rec, a in zip(self.inputs, args):
            if rec["buf"] is None:
                continue
            src = a if rec["offset"] is None else a.narrow(rec.get("dim", 0), rec["offset"], rec["length"])
            rec["buf"].copy_(src, non_blocking=True)

    def refresh_shadow(self):
        if self.shadow is not None:
            ops.cast(self.master, self.shadow)
        self._shadow_stale = False

    def forward(self, *args) -> torch.Tensor:
        if args:
            self.load_inputs(*args)
        if self._shadow_stale:
            self.refresh_shadow()
        self._run_phase("fwd", self.fwd)
        return self.loss[0]

    def _run_phase(self, name: str, closures):
        if not self.launch_lists or torch.cuda.is_current_stream_capturing():
            for f in closures:
                f()
            return
        key = (name, torch.cuda.current_stream().cuda_stream)
        calls = self._lists.get(key)
        if calls is not None:
            ops._lib.replay(calls)
            return
        ops._lib.start_recording()
        try:
            for f in closures:
                f()
        except BaseException:
            ops._lib.stop_recording()
            raise
        self._lists[key] = ops._lib.stop_recording()

    def backward(self):
        self._run_phase("bwd", [self._backward_launches])

    def _backward_launches(self):
        if self.n_vector_region:
            ops.fill_zero(self.flat_grad[:self.n_vector_region])
        if self.n_gathered_vector_region:
            ops.fill_zero(self.gathered_grad[:self.n_gathered_vector_region])
        for f in self.bwd:
            f()
        self._join_side()
        self._reduce_replicated_grads()

    def _reduce_replicated_grads(self):
        for f in self._param_reduce:
            f()

    # ------------------------------------------------------------------ optimizer (worker.py:47, 74-76)
    def configure_optimizer(self, kind: str = "adam", lr: float = 5e-4, betas=(0.9, 0.999), eps: float = 1e-8,
                            clip_grad_norm: Optional[float] = None):
        if kind not in ("adam", "sgd"):
            raise ValueError("optimizer must be 'adam' or 'sgd'")
        self._opt = dict(kind=kind, lr=lr, betas=betas, eps=eps, clip=clip_grad_norm)
        self._lists = {k: v for k, v in self._lists.items() if k[0] != "step"}
        if kind == "adam":
            self.exp_avg = torch.zeros_like(self.master)
            self.exp_avg_sq = torch.zeros_like(self.master)
            self._adam_state = torch.zeros(4, dtype=torch.float32, device=self.dev)   # step, 1-b1^t, 1-b2^t
        if clip_grad_norm is not None:
            self._sumsq = torch.zeros(1, dtype=torch.float32, device=self.dev)
            self._sumsq_ws = torch.empty(max(1, ops.sumsq_workspace_elems(self.flat_grad.numel())), dtype=torch.float32,
                                         device=self.dev)
            self._coef = torch.ones(1, dtype=torch.float32, device=self.dev)
        self._step_count = 0
        self._lists = {k: v for k, v in self._lists.items() if k[0] != "bwd_step"}
        # a global gradient norm needs every gradient, and the gradients of replicated parameters are only final
        # after their reduction at the end of backward: the update then stays one launch after backward
        self._opt_chunks = None
        if self.overlap_optimizer and clip_grad_norm is None and not self._param_reduce and self.n_flat > 0:
            self._opt_chunks = self._build_optimizer_chunks()

    def _build_optimizer_chunks(self):
        """Contiguous stretches of the flat buffers, about 1/24 of it each, with the number of backward launches
        after which the stretch can be updated.  The flat order follows the program (vectors, then matrices in
        the order of first use), so neighbours become final at about the same time."""
        recs = sorted(self.params.items(), key=lambda kv: kv[1]["offset"])
        target = max(self.n_flat // 24, self.optimizer_chunk_min)
        chunks, cur = [], None
        for name, rec in recs:
            ready = self._grad_final_idx.get(name, 0)             # never touched by backward: ready at once
            if cur is None or cur["size"] >= target:
                cur = dict(start=rec["offset"], size=0, ready=0, event=torch.cuda.Event())
                chunks.append(cur)
            cur["size"] = rec["offset"] + _round_up(rec["numel"], 64) - cur["start"]
            cur["ready"] = max(cur["ready"], ready)
        by_ready: Dict[int, list] = {}
        for c in chunks:
            by_ready.setdefault(c["ready"], []).append(c)
        return by_ready

    def step(self):
        if self._opt is None:
            raise RuntimeError("configure_optimizer() first")
        self._step_count += 1
        self._run_phase("step", [self._step_launches])

    def _step_launches(self):
        o = self._opt
        coef = None
        if o["clip"] is not None:
            ops.sumsq(self.flat_grad, self._sumsq, self._sumsq_ws)
            ops.clip_coef(self._sumsq, o["clip"], self._coef)
            coef = self._coef
        if o["kind"] == "sgd":
            ops.sgd_step(self.master, self.flat_grad, self.shadow, o["lr"], coef)
        else:
            ops.adam_step_dev(self.master, self.flat_grad, self.exp_avg, self.exp_avg_sq, self.shadow, o["lr"],
                              o["betas"][0], o["betas"][1], o["eps"], self._adam_state, coef)

    def train_step(self, *args) -> torch.Tensor:
        loss = self.forward(*args)
        self._backward_and_step()
        return loss

    def _backward_and_step(self):
        if self._opt is None:
            raise RuntimeError("configure_optimizer() first")
        if self._opt_chunks is None:
            self.backward()
            self.step()
            return
        self._step_count += 1
        self._run_phase("bwd_step", [self._backward_step_launches])

    def _backward_step_launches(self):
        """Backward with the optimizer folded in: every stretch of the parameters is updated on the optimizer
        stream once the launches that read it or write its gradients are enqueued on the main stream."""
        o = self._opt
        if self.n_vector_region:
            ops.fill_zero(self.flat_grad[:self.n_vector_region])
        if self.n_gathered_vector_region:
            ops.fill_zero(self.gathered_grad[:self.n_gathered_vector_region])
        if o["kind"] == "adam":
            ops.adam_advance(self._adam_state, o["betas"][0], o["betas"][1])
        n = len(self.bwd)
        for i in range(n + 1):
            for c in self._opt_chunks.get(i, ()):
                self._update_chunk(c)
            if i < n:
                self.bwd[i]()
        join, side = self._opt_join, self._opt_stream
        ops._lib.host_call(lambda: (join.record(side), torch.cuda.current_stream().wait_event(join)))

    def _update_chunk(self, c):
        o, side, ev = self._opt, self._opt_stream, c["event"]
        ops._lib.host_call(lambda: (ev.record(torch.cuda.current_stream()), side.wait_event(ev)))
        a, b = c["start"], c["start"] + c["size"]
        shadow = self.shadow[a:b] if self.shadow is not None else None
        with torch.cuda.stream(side):
            if o["kind"] == "sgd":
                ops.sgd_step(self.master[a:b], self.flat_grad[a:b], shadow, o["lr"], None)
            else:
                ops.adam_apply_dev(self.master[a:b], self.flat_grad[a:b], self.exp_avg[a:b], self.exp_avg_sq[a:b], shadow,
                                   o["lr"], o["betas"][0], o["betas"][1], o["eps"], self._adam_state, None)

    def capture_train_step(self):
        """Capture forward + backward + optimizer step (on the inputs loaded last) into a HIP graph and return a
        ``replay()`` callable.  Everything a step launches is a kernel on static buffers (no memset nodes, no
        allocation, Adam's step count lives on the device), so replays equal eager steps."""
        if self._opt is None:
            raise RuntimeError("configure_optimizer() first")
        if self._send_hooks:
            raise RuntimeError("the wire asked to be called after every outgoing message (Wire.send returned callables): "
                               "host calls are not part of a captured graph, so such a step cannot be replayed from one")
        if self._shadow_stale:
            self.refresh_shadow()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                self.forward()
                self._backward_and_step()
        torch.cuda.synchronize()
        self._graph = graph

        def replay() -> torch.Tensor:
            graph.replay()
            return self.loss[0]
        return replay

    def autotune_gemms(self, verbose: bool = False):
        """Run one forward + backward with the loaded inputs while recording every GEMM call, then time the
        legal tile configurations / K splits of each distinct problem signature on the recorded operands and
        pin the winners in the library's plan table (process-wide; other signatures keep the cost model).  Returns one
        row per signature: (signature, configuration, K splits, microseconds of one cold launch, launches per step,
        problems per step).  Buffers that the timed launches overwrite or accumulate into are activations and gradients, which the
        next step rewrites before reading; parameters and optimizer state are not touched."""
        if any(rec["buf"] is None for rec in self.inputs):
            raise RuntimeError("load_inputs() first")
        ops.record_gemms(True)
        try:
            self.forward()
            self.backward()
        finally:
            log = ops.record_gemms(False)
        torch.cuda.synchronize()
        flush = torch.zeros(512 << 20, dtype=torch.int8, device=self.dev)
        def signature(a):
            return (a.M, a.N, a.K, a.batch1 * a.batch2, a.transA, a.transB, a.in_dtype, a.out_dtype,
                    bool(a.A_segments), bool(a.B_segments or a.B_segments_list), bool(a.C_segments), a.a_relu, a.b_relu)
        calls: Dict[tuple, list] = {}
        for a, keep in log:                              # launches and problems (a launch over pointer lists holds several)
            c = calls.setdefault(signature(a), [0, 0])
            c[0] += 1
            c[1] += int(a.batch1 * a.batch2) if a.A_list else 1
        seen, report = set(), []
        for a, keep in log:
            key = signature(a)
            if key in seen:
                continue
            seen.add(key)
            cfg, splits, us = ops.autotune_gemm(a, flush)
            report.append((key, cfg, splits, us, calls[key][0], calls[key][1]))
            if verbose:
                print(f"gemm M{a.M} N{a.N} K{a.K} batch{key[3]} tA{a.transA} tB{a.transB}: config {cfg}, "
                      f"{splits} split(s), {us:.1f} us", flush=True)
        del flush
        torch.cuda.synchronize()
        return report

    def mark_params_dirty(self):
        """Call after parameters were changed from outside (e.g. by a torch.optim optimizer)."""
        self._shadow_stale = True


def compile_program(gm: torch.fx.GraphModule, example_inputs, dtype: str = "fp32", wire: Optional[Wire] = None,
                    rank: int = 0, world_size: int = 1, device: str = "cuda:0", **kw) -> ShardExecutor:
    """Compile the emitted program for the global-batch shapes of ``example_inputs`` (tensors or shapes)."""
    return ShardExecutor(gm, example_inputs, dtype=dtype, wire=wire, rank=rank, world_size=world_size, device=device,
                         **kw)


def _finish_param_reduce(self: ShardExecutor):
    """collectives.replicate backward (collectives.py:176-180): sum the replicated parameters'
    gradients with what the peers send, in rank order, in place."""
    for node in self.gm.graph.nodes:
        if node.op == "call_function" and node.target is collectives.replicate:
            v = self.env[node]
            if v.kind != "param" or not v.meta.get("grad_written"):
                continue
            g = v.meta["grad"]
            peers = self._peers(node.name, "bwd", self.rank_hint, self.world_hint, g.shape, True, torch.float32)
            contribs = [g if s == self.rank_hint else peers.get(s) for s in range(self.world_hint)]
            contribs = [c for c in contribs if c is not None]
            if len(contribs) > 1:
                flat = [c.reshape(1, -1) for c in contribs]
                n = g.numel()
                self._param_reduce.append(lambda flat=flat, n=n, g=g: ops.ragged_reduce(flat, 1, 0, n, g.view(1, -1)))


ShardExecutor._finish_param_reduce = _finish_param_reduce
