"""Stand-ins for the wire half of the uneven collectives.

This package executes ONE device's share of the SPMD program; no data crosses
the device.  Every ``collectives.*`` call is therefore: local preparation
kernel -> wire -> local completion kernel, and the wire is one of the objects
below.  They hand out what the peers would have sent as static GPU tensors.

* ``SilentWire``     peers send nothing to reductions and zeros to gathers.
* ``SyntheticWire``  peers send seeded N(0, scale) data of the right shape
                     (generated on the CPU, uploaded once).
* ``ReplayWire``     peers send what a recorded run of all ranks sent
                     (``log[(tag, direction)][src][dst]`` CPU tensors).

With more than one GPU the wire would be RCCL point-to-point sends of the
exact (unpadded) extents; that transport is not part of this package.
"""
from __future__ import annotations

import zlib
from typing import Dict, Optional, Tuple

import torch


class Wire:
    """``recv(tag, direction, src, shape, dtype, device)`` returns the tensor that rank
    ``src`` sent to this rank at collective ``tag`` (``direction`` 'fwd' or 'bwd'), or
    None when that peer contributes nothing."""

    def recv(self, tag: str, direction: str, src: int, shape, dtype, device, reduction: bool = False,
             into: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """``into``: a contiguous static GPU tensor that the message is to be delivered into (zero-copy receive: the
        executor passes the rows of a concatenation that the piece belongs to); the wire returns it.  It has the
        message's ``shape``, or fewer rows along dim 0: then it takes the message's first rows (a shard that was padded
        to the longest length carries its payload there; a transport that sends exact extents delivers just those).
        The stand-ins below deliver once, when the program is compiled; a transport would post its receive into
        it every step."""
        raise NotImplementedError

    @staticmethod
    def _deliver(message: Optional[torch.Tensor], into: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        if into is None or message is None:
            return message
        rows_ok = into.dim() == message.dim() and into.dim() >= 1 and 0 < into.shape[0] <= message.shape[0]
        if not rows_ok or tuple(into.shape[1:]) != tuple(message.shape[1:]) or into.dtype != message.dtype or not into.is_contiguous():
            raise ValueError("recv(into=...): a contiguous tensor of the message's shape (or its first rows) and dtype expected")
        into.copy_(message[:into.shape[0]])
        return into

    def send(self, tag: str, direction: str, dst: int, buffer: torch.Tensor) -> None:
        """Called once, when the program is compiled, for every message this rank sends: ``buffer`` is the static
        GPU tensor that holds the message for rank ``dst`` after the local preparation kernels of collective
        ``tag`` have run in a step.  A transport would post its sends from these buffers.  May return a callable:
        the executor then calls it in every step right after those kernels are enqueued (the point at which the
        message is complete; later launches of the step may reuse the buffer), whether the step is launched call
        by call or replayed from its recorded launch list; a step with such callables cannot be captured into a
        HIP graph (``capture_train_step`` raises).  The stand-ins send nothing;
        ``ReplayWire`` snapshots the messages so that tests can compare them with the recorded run."""
        return None


class SilentWire(Wire):
    def __init__(self, gather_fill: float = 0.0):
        self.gather_fill = gather_fill
        self._cache: Dict[Tuple, torch.Tensor] = {}

    def recv(self, tag, direction, src, shape, dtype, device, reduction: bool = False, into=None):
        if reduction:
            return None
        key = (tuple(shape), dtype)
        if key not in self._cache:
            self._cache[key] = torch.full(tuple(shape), self.gather_fill, dtype=dtype, device=device)
        return self._deliver(self._cache[key], into)


class SyntheticWire(Wire):
    def __init__(self, seed: int = 0, scale: float = 1.0, grad_scale: float = 1e-3, reduce_params: bool = False,
                 share_shapes: bool = False):
        """``share_shapes``: messages of equal shape, direction and sender reuse one buffer (a benchmark with
        many identical layers then needs one set of peer buffers instead of one per layer)."""
        self.seed = int(seed)
        self.scale, self.grad_scale = scale, grad_scale
        self.reduce_params = reduce_params
        self.share_shapes = share_shapes
        self._cache: Dict[Tuple, torch.Tensor] = {}

    def recv(self, tag, direction, src, shape, dtype, device, reduction: bool = False, into=None):
        if tag.startswith("replicate") and not self.reduce_params:
            return None
        key = (direction, src, tuple(shape), dtype) if self.share_shapes else (tag, direction, src)
        if key not in self._cache:
            s = self.scale if direction == "fwd" else self.grad_scale
            # one stream of random numbers per message, so that the content does not depend on the order in which
            # the executor asks for its buffers
            gen = torch.Generator().manual_seed((self.seed * 1000003 + zlib.crc32(repr(key).encode())) % (1 << 63))
            t = torch.randn(tuple(shape), generator=gen, dtype=torch.float32) * s
            self._cache[key] = t.to(dtype).to(device)
        return self._deliver(self._cache[key], into)


class ReplayWire(Wire):
    def __init__(self, log: dict, rank: int):
        self.log, self.rank = log, rank
        self._cache: Dict[Tuple, torch.Tensor] = {}
        self.sent: Dict[Tuple, torch.Tensor] = {}       # (tag, direction, dst) -> copy of the message this rank sent last

    def send(self, tag, direction, dst, buffer):
        def snapshot():
            self.sent[(tag, direction, dst)] = buffer.detach().clone()
        return snapshot

    def recv(self, tag, direction, src, shape, dtype, device, reduction: bool = False, into=None):
        key = (tag, direction, src)
        if key not in self._cache:
            if (tag, direction) not in self.log:
                raise KeyError(f"no recorded message for collective {tag!r} ({direction})")
            t = self.log[(tag, direction)][src][self.rank]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"recorded message for {tag!r} ({direction}) from rank {src} has shape "
                                 f"{tuple(t.shape)}, the program expects {tuple(shape)}")
            self._cache[key] = t.detach().to(dtype).contiguous().to(device)
        return self._deliver(self._cache[key], into)
