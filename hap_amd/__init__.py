"""hap_amd -- MI355X-native executor for one device's shard of a HAP SPMD program.

Public surface (mirrors what /root/reference exposes for this path):

* ``sharding_round(n, ratios)``          -- hap.sharding_round (hap.rs:211-218)
* ``collectives``                         -- collectives.py's six functions
* ``models``                              -- model zoo + fx leaf ops of models.py
* ``build_program(model, plan, B)``       -- the per-device ``torch.fx`` program
                                             (what ``hap.main`` returns, hap.rs:81-188)
* ``compile(gm, example_inputs, ...)``    -- ``ShardModule``: call it like the
  reference's ``dmodel`` (worker.py:59-76): ``loss = m(x, y); loss.backward();
  optimizer.step()``, or drive ``m.executor`` directly (``train_step``).
* ``planner.stat(gm, {"input_shape": ...})`` -- hap.stat (hap.rs:190-209), plus
  the device_flops calibration and the cost of the fixed plan forms.
"""
from __future__ import annotations

import torch

from . import collectives, models, planner  # noqa: F401
from .sharding import ShardingPlan, shard_inplace, sharding_lengths, sharding_round  # noqa: F401
from .program import build_program  # noqa: F401
from .executor import ShardExecutor, compile_program  # noqa: F401
from .wire import ReplayWire, SilentWire, SyntheticWire, Wire  # noqa: F401


class _RunProgram(torch.autograd.Function):
    @staticmethod
    def forward(ctx, module, x, y, *params):
        ctx.module = module
        loss = module.executor.forward(x, y)
        return loss.clone()

    @staticmethod
    def backward(ctx, grad_output):
        ex = ctx.module.executor
        ex.backward()
        # gradients live in the executor's flat buffer, which the parameters' .grad already view
        if ctx.module.scale_by_grad_output:
            ex.flat_grad.mul_(grad_output)
        return (None, None, None) + tuple(None for _ in ctx.module._plist)


class ShardModule(torch.nn.Module):
    """``GraphModule``-like facade over a compiled shard program."""

    def __init__(self, gm: torch.fx.GraphModule, example_inputs, scale_by_grad_output: bool = False, **kw):
        super().__init__()
        self.gm = gm
        self.executor = ShardExecutor(gm, example_inputs, **kw)
        self._plist = [rec["param"] for rec in self.executor.params.values()]
        self.scale_by_grad_output = scale_by_grad_output

    def parameters(self, recurse: bool = True):
        return iter(self._plist)

    def forward(self, x, y):
        # parameters may have been stepped by an external optimizer since the last call
        self.executor.mark_params_dirty()
        anchor = self._plist[0] if self._plist else None
        out = _RunProgram.apply(self, x, y, *self._plist)
        if anchor is not None and not out.requires_grad:
            out.requires_grad_(True)
        return out

    def zero_grad(self, set_to_none: bool = False):
        # the first contribution to every gradient overwrites it, so there is nothing to clear
        for rec in self.executor.params.values():
            rec["param"].grad = rec["grad"]


def compile(gm: torch.fx.GraphModule, example_inputs, **kw) -> ShardModule:
    return ShardModule(gm, example_inputs, **kw)
