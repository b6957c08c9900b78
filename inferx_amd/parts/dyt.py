"""Dynamic Tanh norm: y = tanh(alpha * v) * weight + bias with v = h + delta, element by element (no mean, no
variance, no eps), fused with the residual add that precedes it.

The kernel also applies, on its way, a gain per channel on the delta (`ScaledDelta`) and a token shift of the
normalised rows (`forward_shifted`); everything in float32, rounded once to the run's type.
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import LazyDelta, Norm, ParamSpec, ScaledDelta, register_part


class DynamicTanh(Norm):
    graph_safe = True
    reads_stream_elsewhere = True

    def __init__(self, width: int, bias: bool = True):
        self.width, self.has_bias = int(width), bool(bias)
        self.weight = self.bias = None
        self.alpha = 1.0

    def param_specs(self) -> List[ParamSpec]:
        specs = [ParamSpec("weight", (self.width,), std=0.1, mean=1.0), ParamSpec("alpha", (), std=0.1, mean=0.6)]
        if self.has_bias:
            specs.append(ParamSpec("bias", (self.width,), std=0.1))
        return specs

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].to(torch.float32).contiguous()
        self.bias = tensors["bias"].to(torch.float32).contiguous() if self.has_bias else None
        self.alpha = float(tensors["alpha"].to(torch.float32).item())  # a constant of the kernel's launch

    @staticmethod
    def _operands(ctx, delta):
        """(tensor or None, gain or None) of whatever the delta is."""
        if isinstance(delta, ScaledDelta):
            return delta.tensor, delta.gain
        if isinstance(delta, LazyDelta):
            return delta.materialize(ctx), None
        return delta, None

    def forward(self, ctx, h, delta=None, rows=None, h_in=None):
        """h [T, width] float32 gets h + delta (unless `rows` picks rows out); returns the normalised rows in the
        run's type.  With `h_in` the stream is read from there and the sum written to h."""
        n = h.shape[0] if rows is None else rows.numel()
        out = ctx.rt.empty((n, self.width))
        tensor, gain = self._operands(ctx, delta)
        if h_in is None:
            ops.add_dyt(h, tensor, gain, self.weight, self.bias, self.alpha, out, rows)
        else:
            ops.add_dyt(h_in, tensor, gain, self.weight, self.bias, self.alpha, out, rows, h_out=h)
        return out

    def forward_shifted(self, ctx, h, delta, shift, cache):
        out = ctx.rt.empty((h.shape[0], self.width))
        tensor, gain = self._operands(ctx, delta)
        moved = torch.empty_like(h)
        ops.add_dyt(h, tensor, gain, self.weight, self.bias, self.alpha, out, None, h_out=moved,
                    shift=shift.operands(ctx, cache))
        return out, moved


register_part("norm", "dynamic_tanh", DynamicTanh)
