"""A short causal convolution over time on the channels of a mixer's q | k | v projection, as mixers use it between
the projection and whatever follows (an activation, a rotation, the cache):

    y[t, c] = sum_j w[c, j] * u[t - taps + 1 + j, c]        zeros before a sequence's start, no bias

The last taps - 1 inputs of every request are part of its state (float32), so that a request may be cut into
steps anywhere.  This is a helper that a mixer owns, not a part of its own: the mixer says how many floats of its
state block it needs (`state_floats`) and hands the view over with every call.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from .. import ops
from .base import ParamSpec
from .dense_mlp import stack_rows


class ShortConv:
    def __init__(self, q_channels: int, k_channels: int, v_channels: int, head_dim: int, value_dim: int, taps: int):
        if taps < 1 or taps > 64:
            raise ValueError(f"a short convolution of {taps} taps: between 1 and 64")
        self.sizes: Tuple[int, int, int, int, int] = (int(q_channels), int(k_channels), int(v_channels),
                                                      int(head_dim), int(value_dim))
        self.taps = int(taps)
        self.weight = self.weight_t = self.bias = self.bias_f32 = None

    @property
    def channels(self) -> int:
        return self.sizes[0] + self.sizes[1] + self.sizes[2]

    @property
    def state_floats(self) -> int:
        return (self.taps - 1) * self.channels

    def param_specs(self, names=("q", "k", "v"), std: float = 0.3) -> List[ParamSpec]:
        """One [channels, taps] tensor per run of channels, named `<name>.conv`."""
        return [ParamSpec(f"{n}.conv", (c, self.taps), std=std) for n, c in zip(names, self.sizes[:3])]

    def bind(self, tensors, names=("q", "k", "v"), bias=None) -> None:
        """`bias`: what is added to the inputs before the convolution (one number per channel), or None."""
        self.bias = bias
        self.bias_f32 = bias.to(torch.float32).contiguous() if bias is not None else None
        self.weight = stack_rows([tensors[f"{n}.conv"] for n in names])
        self.weight_t = self.weight.to(torch.float32).t().contiguous()  # [taps, channels], for the kernel's 16-byte form

    def apply(self, ctx, x, state, out_q, out_k, out_v, slots=None, cos_sin=None, silu: bool = False) -> None:
        """`state`: the float32 view [slots, >= state_floats] of the requests' last inputs (see `ops.short_conv`)."""
        rows = ops.StepRows(ctx.seq_of_token, ctx.q_start, ctx.state_slots)
        ops.short_conv(x, self.bias, self.weight, state, rows, self.sizes, out_q, out_k, out_v, slots=slots,
                       cos_sin=cos_sin, silu=silu, weight_t=self.weight_t, bias_f32=self.bias_f32)
