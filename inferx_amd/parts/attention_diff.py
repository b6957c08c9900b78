"""Differential attention over the paged cache: every head has two score maps over one set of values, and its
result is the first map's minus lambda times the second's.

    q|k|v   = x . [Wq; Wk; Wv]^T + bias           q: heads x [map 0, map 1] x dim, k: kv_heads x [map 0, map 1] x dim,
                                                  v: kv_heads x vdim
    q, k, v = short_conv(.)                       causal, per channel, continued from the request's last inputs
    q, k    = rotated (the position encoding's part of every map)
    a_m     = softmax_j(q_m . k_m[j] * scale) v[j]    over the keys the query sees: j <= i and
                                                      (i - j < window or j < keep_first); window 0: all
    lambda  = exp(lq1 . lk1) - exp(lq2 . lk2) + diff  one number for the layer
    o       = a_0 - lambda a_1;  o / rms(o) * (1 - diff)           rms over a head's vdim, no weight
    y       = concat(o) . Wo^T

The cache keeps the rotated keys of both maps (2 kv_heads "heads" of dim) and the values (kv_heads of vdim,
transposed within a page); with a window the pages that it has passed go back, except those of the kept first
tokens.  The short convolution's last inputs live in the request's state slot.  Scores, softmax, the difference
and the norm are float32 in every run.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from .. import ops
from ..config.spec import PartSpec
from .attention import MIN_KEYS_PER_SPLIT, QUERY_TILE, WAVES_WANTED, plan_tiles
from .base import CacheArray, CacheNeed, Mixer, ParamSpec, StateNeed, build_part, register_part
from .dense_mlp import stack_rows
from .short_conv import ShortConv


class DifferentialAttention(Mixer):
    graph_safe = True  # every launch reads the step's device arrays only

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 diff: float, conv_taps: int = 1, scale: Optional[float] = None, window: int = 0, keep_first: int = 0,
                 norm_eps: float = 1e-6, position: Optional[PartSpec] = None, init_std: float = 0.02):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if not 0 < head_dim <= 256 or not 0 < value_dim <= 256:
            raise ValueError(f"head_dim {head_dim} and value_dim {value_dim} must be between 1 and 256")
        if window < 0 or keep_first < 0:
            raise ValueError("window and keep_first must not be negative")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.diff, self.norm_eps, self.init_std = float(diff), float(norm_eps), float(init_std)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window, self.keep_first = int(window), int(keep_first) if window > 0 else 0
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None:
            dims = int(getattr(self.position, "rotary_dim", 0))
            if getattr(self.position, "begin", 0) != 0 or dims <= 0 or dims % 2 or dims > self.head_dim:
                raise ValueError(f"the position encoding must rotate the first {dims} elements of maps of "
                                 f"{self.head_dim}: an even number within the map, from its start")
        self.q_dim, self.k_dim = 2 * self.num_heads * self.head_dim, 2 * self.num_kv_heads * self.head_dim
        self.v_dim, self.o_dim = self.num_kv_heads * self.value_dim, self.num_heads * self.value_dim
        self.conv = ShortConv(self.q_dim, self.k_dim, self.v_dim, self.head_dim, self.value_dim, conv_taps)
        self.w_qkv = self.b_qkv = self.w_out = None
        self.lam = 0.0

    def cache_need(self) -> CacheNeed:
        return CacheNeed((CacheArray("k", 2 * self.num_kv_heads, self.head_dim),
                          CacheArray("v", self.num_kv_heads, self.value_dim, transposed=True)),
                         self.window, self.keep_first)

    def state_need(self) -> StateNeed:
        return StateNeed((max(1, self.conv.state_floats),), "float32")

    def subparts(self):
        return [self.position]

    def param_specs(self) -> List[ParamSpec]:
        W, s, D = self.hidden_size, self.init_std, self.head_dim
        return [ParamSpec("q.weight", (self.q_dim, W), std=s), ParamSpec("k.weight", (self.k_dim, W), std=s),
                ParamSpec("v.weight", (self.v_dim, W), std=s), ParamSpec("q.bias", (self.q_dim,), std=s),
                ParamSpec("k.bias", (self.k_dim,), std=s), ParamSpec("v.bias", (self.v_dim,), std=s),
                ParamSpec("lq1", (D,), std=0.1), ParamSpec("lk1", (D,), std=0.1), ParamSpec("lq2", (D,), std=0.1),
                ParamSpec("lk2", (D,), std=0.1), ParamSpec("o.weight", (W, self.o_dim), std=s)] + self.conv.param_specs()

    def bind(self, tensors, rt) -> None:
        self.w_qkv = stack_rows([tensors[f"{n}.weight"] for n in "qkv"])
        self.b_qkv = stack_rows([tensors[f"{n}.bias"] for n in "qkv"])
        self.w_out = tensors["o.weight"].contiguous()
        self.conv.bind(tensors, bias=self.b_qkv)
        dot = lambda a, b: float((tensors[a].double() * tensors[b].double()).sum().item())
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff
        if self.position is not None:
            self.position.bind({}, rt)

    def forward(self, ctx, x, cache):
        rt, T = ctx.rt, x.shape[0]
        table = self.position.prepare(ctx) if self.position is not None else None
        proj = rt.linear(x, self.w_qkv)
        q = rt.empty((T, self.num_heads, 2, self.head_dim))
        if cache.writes:
            self.conv.apply(ctx, proj, cache.state, q, cache.k, cache.v, slots=ctx.slots[cache.group], cos_sin=table)
        else:  # the keys and values are another execution's: only the queries are wanted
            self.conv.apply(ctx, proj, cache.state, q, rt.empty((T, self.k_dim)), rt.empty((T, self.v_dim)),
                            cos_sin=table)
        out = rt.empty((T, self.num_heads, self.value_dim))
        self.attend(ctx, q, cache, out)
        return rt.linear(out.view(T, self.o_dim), self.w_out)

    def capture_plan(self, ctx, requests: int, longest: int) -> None:
        """The query tiles of a step of one token per request never change (tile i = request i, row i, one query);
        the slices of the keys follow from `longest`.  (The same plan, under the same key, as plain attention's.)"""
        key = ("attention_tiles_host", QUERY_TILE)
        if key not in ctx.memo:
            tiles = torch.tensor([list(range(requests)), list(range(requests)), [1] * requests], dtype=torch.int32,
                                 device=ctx.rt.device)
            ctx.memo[key] = (tiles, requests, longest)

    def key_slices(self, units: int, longest: int) -> int:
        """Into how many slices each tile's keys are cut: enough wavefronts for the machine, no slice shorter than
        MIN_KEYS_PER_SPLIT, a power of two (few distinct values, few captured graphs), 64 at most."""
        span = min(longest, self.window + self.keep_first + QUERY_TILE + 32) if self.window > 0 else longest
        n = 1 if units >= WAVES_WANTED else max(1, min(WAVES_WANTED // max(1, units), -(-span // MIN_KEYS_PER_SPLIT), 64))
        return 1 << (n.bit_length() - 1)

    def attend(self, ctx, q, cache, out) -> None:
        """bfloat16 with heads and pages that the matrix-core kernel is built for: that kernel, in tiles of up to 16
        queries of a request, a (head, map) pair per wavefront (a step of one token per request: the query heads of
        a key/value head side by side); else the plain one."""
        page_size = cache.k.shape[2]
        if q.dtype == torch.bfloat16 and ops.attention_diff_mfma_fits(self.head_dim, self.value_dim, page_size):
            tiles, n_tiles, longest = plan_tiles(ctx, QUERY_TILE)
            group = self.num_heads // self.num_kv_heads
            grouped = ctx.one_token_each and 2 <= group <= 16
            n_splits = self.key_slices(n_tiles * 2 * (self.num_kv_heads if grouped else self.num_heads), longest)
            work = ctx.rt.empty((q.shape[0] * self.num_heads * 2 * n_splits * (self.value_dim + 2),), torch.float32)
            ops.attention_diff_mfma(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, out,
                                    n_splits, work, self.scale, self.window, self.keep_first, self.lam, self.norm_eps,
                                    1.0 - self.diff, grouped=grouped)
            return
        ops.attention_diff_plain(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.seq_of_token, ctx.positions,
                                 out, self.scale, self.window, self.keep_first, self.lam, self.norm_eps,
                                 1.0 - self.diff)


register_part("mixer", "differential_attention", DifferentialAttention)
