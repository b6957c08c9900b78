"""Causal attention over the paged cache whose heads talk to each other, grouped-query, without positions.

    q|k|v|gate = x . [Wq; Wk; Wv; Wg]^T                      one product, rows of the four weights stacked
    q, k       = RMS norm over the WHOLE projection (all heads of a token at once), plain weights
    v          = (1 - lambda) v + lambda v_source            v_source: the values that the model's first
                                                             value-mixing layer made for the same token
    s_h        = sum_g talk[h, g] (q_g . k_c(g)) * scale     scores of all heads mixed before the softmax
    p_h        = exp(s_h) / (exp(sink_h) + sum_j exp(s_h[j]))  a learned sink per head: no key, no value
    out_h      = sigmoid(gate_h) * sum_j p_h[j] v_c(h)[j]
    y          = concat(out) . Wo^T

Each of these is an option of the part (`qk_norm`, `value_mix`, `head_mixing`, `sink`, `gate`), keys and values
may differ in size (`head_dim`, `value_dim`), and the scale is a parameter.  What is cached is the normalised key
and the blended value.  Scores, mixing, softmax, norms are float32 in every run; in a bfloat16 run the products
take bfloat16 operands (matrix cores where the sizes allow: heads of a multiple of 16 numbers, pages of a multiple
of 16 tokens), else the plain kernel.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .attention import QUERY_TILE, plan_tiles
from .base import CacheNeed, Mixer, ParamSpec, register_part
from .dense_mlp import stack_rows

VALUE_MIX = ("none", "source", "mix")


class TalkingAttention(Mixer):
    graph_safe = True  # every launch reads the step's device arrays only

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: Optional[int] = None,
                 scale: Optional[float] = None, window: int = 0, qk_norm: bool = True, qk_norm_eps: float = 1e-6,
                 head_mixing: bool = True, sink: bool = True, gate: bool = True, value_mix: str = "none",
                 value_mix_group: str = "values", init_std: float = 0.02):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if value_mix not in VALUE_MIX:
            raise ValueError(f"value_mix {value_mix!r} is not one of {VALUE_MIX}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim) if value_dim is not None else self.head_dim
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window = int(window)
        self.qk_norm, self.qk_norm_eps = bool(qk_norm), float(qk_norm_eps)
        self.head_mixing, self.has_sink, self.has_gate = bool(head_mixing), bool(sink), bool(gate)
        self.value_mix, self.value_mix_group = value_mix, str(value_mix_group)
        self.init_std = float(init_std)
        self.w_in = self.w_out = self.q_norm = self.k_norm = self.talk = self.sink = None
        self.blend = 0.0

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def k_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_dim(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def out_dim(self) -> int:
        return self.num_heads * self.value_dim

    def cache_need(self) -> CacheNeed:
        return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, self.window, self.value_dim)

    def param_specs(self) -> List[ParamSpec]:
        W, s, H = self.hidden_size, self.init_std, self.num_heads
        specs = [ParamSpec("q.weight", (self.q_dim, W), std=s), ParamSpec("k.weight", (self.k_dim, W), std=s),
                 ParamSpec("v.weight", (self.v_dim, W), std=s), ParamSpec("o.weight", (W, self.out_dim), std=s)]
        if self.qk_norm:
            specs += [ParamSpec("q_norm.weight", (self.q_dim,), std=0.1, mean=1.0),
                      ParamSpec("k_norm.weight", (self.k_dim,), std=0.1, mean=1.0)]
        if self.value_mix != "none":  # (the source layer's own number is in the checkpoint and is not used)
            specs.append(ParamSpec("value_mix", (), std=0.1, mean=0.4))
        if self.head_mixing:
            specs.append(ParamSpec("talk", (H, H), std=0.5))
        if self.has_sink:
            specs.append(ParamSpec("sink", (H,), std=1.0))
        if self.has_gate:
            specs.append(ParamSpec("g.weight", (H, W), std=s))
        return specs

    def bind(self, tensors, rt) -> None:
        rows = [tensors["q.weight"], tensors["k.weight"], tensors["v.weight"]]
        if self.has_gate:
            rows.append(tensors["g.weight"])
        n = sum(t.shape[0] for t in rows)
        if n % 16:  # rows of zeros up to a multiple of sixteen: the product's rows then start at 32-byte steps
            rows.append(torch.zeros((16 - n % 16, self.hidden_size), dtype=rows[0].dtype, device=rows[0].device))
        self.w_in = stack_rows(rows)
        self.w_out = tensors["o.weight"].contiguous()
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()
        if self.qk_norm:
            self.q_norm, self.k_norm = f32("q_norm.weight"), f32("k_norm.weight")
        if self.head_mixing:
            self.talk = f32("talk")
        if self.has_sink:
            self.sink = f32("sink")
        if self.value_mix == "mix":
            self.blend = float(tensors["value_mix"].to(torch.float32).item())  # a constant of the launch

    def forward(self, ctx, x, cache):
        rt = ctx.rt
        T = x.shape[0]
        qkvg = rt.linear(x, self.w_in)
        q = rt.empty((T, self.num_heads, self.head_dim))
        # the values of the model's first value-mixing layer, for this step's tokens, go from layer to layer
        # in the step's memo
        key = ("value_mix", self.value_mix_group)
        v_first = v_out = None
        if self.value_mix == "source":
            v_out = ctx.memo[key] = rt.empty((T, self.v_dim))
        elif self.value_mix == "mix":
            v_first = ctx.memo.get(key)
            if v_first is None or v_first.shape != (T, self.v_dim):
                raise RuntimeError("a layer mixes its values with an earlier layer's, and no earlier layer of the same "
                                   "value size has left its values")
        writes = cache.writes
        ops.qk_norm_append(qkvg, self.q_norm, self.k_norm, self.qk_norm_eps, v_first, self.blend, v_out,
                           ctx.slots[cache.group] if writes else None, q, cache.k if writes else None,
                           cache.v if writes else None, self.num_heads, self.num_kv_heads, self.head_dim,
                           self.value_dim)
        out = rt.empty((T, self.num_heads, self.value_dim))
        gate = None
        if self.has_gate:
            at = self.q_dim + self.k_dim + self.v_dim
            gate = qkvg[:, at:at + self.num_heads]
        self.attend(ctx, q, cache, gate, out)
        return rt.linear(out.view(T, self.out_dim), self.w_out)

    def capture_plan(self, ctx, requests: int, longest: int) -> None:
        """The query tiles of a step of one token per request never change: tile i = request i, row i, one query
        (the plan that `plan_tiles` would make from the host's arrays)."""
        key = ("attention_tiles_host", QUERY_TILE)
        if key not in ctx.memo:
            tiles = torch.tensor([list(range(requests)), list(range(requests)), [1] * requests], dtype=torch.int32,
                                 device=ctx.rt.device)
            ctx.memo[key] = (tiles, requests, longest)

    def attend(self, ctx, q, cache, gate, out) -> None:
        """bfloat16 with heads, values and pages in multiples of 16 and no window: the matrix-core kernel, a workgroup
        per tile of sixteen queries and slice of keys; else the plain one."""
        page_size = cache.k.shape[2]
        table = ctx.block_tables[cache.group]
        per_wave = 0
        if q.dtype == torch.bfloat16 and self.window == 0:
            per_wave = ops.attention_talk_mfma_heads_per_wave(self.num_heads, self.num_kv_heads, self.head_dim,
                                                              self.value_dim, page_size)
        if per_wave == 0:
            ops.attention_talk_plain(q, cache.k, cache.v, table, ctx.seq_of_token, ctx.positions, out, self.talk,
                                     self.sink, gate, self.scale, self.window)
            return
        tiles, n_tiles, longest = plan_tiles(ctx, QUERY_TILE)
        n_splits = key_slices(n_tiles, longest, ctx.one_token_each)
        work = None
        if n_splits > 1:
            work = ctx.rt.empty((q.shape[0] * self.num_heads * n_splits * (self.value_dim + 2),), torch.float32)
        ops.attention_talk_mfma(q, cache.k, cache.v, table, tiles, ctx.positions, out, n_splits, work, self.talk,
                                self.sink, gate, self.scale)


WORKGROUPS_WANTED = 512  # two per compute unit: the tiles of a causal triangle end at very different times
MIN_KEYS_PER_SLICE = 128  # (a step of one token per request: a few rounds of the kernel)
MIN_KEYS_PER_SLICE_OF_PORTIONS = 256


def key_slices(n_tiles: int, longest: int, one_token_each: bool) -> int:
    """Into how many slices the matrix-core kernel cuts each tile's keys (a workgroup each): enough for
    WORKGROUPS_WANTED workgroups, no slice shorter than a few rounds, a power of two, 64 at most.  Measured at 16
    heads of 128: a prompt of 2,048 tokens 322 / 186 / 130 / 152 us in 1 / 2 / 4 / 8 slices (the parts of more slices
    cost the second kernel more than they even out), eight requests of one token on 2,048 keys 304 / 50 / 23 / 31 us
    in 1 / 8 / 32 / 64."""
    least = MIN_KEYS_PER_SLICE if one_token_each else MIN_KEYS_PER_SLICE_OF_PORTIONS
    n = max(1, min(-(-WORKGROUPS_WANTED // max(1, n_tiles)), longest // least, 64))
    return 1 << (n.bit_length() - 1)


register_part("mixer", "talking_attention", TalkingAttention)
