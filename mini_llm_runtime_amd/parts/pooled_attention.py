"""Windowed attention that also sees pooled blocks of what left the window."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ..cache.spec import CompositeSpec, PagedKVSpec
from ..kernels.limits import check_attention_sizes
from .base import Mixer, Part, PositionEncoding
from .context import MixerPlan, PlanInput, StepContext, site_member
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "pooled_window_attention")
class PooledWindowAttention(Mixer):
    """Grouped-query softmax attention over a sliding window and, before the window, one pooled key and
    value per block of tokens.

    With h the input: q = Wq h + bq, k = Wk h + bk, v = Wv h + bv (biases if `qkv_bias`).
    `qk_norm`: q and k are each divided by the root mean square of their WHOLE projection (all heads at
    once, eps inside the root) and multiplied by a weight of that size.  Then the position encoding (q
    and k), then q of head i times `temperature[i]` (a learned number per head, if `temperature`).

    A query at position p sees the tokens j with 0 <= p - j < window and, if `pool` = P is given, block b
    (positions bP .. bP + P - 1) once bP + P - 1 <= p - window, through the means of the block's cached keys
    and of its values; tokens that have left the window and whose block is not complete yet are not seen.
    Tokens and blocks share one softmax, score = q . k * scale, whose denominator also holds exp(sink_i)
    (a learned number per head, if `sink`).  `head_gate`: head i's output times sigmoid(Wg h)_i, one number
    per head.  Output: Wo on the heads side by side.

    Cache: the window's keys and values in pages that are given back behind the window, and the pooled
    entries in pages of their own kind (one entry per P tokens, kept for good), written when a block's
    last token comes in, from the pages of the block's tokens: so those stay for max(window, P)
    positions.  One product makes q, k, v and the gate logits in 32-bit sums; norm, rotation, scaling and
    gates are one 32-bit kernel that rounds once.
    """

    replayable = True
    open_output = True
    open_input = True  # `activations(projected=)` takes the input product's sums from whoever made them

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        window: int,
        scale: float,
        value_dim: Optional[int] = None,
        pool: Optional[int] = None,
        position: Optional[PartSpec] = None,
        qkv_bias: bool = True,
        qk_norm: bool = False,
        norm_eps: float = 1e-6,
        temperature: bool = False,
        sink: bool = False,
        head_gate: bool = False,
    ) -> None:
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError("num_heads must be a positive multiple of num_kv_heads")
        if head_dim <= 0 or window <= 0 or (pool is not None and pool <= 0) or not scale > 0:
            raise ValueError("head_dim, window, pool and scale must be > 0")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        if self.value_dim <= 0:
            raise ValueError("value_dim must be > 0")
        # the one head size that kernels and pages see
        self.kernel_dim = -(-max(self.head_dim, self.value_dim) // 16) * 16
        check_attention_sizes(num_heads, num_kv_heads, self.kernel_dim)
        self.window = int(window)
        self.pool = None if pool is None else int(pool)
        self.scale = float(scale)
        self.qkv_bias = bool(qkv_bias)
        self.qk_norm = bool(qk_norm)
        self.norm_eps = float(norm_eps)
        self.temperature = bool(temperature)
        self.sink = bool(sink)
        self.head_gate = bool(head_gate)
        self.position: Optional[PositionEncoding] = build_part("position", position) if position is not None else None
        self.in_weight: Optional[torch.Tensor] = None
        self.in_bias: Optional[torch.Tensor] = None
        self.q_norm_weight: Optional[torch.Tensor] = None
        self.k_norm_weight: Optional[torch.Tensor] = None
        self.head_scale: Optional[torch.Tensor] = None
        self.sinks: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def in_rows(self) -> int:
        return self.q_size + self.k_size + self.v_size + (self.num_heads if self.head_gate else 0)

    @property
    def out_width(self) -> int:
        return self.num_heads * self.value_dim

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {
            "in_weight": ParamSpec((self.in_rows, self.hidden_size)),
            "o_weight": ParamSpec((self.hidden_size, self.out_width)),
        }
        if self.qkv_bias:
            # biases of q, k and v; the gate logits have none (their rows of the product's bias are zeros)
            specs["in_bias"] = ParamSpec((self.q_size + self.k_size + self.v_size,), keep_stored_precision=True)
        if self.qk_norm:
            specs["q_norm_weight"] = ParamSpec((self.q_size,), init="one_plus_normal", keep_stored_precision=True)
            specs["k_norm_weight"] = ParamSpec((self.k_size,), init="one_plus_normal", keep_stored_precision=True)
        if self.temperature:
            specs["head_scale"] = ParamSpec((self.num_heads,), init="one_plus_normal", keep_stored_precision=True)
        if self.sink:
            specs["sinks"] = ParamSpec((self.num_heads,), keep_stored_precision=True)
        return specs

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        # numbers per head are used in 32-bit
        if self.head_scale is not None:
            self.head_scale = self.head_scale.to(torch.float32).contiguous()
        if self.sinks is not None:
            self.sinks = self.sinks.to(torch.float32).contiguous()
        biased = self.q_size + self.k_size + self.v_size
        order = self.position.half_split_order() if hasattr(self.position, "half_split_order") else None
        if order is not None and order != list(range(self.head_dim)):
            # the checkpoint pairs neighbouring dims: both projections list their dims the kernels' way
            rows = []
            for first, heads in ((0, self.num_heads), (self.q_size, self.num_kv_heads)):
                for head in range(heads):
                    rows += [first + head * self.head_dim + j for j in order]
            index = torch.tensor(rows + list(range(self.q_size + self.k_size, self.in_rows)), device=self.in_weight.device)
            self.in_weight = self.in_weight.index_select(0, index).contiguous()
            if self.in_bias is not None:
                self.in_bias = self.in_bias.index_select(0, index[:biased]).contiguous()
            if self.q_norm_weight is not None:
                self.q_norm_weight = self.q_norm_weight.index_select(0, index[: self.q_size]).contiguous()
                self.k_norm_weight = self.k_norm_weight.index_select(0, index[self.q_size : self.q_size + self.k_size] - self.q_size).contiguous()

        if self.in_bias is not None and self.in_rows > biased:
            self.in_bias = torch.cat([self.in_bias, self.in_bias.new_zeros(self.in_rows - biased)]).contiguous()

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> Any:
        # a block is pooled from its tokens' pages when its last token comes in: they stay that long
        keep = self.window if self.pool is None else max(self.window, self.pool)
        tokens = PagedKVSpec(self.num_kv_heads, self.kernel_dim, keep)
        if self.pool is None:
            return tokens
        return CompositeSpec({"tokens": tokens, "pooled": PagedKVSpec(self.num_kv_heads, self.kernel_dim, tokens_per_entry=self.pool)})

    def plan(self, ops, shape: PlanInput) -> Optional[MixerPlan]:
        make = getattr(ops, "attention_plan", None)
        return make(shape) if make is not None else None

    def activations(
        self, ctx: StepContext, h, site: Any, *, out: torch.Tensor, column: int, scale: float = 1.0, projected=None
    ) -> None:
        """`projected`: (float32 sums [T, ...], first column) of h times `in_weight` (+ `in_bias`), when the
        caller made them within a larger product."""
        ops = ctx.ops
        if self.pool is None:
            cache, pooled = ctx.kv(site), None
        else:
            cache, pooled = ctx.kv(site_member(site, "tokens")), ctx.kv(site_member(site, "pooled"))
        rotation = self.position.rotation(ctx) if self.position is not None else None
        if self.position is not None and rotation is None:
            raise RuntimeError("pooled_window_attention takes position encodings that are rotations of halves")
        first = 0
        if projected is None:
            projected = ops.linear(h, self.in_weight, self.in_bias, out_dtype=torch.float32)  # norm and rotation read 32-bit sums
        else:
            projected, first = projected
        q, gate = ops.qk_norm_rope_write(
            projected, self.q_norm_weight, self.k_norm_weight, self.norm_eps, self.head_scale, rotation,
            cache.slot_mapping, cache.key, cache.value,
            num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, dim=self.head_dim, value_dim=self.value_dim,
            head_dim=self.kernel_dim, block_size=cache.block_size, gated=self.head_gate,
            **({"projected_column": first} if first else {}),
        )
        cache.written()
        cache.reading()
        seen = None
        if pooled is not None:
            ops.pool_kv_write(
                cache.key, cache.value, cache.block_table, pooled.slot_mapping, pooled.key, pooled.value, ctx,
                num_kv_heads=self.num_kv_heads, head_dim=self.kernel_dim, block_size=cache.block_size, pool=self.pool,
            )
            pooled.written()
            pooled.reading()
            seen = (pooled.key, pooled.value, pooled.block_table, self.pool)
        attended = ops.paged_attention(
            q, cache.key, cache.value, cache.block_table, ctx,
            num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=self.kernel_dim,
            block_size=cache.block_size, scale=self.scale, window=self.window, sinks=self.sinks,
            plan=ctx.plan(getattr(ops, "ATTENTION_PLAN", None)),
            **({"pooled": seen} if seen is not None else {}),
        )
        ops.scale_heads(
            attended, gate, heads=self.num_heads, head_dim=self.kernel_dim, out_dim=self.value_dim, scale=scale,
            out=out, column=column,
        )

    def forward(self, ctx: StepContext, h: torch.Tensor, site: Any) -> torch.Tensor:
        out = torch.empty((h.shape[0], self.out_width), dtype=ctx.dtype, device=ctx.device)
        self.activations(ctx, h, site, out=out, column=0)
        return ctx.ops.linear(out, self.o_weight, None, for_stream=True)
