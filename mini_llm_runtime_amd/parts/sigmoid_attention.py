"""Attention without a softmax: every visible key weighs by a sigmoid of its own score."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.spec import PagedKVSpec
from ..kernels.limits import check_attention_sizes
from .base import Mixer, Part, PositionEncoding
from .context import MixerPlan, PlanInput, StepContext
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "sigmoid_attention")
class SigmoidAttention(Mixer):
    """Grouped-query causal attention over the paged cache in which the weight of key j for the query at
    position t >= j is

        a_tj = sigmoid((q_t . k_j) * scale + b_head),

    a learned number b per query head added to the score; the weights are not normalised over the keys, so
    a key's weight does not depend on the others.  With h the mixer's input:

        q = rot(Wq h + bq), k = rot(Wk h + bk), v = Wv h + bv   (biases if `qkv_bias`; rotation if `position`),
        then every head of q and k divided by its root mean square over head_dim and every head of v by its
        own over value_dim (eps inside the root, no weights), all in 32-bit;
        out = Wo [ sigmoid(Wg h)_head * sum_j a_tj v_j ]_head      (`output_gate`: one number per head).

    value_source: None, "first" or "mixed".  Layers that say "first" keep their normed values of the step's
    tokens for the layers that say "mixed", whose values become (1 - w) v + w v_first with w the parameter
    `value_mix` (the same token's values of the first such layer; the mixed values are what is cached).  All
    such layers have equal kv_heads * value_dim.

    One input product (rows q, k, v, gate; 32-bit sums), one kernel for rotation, norms, mixing, cache write
    and the gates' sigmoids, the attention kernels with `score_bias`, the gate multiplied into the heads
    while they move to their own width, the output product.  Kernels and pages know one head size D = the
    larger of head_dim and value_dim, rounded up to 16, zero beyond a head's own width.
    """

    replayable = True
    MEMO_KEY = "sigmoid_attention.first_values"

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        value_dim: int,
        scale: float,
        norm_eps: float,
        position: Optional[PartSpec] = None,
        qkv_bias: bool = True,
        output_gate: bool = True,
        value_source: Optional[str] = None,
    ) -> None:
        if min(hidden_size, num_heads, num_kv_heads, head_dim, value_dim) <= 0 or num_heads % num_kv_heads:
            raise ValueError("SigmoidAttention sizes must be > 0, num_heads a multiple of num_kv_heads")
        if not scale > 0:
            raise ValueError("scale must be > 0")
        if value_source not in (None, "first", "mixed"):
            raise ValueError("value_source is None, 'first' or 'mixed'")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.scale = float(scale)
        self.norm_eps = float(norm_eps)
        self.qkv_bias = bool(qkv_bias)
        self.output_gate = bool(output_gate)
        self.value_source = value_source
        self.kernel_dim = -(-max(self.head_dim, self.value_dim) // 16) * 16
        check_attention_sizes(num_heads, num_kv_heads, self.kernel_dim)
        self.position: Optional[PositionEncoding] = build_part("position", position) if position is not None else None
        if self.position is not None and getattr(self.position, "rotary_dim", 0) > self.head_dim:
            raise ValueError("the rotation covers more dimensions than a head has")
        self.in_weight: Optional[torch.Tensor] = None
        self.in_bias: Optional[torch.Tensor] = None
        self.qkv_bias_vec: Optional[torch.Tensor] = None
        self.score_bias: Optional[torch.Tensor] = None
        self.value_mix: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    @property
    def in_rows(self) -> int:
        rows = (self.num_heads + self.num_kv_heads) * self.head_dim + self.num_kv_heads * self.value_dim
        return rows + (self.num_heads if self.output_gate else 0)

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {
            "in_weight": ParamSpec((self.in_rows, self.hidden_size)),
            "score_bias": ParamSpec((self.num_heads,), keep_stored_precision=True),
            "o_weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim)),
        }
        if self.qkv_bias:
            gate_rows = self.num_heads if self.output_gate else 0
            specs["qkv_bias_vec"] = ParamSpec((self.in_rows - gate_rows,), keep_stored_precision=True)
        if self.value_source is not None:  # a checkpoint holds one for the first such layer too, which never reads it
            specs["value_mix"] = ParamSpec((), keep_stored_precision=True)
        return specs

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        self.score_bias = self.score_bias.to(torch.float32)
        if self.value_mix is not None:
            self.value_mix = self.value_mix.to(torch.float32).reshape(1)
        if self.qkv_bias:  # the gate's rows of the one product have no bias
            bias = self.qkv_bias_vec
            self.in_bias = torch.cat([bias, bias.new_zeros(self.in_rows - bias.shape[0])]).contiguous()

    def children(self) -> dict[str, Part]:
        return {"position": self.position} if self.position is not None else {}

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.num_kv_heads, self.kernel_dim)

    def plan(self, ops, shape: PlanInput) -> Optional[MixerPlan]:
        make = getattr(ops, "attention_plan", None)
        return make(shape) if make is not None else None

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        cache = ctx.kv(site)
        rotation = self.position.rotation(ctx) if self.position is not None else None
        projected = ops.linear(h, self.in_weight, self.in_bias, out_dtype=torch.float32)  # norms read it unrounded
        first = None
        if self.value_source == "mixed":
            first = ctx.memo.get(self.MEMO_KEY)
            if first is None:
                raise RuntimeError("a layer that mixes the first layer's values in runs before any layer that keeps them")
        keep = self.value_source == "first" and self.MEMO_KEY not in ctx.memo
        q, gate, kept = ops.head_norm_rope_write(
            projected,
            heads=self.num_heads,
            kv_heads=self.num_kv_heads,
            head_dim=self.head_dim,
            value_dim=self.value_dim,
            kernel_dim=self.kernel_dim,
            eps=self.norm_eps,
            rotation=rotation,
            slot_mapping=cache.slot_mapping,
            key_pages=cache.key,
            value_pages=cache.value,
            block_size=cache.block_size,
            gated=self.output_gate,
            keep_values=keep,
            first_values=first,
            mix_weight=self.value_mix,
        )
        if keep:
            ctx.memo[self.MEMO_KEY] = kept
        cache.written()
        cache.reading()
        attended = ops.paged_attention(
            q,
            cache.key,
            cache.value,
            cache.block_table,
            ctx,
            num_heads=self.num_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.kernel_dim,
            block_size=cache.block_size,
            scale=self.scale,
            window=None,
            plan=ctx.plan(getattr(ops, "ATTENTION_PLAN", None)),
            score_bias=self.score_bias,
        )
        if self.output_gate or self.kernel_dim != self.value_dim:
            attended = ops.scale_heads(
                attended, gate, heads=self.num_heads, head_dim=self.kernel_dim, out_dim=self.value_dim
            )
        return ops.linear(attended, self.o_weight, None, for_stream=True)
