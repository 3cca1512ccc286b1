"""Linear attention whose state forgets per key channel, by a gate computed from the token."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ..cache.spec import SlotStateSpec
from ..kernels.limits import MAX_STATE_ROWS
from .base import Mixer
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Per head, with state S (head_dim x value_dim, 32-bit, zero at a request's start):

        S_t = diag(a_t) S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t,

    q = Wq h * head_dim^-0.5, k = Wk h, v = Wv h, and a decay per key channel and token a_t = sigmoid(z_t)^(1/tau),
    z_t = W2 (W1 h) + b (a product through `decay_rank` numbers), laid out heads x head_dim.  Every head's o_t is
    divided by its root mean square and multiplied by one weight [value_dim] that all heads share; the heads side
    by side are multiplied by silu(Wg h) and projected by Wo.

    The state is all a request keeps (one slot of the cache manager's state banks), so a prompt can be cut
    anywhere.  The five products that read h are one (rows q, k, v, gate, W1; 32-bit sums); the small product with W2,
    the decay, the recurrence, the heads' norm and the gate are 32-bit.
    """

    replayable = True
    open_output = True
    open_input = True  # `activations(projected=)` takes the input product's sums from whoever made them
    in_bias = None

    def __init__(
        self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay_rank: int, tau: float, norm_eps: float
    ) -> None:
        if min(hidden_size, num_heads, head_dim, value_dim, decay_rank) <= 0 or not tau > 0:
            raise ValueError("GatedLinearAttention sizes and tau must be > 0")
        if head_dim > MAX_STATE_ROWS:
            raise ValueError(f"head_dim {head_dim}: the recurrence kernels take heads of up to {MAX_STATE_ROWS} dims")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.decay_rank = int(decay_rank)
        self.tau = float(tau)
        self.norm_eps = float(norm_eps)
        self.q_scale = float(head_dim) ** -0.5
        self.in_weight: Optional[torch.Tensor] = None
        self.decay_weight: Optional[torch.Tensor] = None
        self.decay_bias: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    @property
    def qk_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def out_width(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def in_rows(self) -> int:
        return 2 * self.qk_size + 2 * self.out_width + self.decay_rank

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "in_weight": ParamSpec((self.in_rows, self.hidden_size)),
            "decay_weight": ParamSpec((self.qk_size, self.decay_rank)),
            "decay_bias": ParamSpec((self.qk_size,), keep_stored_precision=True),
            "norm_weight": ParamSpec((self.value_dim,), init="one_plus_normal", keep_stored_precision=True),
            "o_weight": ParamSpec((self.hidden_size, self.out_width)),
        }

    def cache_spec(self) -> SlotStateSpec:
        return SlotStateSpec((self.num_heads, self.head_dim, self.value_dim), "float32")

    def activations(
        self, ctx: StepContext, h, site: Any, *, out: torch.Tensor, column: int, scale: float = 1.0, projected=None
    ) -> None:
        """`projected`: (float32 sums [T, ...], first column) of h times `in_weight`, when the caller made them
        within a larger product."""
        ops = ctx.ops
        state = ctx.state(site)
        first = 0
        if projected is None:
            projected = ops.linear(h, self.in_weight, None, out_dtype=torch.float32)  # what enters the recurrence stays 32-bit
        else:
            projected, first = projected
        retained = ops.gla_scan(
            projected, state.tensor, state.read_rows, state.write_rows, ctx,
            heads=self.num_heads, head_dim=self.head_dim, value_dim=self.value_dim,
            decay_weight=self.decay_weight, decay_bias=self.decay_bias,
            low_offset=2 * self.qk_size + 2 * self.out_width, tau=self.tau, q_scale=self.q_scale,
            **({"projected_column": first} if first else {}),
        )
        ops.retention_gate(
            retained, projected, heads=self.num_heads, value_dim=self.value_dim, gate_offset=first + 2 * self.qk_size + self.out_width,
            eps=self.norm_eps, norm_weight=self.norm_weight, scale=scale, out=out, column=column,
        )

    def forward(self, ctx: StepContext, h: torch.Tensor, site: Any) -> torch.Tensor:
        out = torch.empty((h.shape[0], self.out_width), dtype=ctx.dtype, device=ctx.device)
        self.activations(ctx, h, site, out=out, column=0)
        return ctx.ops.linear(out, self.o_weight, None, for_stream=True)
