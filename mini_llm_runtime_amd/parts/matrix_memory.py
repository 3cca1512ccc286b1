"""A matrix memory per head with exponential gates (the mLSTM cell)."""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.spec import SlotStateSpec
from ..kernels.limits import MAX_STATE_ROWS
from .base import Mixer
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("mixer", "matrix_memory")
class MatrixMemory(Mixer):
    """Per head a matrix C (head_dim x value_dim), a vector n (head_dim) and a running maximum m, all 32-bit and
    zero at a request's start (m too).  With h the mixer's input, q = Wq h * head_dim^-0.5, k = Wk h, v = Wv h and
    per head the log gates i = cap tanh((Wi h + bi) / cap), f = logsigmoid(cap tanh((Wf h + bf) / cap)):

        m_t = max(f + m_(t-1), i),
        C_t = exp(f + m_(t-1) - m_t) C_(t-1) + exp(i - m_t) k v^T,     n_t likewise with k alone,
        o_t = C_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6).

    Every head's o is divided by its root mean square (eps inside the root); the heads side by side are
    multiplied by a weight over all of them and by sigmoid(Wg h), then projected by Wo.

    The state (C, n, m of every head, one row of the cache manager's state banks per request) is all a
    request keeps, so a prompt can be cut anywhere.  The five input products and the gate are one product
    (rows q, k, v, gate, input gate, forget gate) whose 32-bit sums the recurrence reads unrounded.
    """

    replayable = True

    def __init__(
        self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, gate_cap: float, norm_eps: float
    ) -> None:
        if min(hidden_size, num_heads, head_dim, value_dim) <= 0:
            raise ValueError("MatrixMemory sizes must be > 0")
        if head_dim > MAX_STATE_ROWS:  # refused here, not at the first step
            raise ValueError(f"head_dim {head_dim}: the memory kernels take heads of up to {MAX_STATE_ROWS} dims")
        if not gate_cap > 0:
            raise ValueError("gate_cap must be > 0")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.gate_cap = float(gate_cap)
        self.norm_eps = float(norm_eps)
        qk, vg = self.num_heads * self.head_dim, self.num_heads * self.value_dim
        # columns of the one input product
        self.q_at, self.k_at, self.v_at, self.gate_at = 0, qk, 2 * qk, 2 * qk + vg
        self.i_at = 2 * qk + 2 * vg
        self.f_at = self.i_at + self.num_heads
        self.in_rows = self.f_at + self.num_heads
        self.in_weight: Optional[torch.Tensor] = None
        self.gate_bias: Optional[torch.Tensor] = None
        self.in_bias: Optional[torch.Tensor] = None
        self.head_norm_weight: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "in_weight": ParamSpec((self.in_rows, self.hidden_size)),
            "gate_bias": ParamSpec((2 * self.num_heads,), keep_stored_precision=True),  # input gates, then forget gates
            "head_norm_weight": ParamSpec(
                (self.num_heads * self.value_dim,), init="one_plus_normal", keep_stored_precision=True
            ),
            "o_weight": ParamSpec((self.hidden_size, self.num_heads * self.value_dim)),
        }

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        bias = self.gate_bias
        self.in_bias = torch.cat([bias.new_zeros(self.i_at), bias]).contiguous()  # only the two gates have one

    def cache_spec(self) -> SlotStateSpec:
        return SlotStateSpec((self.num_heads, self.head_dim * self.value_dim + self.head_dim + 1), "float32")

    def forward(self, ctx: StepContext, h: torch.Tensor, site: int) -> torch.Tensor:
        ops = ctx.ops
        state = ctx.state(site)
        projected = ops.linear(h, self.in_weight, self.in_bias, out_dtype=torch.float32)  # what enters the recurrence stays 32-bit
        remembered = ops.matrix_memory_scan(
            projected,
            state.tensor,
            state.read_rows,
            state.write_rows,
            ctx,
            heads=self.num_heads,
            head_dim=self.head_dim,
            value_dim=self.value_dim,
            offsets=(self.q_at, self.k_at, self.v_at, self.i_at, self.f_at),
            cap=self.gate_cap,
            q_scale=float(self.head_dim) ** -0.5,
        )
        gated = ops.retention_gate(
            remembered, projected, heads=self.num_heads, value_dim=self.value_dim, gate_offset=self.gate_at,
            eps=self.norm_eps, norm_weight=self.head_norm_weight, gate="sigmoid",
        )
        return ops.linear(gated, self.o_weight, None, for_stream=True)
