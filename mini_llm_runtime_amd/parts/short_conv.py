"""Filters on a mixer's input."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ..cache.spec import SlotStateSpec
from .base import Part
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("input_filter", "causal_conv")
class CausalConv(Part):
    """A causal convolution over time on each channel, added to its input:

        out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j),   j = 0 .. taps - 1, zeros before a request's start

    (`residual=False`: the convolution alone).  No bias.  The last `taps - 1` inputs of a request are
    its state (a slot of the cache manager's state banks, 32-bit), so a prompt can be cut anywhere.
    Sums in 32-bit, one rounding.
    """

    replayable = True

    def __init__(self, width: int, taps: int, residual: bool = True) -> None:
        if width <= 0 or taps <= 0:
            raise ValueError("CausalConv sizes must be > 0")
        self.width = int(width)
        self.taps = int(taps)
        self.residual = bool(residual)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.width, self.taps), keep_stored_precision=True)}

    def cache_spec(self) -> Optional[SlotStateSpec]:
        if self.taps == 1:
            return None
        return SlotStateSpec((self.taps - 1, self.width), "float32")

    def forward(self, ctx: StepContext, h: torch.Tensor, site: Any) -> torch.Tensor:
        """`site`: what `ctx.cache` takes to find this filter's carried inputs (unused with one tap)."""
        if self.taps == 1:
            return ctx.ops.short_conv(h, self.weight, None, None, None, ctx, add_input=self.residual)
        state = ctx.state(site)
        return ctx.ops.short_conv(h, self.weight, state.tensor, state.read_rows, state.write_rows, ctx, add_input=self.residual)
