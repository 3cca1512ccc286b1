"""Position encodings."""

from __future__ import annotations

from typing import Mapping, Optional

import math

import numpy as np
import torch

from .base import PositionEncoding
from .context import StepContext
from .registry import register_part


@register_part("position", "rotary")
class RotaryEmbedding(PositionEncoding):
    """Half-split rotary encoding: dims j and j + r/2 of a head are rotated by the
    angle `pos * theta^(-2j/r)`.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:34-61 (`rotate_half` pairs the
    two halves; the reference rotates the whole head, r = head_dim).  The inverse
    frequencies are computed once in float64 on the host; the angles and their
    cosines and sines are computed once per step for all layers that share this
    encoding's constants.

    scaling: None, or the four numbers (factor, original, fast, slow) of a stretch for contexts
    beyond the `original` length.  With dim(t) = r ln(original / (2 pi t)) / (2 ln theta), lo =
    max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), r - 1) and ramp_j = clamp((j - lo) / max(hi -
    lo, 0.001), 0, 1), pair j turns at f_j / factor * ramp_j + f_j * (1 - ramp_j): fast pairs keep
    their frequency, slow ones are stretched by `factor`.  Cosines and sines are then multiplied by
    0.1 ln(factor) + 1.  A scaling that gives `factor` alone is the linear one: every pair turns at f_j /
    factor, amplitudes stay 1.

    interleaved: the checkpoint pairs dim 2j with dim 2j + 1 (instead of j with j + r/2).  The kernels
    rotate halves; a dot product of a query and a key does not care in which order both list their
    dims, so a mixer that projects q and k reorders the rows of both projections once, when its weights
    are bound, by `half_split_order()` (pair j's first members to the front half, its second members
    behind them), and everything after that is the half-split rotation.
    """

    replayable = True

    def __init__(
        self,
        head_dim: int,
        theta: float,
        rotary_dim: Optional[int] = None,
        scaling: Optional[Mapping[str, float]] = None,
        interleaved: bool = False,
    ) -> None:
        self.interleaved = bool(interleaved)
        rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        if rotary_dim <= 0 or rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError("rotary_dim must be even and within head_dim")
        if not theta > 0:
            raise ValueError("theta must be > 0")
        self.head_dim = int(head_dim)
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        exponents = np.arange(0, rotary_dim, 2, dtype=np.float64) / rotary_dim
        self._inv_freq_host = 1.0 / (self.theta**exponents)
        self.amplitude = 1.0
        self.scaling = None
        if scaling is not None and "original" not in scaling:
            factor = float(scaling["factor"])
            if not factor > 0:
                raise ValueError("the factor of a rotary scaling must be > 0")
            self.scaling = (factor,)
            self._inv_freq_host = self._inv_freq_host / factor
        elif scaling is not None:
            factor, original = float(scaling["factor"]), float(scaling["original"])
            fast, slow = float(scaling["fast"]), float(scaling["slow"])
            if not (factor > 0 and original > 0 and fast > 0 and slow > 0):
                raise ValueError("the numbers of a rotary scaling must be > 0")
            self.scaling = (factor, original, fast, slow)

            def pair_of(turns: float) -> float:  # the (fractional) pair that makes `turns` turns over `original` positions
                return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

            lo = max(math.floor(pair_of(fast)), 0)
            hi = min(math.ceil(pair_of(slow)), rotary_dim - 1)
            ramp = np.clip((np.arange(rotary_dim // 2, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            self._inv_freq_host = self._inv_freq_host / factor * ramp + self._inv_freq_host * (1.0 - ramp)
            self.amplitude = 0.1 * math.log(factor) + 1.0
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, params: Mapping[str, torch.Tensor], *, dtype: torch.dtype, device: torch.device) -> None:
        self.inv_freq = torch.from_numpy(self._inv_freq_host).to(device)

    def half_split_order(self) -> list[int]:
        """For every dim of a head in the order the kernels want, the dim of the checkpoint's order
        that goes there (the identity unless `interleaved`)."""
        r = self.rotary_dim
        if not self.interleaved:
            return list(range(self.head_dim))
        return list(range(0, r, 2)) + list(range(1, r, 2)) + list(range(r, self.head_dim))

    def rotation(self, ctx: StepContext):
        key = ("rotary", self.rotary_dim, self.theta, self.scaling)
        if key not in ctx.memo:
            if self.amplitude != 1.0:
                cos, sin = ctx.ops.rope_table(ctx.positions, self.inv_freq, amplitude=self.amplitude)
            else:
                cos, sin = ctx.ops.rope_table(ctx.positions, self.inv_freq)
            ctx.memo[key] = (cos, sin, self.rotary_dim)
        return ctx.memo[key]


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding at all (order enters through the causal mask only)."""

    replayable = True


    def __init__(self, head_dim: int = 0) -> None:
        self.head_dim = head_dim

    def apply(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor) -> None:
        return None
