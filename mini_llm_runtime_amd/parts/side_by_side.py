"""Several mixers on one input."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..cache.spec import CompositeSpec
from .base import Mixer, Part
from .context import StepContext, site_member
from .registry import build_part, register_part
from .spec import ParamSpec, PartSpec


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """Mixers that all read the same input; the result is the sum of their results, each times a
    constant:  sum_m scale_m * mixer_m(h).

    Every member leaves its output product open (`Mixer.open_output`): the members' activations, each
    already times its constant (in 32-bit, before their one rounding), stand side by side in one
    tensor and ONE product with the members' output matrices side by side, [Wo_a | Wo_b | ...], makes
    the sum.  That matrix is put together when the weights are bound; the members' own copies are
    dropped.  Members that take their input product's sums from outside (`open_input`: an `in_weight`
    [rows, hidden], maybe an `in_bias`, and `activations(projected=)`) share ONE input product too: their
    matrices one under the other, 32-bit sums, each member reading its own columns.  Every member keeps its own cache: the site's cache is a composite with one member per mixer
    that keeps one, under the mixer's name.
    """

    replayable = True
    open_output = True

    def __init__(self, hidden_size: int, members: Mapping[str, PartSpec], scales: Optional[Mapping[str, float]] = None) -> None:
        if not members:
            raise ValueError("side_by_side needs at least one mixer")
        self.hidden_size = int(hidden_size)
        self.members: dict[str, Mixer] = {name: build_part("mixer", spec) for name, spec in members.items()}
        self.scales = {name: float((scales or {}).get(name, 1.0)) for name in self.members}
        for name, member in self.members.items():
            if not member.open_output:
                raise ValueError(f"side_by_side member {name!r} does not leave its output product open")
        self.columns: dict[str, int] = {}
        at = 0
        for name, member in self.members.items():
            self.columns[name] = at
            at += member.out_width
        self._width = at
        self.o_weight: Optional[torch.Tensor] = None
        self.in_weight: Optional[torch.Tensor] = None
        self.in_bias: Optional[torch.Tensor] = None
        self.in_columns: dict[str, int] = {}

    @property
    def out_width(self) -> int:
        return self._width

    def children(self) -> dict[str, Part]:
        return dict(self.members)

    def bound(self) -> None:
        """[hidden, sum of the members' widths]; the members' own matrices are let go."""
        parts = []
        for name, member in self.members.items():
            if member.o_weight is None:
                raise RuntimeError(f"side_by_side: the output matrix of member {name!r} is not bound")
            parts.append(member.o_weight)
        self.o_weight = torch.cat(parts, dim=1).contiguous()
        for member in self.members.values():
            member.o_weight = None
        if len(self.members) > 1 and all(getattr(m, "open_input", False) and m.in_weight is not None for m in self.members.values()):
            at, weights, biases = 0, [], []
            for name, member in self.members.items():
                self.in_columns[name] = at
                at += member.in_weight.shape[0]
                weights.append(member.in_weight)
                biases.append(getattr(member, "in_bias", None))
            self.in_weight = torch.cat(weights, dim=0).contiguous()
            if any(b is not None for b in biases):
                kind = next(b.dtype for b in biases if b is not None)
                self.in_bias = torch.cat(
                    [b.to(kind) if b is not None else w.new_zeros(w.shape[0], dtype=kind) for b, w in zip(biases, weights)]
                ).contiguous()
            for member in self.members.values():
                member.in_weight = None
                if getattr(member, "in_bias", None) is not None:
                    member.in_bias = None

    def held_tensors(self) -> list:
        return [self.o_weight, self.in_weight, self.in_bias]

    def cache_spec(self) -> Any:
        specs = {name: member.cache_spec() for name, member in self.members.items()}
        specs = {name: spec for name, spec in specs.items() if spec is not None}
        return CompositeSpec(specs) if specs else None

    def plan(self, ops, shape):
        for member in self.members.values():
            plan = member.plan(ops, shape)
            if plan is not None:
                return plan
        return None

    def activations(self, ctx: StepContext, h, site: Any, *, out: torch.Tensor, column: int, scale: float = 1.0) -> None:
        projected = None
        if self.in_weight is not None:
            projected = ctx.ops.linear(h, self.in_weight, self.in_bias, out_dtype=torch.float32)
        for name, member in self.members.items():
            member.activations(
                ctx, h, site_member(site, name), out=out, column=column + self.columns[name], scale=scale * self.scales[name],
                **({"projected": (projected, self.in_columns[name])} if projected is not None else {}),
            )

    def forward(self, ctx: StepContext, h: torch.Tensor, site: Any) -> torch.Tensor:
        weight = self.o_weight
        out = torch.empty((h.shape[0], self._width), dtype=ctx.dtype, device=ctx.device)
        self.activations(ctx, h, site, out=out, column=0)
        return ctx.ops.linear(out, weight, None, for_stream=True)
