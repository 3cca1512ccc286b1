"""Arrangements of parts around the residual stream."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import Block, FeedForward, Mixer, Norm, Part
from ..kernels.pending import NormedDelta, StreamUpdate
from ..cache.spec import CompositeSpec
from .context import StepContext, site_member
from .registry import register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm_in(x)); x += feed_forward(norm_post(x)).

    src/mini_llm_runtime/qwen_model_runner.py:198-218.  The residual stream is kept
    in 32-bit; each addition is fused into the norm that follows it, so the block
    hands its last output to the next block (or the model) un-added.  A layer without a
    feed-forward (`feed_forward` None) is its first half only and needs only the "input" norm.
    """

    replayable = True


    norm_names = ("input", "post_mixer")

    def __init__(self, mixer: Mixer, feed_forward: Optional[FeedForward], norms: Mapping[str, Norm]) -> None:
        needed = self.norm_names if feed_forward is not None else self.norm_names[:1]
        missing = [n for n in needed if n not in norms]
        if missing:
            raise ValueError(f"pre_norm block needs the norms {needed}, missing {missing}")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_input = norms["input"]
        self.norm_post_mixer = norms["post_mixer"] if feed_forward is not None else None

    def children(self) -> dict[str, Part]:
        parts: dict[str, Part] = {"mixer": self.mixer, "norm_input": self.norm_input}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
            parts["norm_post_mixer"] = self.norm_post_mixer
        return parts

    def forward(
        self, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor], site: int
    ) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        h = _norm(self.norm_input, self.mixer, ctx, x, delta)
        mixed = self.mixer.forward(ctx, h, site)
        x = _stream_after(h, x)
        if self.feed_forward is None:
            return x, mixed
        h = _norm(self.norm_post_mixer, self.feed_forward, ctx, x, mixed)
        out = self.feed_forward.forward(ctx, h)
        return _stream_after(h, x), out


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """Norms before AND after each sublayer:

        x += norm_mixer_out(mixer(norm_input(x)));  x += norm_ff_out(feed_forward(norm_post_mixer(x)));
        x += norm(token_input(x))      (if the layer has a token input; it reads the stream itself, un-normed)

    A sublayer's output y enters the stream as w * y * rsqrt(mean(y^2) + eps), computed in 32-bit.  Each
    such addition is one kernel with the norm (or the rounding of the stream to the engine's dtype)
    that reads the stream next; the last one is handed to the next block as a `NormedDelta`.
    A layer may have no feed-forward and no token input.
    """

    replayable = True

    def __init__(
        self,
        mixer: Mixer,
        feed_forward: Optional[FeedForward],
        norms: Mapping[str, Norm],
        token_input: Optional[Part] = None,
    ) -> None:
        needed = ["input", "mixer_out"] + (["post_mixer", "ff_out"] if feed_forward is not None else [])
        missing = [n for n in needed if n not in norms]
        if missing:
            raise ValueError(f"sandwich_norm block needs the norms {needed}, missing {missing}")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.token_input = token_input
        self.norm_input = norms["input"]
        self.norm_mixer_out = norms["mixer_out"]
        self.norm_post_mixer = norms.get("post_mixer") if feed_forward is not None else None
        self.norm_ff_out = norms.get("ff_out") if feed_forward is not None else None
        for norm in (self.norm_mixer_out, self.norm_post_mixer, self.norm_ff_out):
            if norm is not None and not hasattr(norm, "eps"):
                raise ValueError("sandwich_norm takes RMS norms (a weight and an eps)")

    def children(self) -> dict[str, Part]:
        parts: dict[str, Part] = {"mixer": self.mixer, "norm_input": self.norm_input, "norm_mixer_out": self.norm_mixer_out}
        if self.feed_forward is not None:
            parts.update(feed_forward=self.feed_forward, norm_post_mixer=self.norm_post_mixer, norm_ff_out=self.norm_ff_out)
        if self.token_input is not None:
            parts["token_input"] = self.token_input
        return parts

    def forward(
        self, ctx: StepContext, x: torch.Tensor, delta, site: int
    ) -> tuple[torch.Tensor, Optional[NormedDelta]]:
        ops = ctx.ops
        h = self.norm_input.forward(ctx, x, delta)
        mixed = self.mixer.forward(ctx, h, site)
        owed = NormedDelta(mixed, self.norm_mixer_out.weight, self.norm_mixer_out.eps)
        if self.feed_forward is not None:
            h = ops.add_normed(
                x, owed.y, owed.weight, owed.eps, next_weight=self.norm_post_mixer.weight, next_eps=self.norm_post_mixer.eps
            )
            out = self.feed_forward.forward(ctx, h)
            owed = NormedDelta(out, self.norm_ff_out.weight, self.norm_ff_out.eps)
        if self.token_input is not None:
            stream = ops.add_normed(x, owed.y, owed.weight, owed.eps, cast=True)
            fed = self.token_input.forward(ctx, stream)
            owed = NormedDelta(fed, self.token_input.norm_weight, self.token_input.norm_eps)
        return x, owed


@register_part("block", "parallel")
class ParallelBlock(Block):
    """One norm, both sublayers read it, both results enter the stream together:

        h = norm_input(x);   x += mixer(filter(h)) + feed_forward(h)

    `mixer_filter` (optional): a part the normed activations pass on their way into the mixer only, e.g. a
    short convolution over time with carried inputs; the feed-forward reads h as it is.  A layer may have no
    feed-forward.  The mixer's result is added to the 32-bit stream by a kernel of its own; the
    feed-forward's is handed to the next block un-added, like every block's last output.  What the filter
    carries from step to step is a member of the site's cache beside the mixer's.
    """

    replayable = True

    def __init__(
        self,
        mixer: Mixer,
        feed_forward: Optional[FeedForward],
        norms: Mapping[str, Norm],
        mixer_filter: Optional[Part] = None,
    ) -> None:
        if "input" not in norms:
            raise ValueError("parallel block needs the norm 'input'")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_filter = mixer_filter
        self.norm_input = norms["input"]
        filter_spec = mixer_filter.cache_spec() if mixer_filter is not None and hasattr(mixer_filter, "cache_spec") else None
        self._filter_keeps = filter_spec is not None

    def children(self) -> dict[str, Part]:
        parts: dict[str, Part] = {"mixer": self.mixer, "norm_input": self.norm_input}
        if self.feed_forward is not None:
            parts["feed_forward"] = self.feed_forward
        if self.mixer_filter is not None:
            parts["mixer_filter"] = self.mixer_filter
        return parts

    def cache_spec(self):
        own = self.mixer.cache_spec()
        if not self._filter_keeps:
            return own
        members = {"filter": self.mixer_filter.cache_spec()}
        if own is not None:
            members["mixer"] = own
        return CompositeSpec(members)

    def forward(
        self, ctx: StepContext, x: torch.Tensor, delta, site: int
    ) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        h = self.norm_input.forward(ctx, x, delta)
        m = h
        if self.mixer_filter is not None:
            m = self.mixer_filter.forward(ctx, h, site_member(site, "filter") if self._filter_keeps else site)
        mixed = self.mixer.forward(ctx, m, site_member(site, "mixer") if self._filter_keeps else site)
        if self.feed_forward is None:
            return x, mixed
        ctx.ops.add_(x, mixed)
        return x, self.feed_forward.forward(ctx, h)


@register_part("block", "hyper_connections")
class HyperConnectionBlock(Block):
    """Several residual streams x_1 .. x_S instead of one (`x` is [S, T, hidden], float32).  For each sublayer
    (the mixer, then the feed-forward) with its own read weights r [S], mixing matrix M [S, S] (indexed [from,
    to]) and write weights w [S]:

        u = sum_s r[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s M[s, t] x_s + w[t] * y   (all t at once).

    This takes the place of the residual addition.  The update of one sublayer and the weighted sum and norm
    of the next are one kernel; the last update is handed to the next block (or the model, which sums the
    streams before its final norm) as a `StreamUpdate`.  A layer may have no feed-forward.
    """

    replayable = True

    def __init__(
        self, mixer: Mixer, feed_forward: Optional[FeedForward], norms: Mapping[str, Norm], streams: int = 1
    ) -> None:
        needed = ("input", "post_mixer") if feed_forward is not None else ("input",)
        missing = [n for n in needed if n not in norms]
        if missing:
            raise ValueError(f"hyper_connections block needs the norms {needed}, missing {missing}")
        if streams <= 0 or streams > 16:
            raise ValueError("hyper_connections keeps 1 to 16 streams")
        self.streams = int(streams)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norm_input = norms["input"]
        self.norm_post_mixer = norms["post_mixer"] if feed_forward is not None else None
        for norm in (self.norm_input, self.norm_post_mixer):
            if norm is not None and not hasattr(norm, "eps"):
                raise ValueError("hyper_connections takes RMS norms (a weight and an eps)")

    def children(self) -> dict[str, Part]:
        parts: dict[str, Part] = {"mixer": self.mixer, "norm_input": self.norm_input}
        if self.feed_forward is not None:
            parts.update(feed_forward=self.feed_forward, norm_post_mixer=self.norm_post_mixer)
        return parts

    def param_specs(self):
        from .spec import ParamSpec

        S = self.streams
        specs = {}
        for name in ("mixer", "ff") if self.feed_forward is not None else ("mixer",):
            specs[f"{name}_read"] = ParamSpec((S,), init="one_plus_normal", keep_stored_precision=True)
            specs[f"{name}_write"] = ParamSpec((S,), init="one_plus_normal", keep_stored_precision=True)
            specs[f"{name}_mix"] = ParamSpec((S, S), init="eye_plus_normal", keep_stored_precision=True)
        return specs

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        # the streams and everything that is added into them are 32-bit
        for name, tensor in params.items():
            setattr(self, name, tensor.to(torch.float32).contiguous())

    def forward(self, ctx: StepContext, x: torch.Tensor, delta, site: int):
        ops = ctx.ops
        if x.dim() != 3 or x.shape[0] != self.streams:
            raise RuntimeError(f"hyper_connections block of {self.streams} streams was handed a stream of shape {tuple(x.shape)}")
        owed = delta.as_update() if delta is not None else None
        h, _ = ops.streams_step(
            x, update=owed, read_weights=self.mixer_read, norm_weight=self.norm_input.weight, eps=self.norm_input.eps
        )
        mixed = self.mixer.forward(ctx, h, site)
        if self.feed_forward is None:
            return x, StreamUpdate(mixed, self.mixer_mix, self.mixer_write)
        h, _ = ops.streams_step(
            x, update=(mixed, self.mixer_mix, self.mixer_write), read_weights=self.ff_read,
            norm_weight=self.norm_post_mixer.weight, eps=self.norm_post_mixer.eps,
        )
        return x, StreamUpdate(self.feed_forward.forward(ctx, h), self.ff_mix, self.ff_write)


def _norm(norm: Norm, consumer: Part, ctx: StepContext, x: torch.Tensor, delta: Optional[torch.Tensor]):
    """norm(x + delta) for `consumer`: possibly not run yet, if both sides can deal with that."""
    if norm.can_defer and consumer.takes_pending_norm:
        return norm.forward(ctx, x, delta, defer=True)
    return norm.forward(ctx, x, delta)


def _stream_after(h, x: torch.Tensor) -> torch.Tensor:
    """The residual stream once `h` was consumed: the tensor the norm updated in place, or the
    new one that the consumer of a pending norm wrote."""
    if isinstance(h, torch.Tensor):
        return x
    if h.residual is None:
        raise RuntimeError("a part that takes pending norms did not hand its input to an operation that runs them")
    return h.residual
