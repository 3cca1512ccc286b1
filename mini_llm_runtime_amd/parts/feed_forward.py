"""Feed-forward parts."""

from __future__ import annotations

from typing import Optional

import torch

from .base import FeedForward
from .context import StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """Dense gated feed-forward: `down(silu(gate(x)) * up(x))`, without biases or (`bias`) with one on each of
    the three products; with biases the rows are [Wgate ; Wup] and the gating is a kernel of its own.

    Formula: src/mini_llm_runtime/qwen_model_runner.py:215-217.  Gate and up are one
    matrix product over a matrix that holds the rows of Wgate and Wup woven in pairs
    (gate 0, gate 1, up 0, up 1, gate 2, ...; made by the weight rules), and
    silu(gate) * up is that product's epilogue.  An odd intermediate size cannot be woven in
    pairs (`woven` is False): its rows are [Wgate ; Wup] and the gating is a kernel of its own
    behind the product.
    """

    replayable = True
    takes_pending_norm = True  # `h` goes to the gate/up product only

    def __init__(self, hidden_size: int, intermediate_size: int, bias: bool = False) -> None:
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("SwiGLU sizes must be > 0")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.bias = bool(bias)
        self.woven = self.intermediate_size % 2 == 0 and not self.bias
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None
        self.gate_up_bias: Optional[torch.Tensor] = None
        self.down_bias: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = {
            "gate_up_weight": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
            "down_weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }
        if self.bias:
            specs["gate_up_bias"] = ParamSpec((2 * self.intermediate_size,), keep_stored_precision=True)
            specs["down_bias"] = ParamSpec((self.hidden_size,), keep_stored_precision=True)
        return specs

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        ops = ctx.ops
        if self.woven:
            hidden = ops.linear(h, self.gate_up_weight, None, swiglu=True)
        else:
            hidden = ops.silu_mul(ops.linear(h, self.gate_up_weight, self.gate_up_bias))
        return ops.linear(hidden, self.down_weight, self.down_bias, for_stream=True)  # the next norm's delta


@register_part("feed_forward", "clamped_glu")
class ClampedGLU(FeedForward):
    """Dense gated feed-forward with clamped halves and biases on all three products:

        g = min(Wgate x + bgate, limit),  u = clamp(Wup x + bup, -limit, limit),
        y = Wdown (g * sigmoid(alpha * g) * (u + 1)) + bdown.

    Gate and up are one product over a matrix that holds the rows of Wgate and Wup woven in pairs (gate
    0, gate 1, up 0, up 1, gate 2, ...; made by the weight rules, the biases alike), and the gating is that
    product's epilogue, on its 32-bit sums.  An odd intermediate size cannot be woven in pairs (`woven` is
    False): its rows are [Wgate ; Wup] and the gating is a kernel of its own behind the product.
    """

    replayable = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702) -> None:
        if hidden_size <= 0 or intermediate_size <= 0 or not limit > 0:
            raise ValueError("ClampedGLU sizes and limit must be > 0")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.limit = float(limit)
        self.alpha = float(alpha)
        self.woven = self.intermediate_size % 2 == 0
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.gate_up_bias: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None
        self.down_bias: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "gate_up_weight": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
            "gate_up_bias": ParamSpec((2 * self.intermediate_size,), keep_stored_precision=True),
            "down_weight": ParamSpec((self.hidden_size, self.intermediate_size)),
            "down_bias": ParamSpec((self.hidden_size,), keep_stored_precision=True),
        }

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        ops = ctx.ops
        if self.woven:
            hidden = ops.linear(h, self.gate_up_weight, self.gate_up_bias, clamped_glu=(self.limit, self.alpha))
        else:
            sums = ops.linear(h, self.gate_up_weight, self.gate_up_bias, out_dtype=torch.float32)
            hidden = ops.glu_clamped(sums, self.limit, self.alpha)
        return ops.linear(hidden, self.down_weight, self.down_bias, for_stream=True)


ACTIVATIONS = ("relu2", "sigmoid")  # what `ops.linear(..., activation=)` applies to its sums
EXPERT_ACTIVATIONS = ACTIVATIONS + ("swiglu",)  # an expert may also be gated: down(silu(gate(x)) * up(x))


@register_part("feed_forward", "mlp")
class MLP(FeedForward):
    """Dense feed-forward without a gate: `down(act(up(x)))`, no biases.  `activation` is applied
    in the epilogue of the first product; "relu2" is max(z, 0)^2."""

    replayable = True
    takes_pending_norm = True  # `h` goes to the up product only

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2") -> None:
        if hidden_size <= 0 or intermediate_size <= 0:
            raise ValueError("MLP sizes must be > 0")
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.activation = activation
        self.up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "up_weight": ParamSpec((self.intermediate_size, self.hidden_size)),
            "down_weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        ops = ctx.ops
        hidden = ops.linear(h, self.up_weight, None, activation=self.activation)
        return ops.linear(hidden, self.down_weight, None, for_stream=True)  # the next norm's delta


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """A mixture of `experts` small feed-forwards (`down_e(act(up_e(x)))`, no biases) of which every
    token uses `top`.

    Routing, all in 32-bit: z = Wr h, s = sigmoid(z), c = s + correction (a stored vector; c only
    decides, the mixture's weights come from s).  The expert axis is cut into `groups` contiguous
    blocks of experts / groups; block score = top-2 sum of its c; eligible = experts of the
    `keep_groups` highest blocks (c := -inf elsewhere, since c may be negative); chosen = arg-top-`top`
    of c over the eligible; y = sum over chosen e of (router_scale * s_e) * expert_e(h), with no
    division by the sum of the weights.

    Everything runs on the device, so steps can be recorded: the routing kernel leaves expert ids
    and weights per token, an alignment kernel sorts the (token, choice) pairs by expert into row
    tiles, and two grouped products run over those tiles (up with the activation, down with the
    pair's weight).  The result is a float32 stack [top, tokens, hidden] of the weighted expert
    outputs, which the next norm adds to the stream in that fixed order.
    Expert matrices are stacked along the rows: up [experts * inner, hidden], down [experts *
    hidden, inner].

    What other routers do differently, each an option:
    scores: "softmax" makes s the softmax of z over all router outputs instead of sigmoids.
    normalise: the chosen experts' weights are divided by their sum (+ 1e-20) before `router_scale`.
    identity: the router has `experts + identity` outputs; the last `identity` of them are experts without
        matrices whose output is their input itself (times the weight).
    activation "swiglu": every expert is gated, down_e(silu(gate_e(x)) * up_e(x)); `up_weight` then holds, per
        expert, its gate rows and then its up rows ([experts * 2 * inner, hidden]).
    """

    replayable = True

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        experts: int,
        top: int,
        router_scale: float = 1.0,
        groups: int = 1,
        keep_groups: int = 1,
        activation: str = "relu2",
        scores: str = "sigmoid",
        normalise: bool = False,
        identity: int = 0,
    ) -> None:
        if hidden_size <= 0 or intermediate_size <= 0 or experts <= 0 or top <= 0 or identity < 0:
            raise ValueError("RoutedExperts sizes must be > 0")
        routed = experts + identity  # what the router chooses among
        if groups <= 0 or routed % groups or not 0 < keep_groups <= groups:
            raise ValueError("the experts must divide into equal groups, of which 1..groups are kept")
        if top > keep_groups * (routed // groups):
            raise ValueError("the kept groups hold fewer experts than a token uses")
        if scores not in ("sigmoid", "softmax"):
            raise ValueError("scores are 'sigmoid' or 'softmax'")
        if activation not in EXPERT_ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.experts = int(experts)
        self.top = int(top)
        self.router_scale = float(router_scale)
        self.groups = int(groups)
        self.keep_groups = int(keep_groups)
        self.activation = activation
        self.scores = scores
        self.normalise = bool(normalise)
        self.identity = int(identity)
        self.routed = routed
        self.router_weight: Optional[torch.Tensor] = None
        self.correction: Optional[torch.Tensor] = None
        self.up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def param_specs(self) -> dict[str, ParamSpec]:
        return {
            "router_weight": ParamSpec((self.routed, self.hidden_size)),
            "correction": ParamSpec((self.routed,), keep_stored_precision=True),
            "up_weight": ParamSpec(
                (self.experts * self.intermediate_size * (2 if self.activation == "swiglu" else 1), self.hidden_size)
            ),
            "down_weight": ParamSpec((self.experts * self.hidden_size, self.intermediate_size)),
        }

    def bind(self, params, *, dtype: torch.dtype, device: torch.device) -> None:
        super().bind(params, dtype=dtype, device=device)
        self.correction = self.correction.to(torch.float32)  # the routing is 32-bit throughout

    def forward(self, ctx: StepContext, h: torch.Tensor):
        ops = ctx.ops
        logits = ops.linear(h, self.router_weight, None, out_dtype=torch.float32)
        ids, weights = ops.route_experts(
            logits, self.correction, top=self.top, groups=self.groups, keep_groups=self.keep_groups,
            scale=self.router_scale,
            **({"scores": self.scores, "normalise": self.normalise} if (self.scores != "sigmoid" or self.normalise) else {}),
        )
        return ops.expert_products(
            h, self.up_weight, self.down_weight, ids, weights, experts=self.experts, activation=self.activation,
            **({"pass_through": self.identity} if self.identity else {}),
        )
