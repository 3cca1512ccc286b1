"""The Vobisun decoder as a list of parts.

Every layer is a parallel one: one norm, whose output the mixer reads through a short causal
convolution (added to its input) and the feed-forward reads as it is; both results enter the stream
together.  The mixer is two mixers side by side on the same input: softmax attention over a sliding
window plus pooled blocks of what left the window (biased projections, queries and keys normed over
their whole projection, a rotation of neighbouring pairs with linearly stretched positions, a learned
temperature and sink per head, a gate per head), and linear attention with a decay per key channel
computed from the token; their results are added with constant weights.  The feed-forward is a dense
SwiGLU or absent.  A span of layers may run several times in a row with the same weights; every run is
an execution site with a cache and state of its own.  The embedding is scaled; the head is a matrix of
its own.

Checkpoint tensors: `embed`, `final.norm`, `head`, and per layer i `l<i>.norm1`, `l<i>.canon1` [width,
taps], `l<i>.mix.left.{q,k,v}` with `.b` biases, `.q.norm`, `.k.norm`, `.temp`, `.sink`, `.g`, `.o`,
`l<i>.mix.right.{q,k,v,g,o,norm,a1,a2,a2.b}`, `l<i>.mlp.{gate,up,down}`; linear weights are stored
[out, in].
"""

from __future__ import annotations

from ..config.vobisun import VobisunConfig
from ..parts.spec import LayerSpec, ModelSpec, OrderEntry, PartSpec, WeightRule
from .registry import register_architecture

# positions are only limited by what a rotation can tell apart
_NO_POSITION_LIMIT = 1 << 30


def vobisun_spec(config: VobisunConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps})
    layers: list[LayerSpec] = []
    rules: list[WeightRule] = [WeightRule("embed", "embed.weight")]
    for i, layer in enumerate(config.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        a, b = layer.left, layer.right
        rank = b.rank  # from the stored tensor's shape when the configuration was read beside a checkpoint
        rotary = PartSpec(
            "rotary",
            {
                "head_dim": a.dim, "theta": a.rot.base, "rotary_dim": a.rot.dims, "interleaved": True,
                "scaling": None if a.rot.factor == 1.0 else {"factor": a.rot.factor},
            },
        )
        left = PartSpec(
            "pooled_window_attention",
            {
                "hidden_size": width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
                "value_dim": a.vdim, "window": a.window, "pool": a.pool, "scale": a.scale,
                "position": rotary if a.rot.dims > 0 else None,  # no dims turn: no position encoding at all
                "qkv_bias": True, "qk_norm": True, "norm_eps": eps, "temperature": True, "sink": True, "head_gate": True,
            },
        )
        right = PartSpec(
            "gated_linear_attention",
            {
                "hidden_size": width, "num_heads": b.heads, "head_dim": b.dim, "value_dim": b.vdim, "decay_rank": rank,
                "tau": b.tau, "norm_eps": eps,
            },
        )
        mixer = PartSpec(
            "side_by_side",
            {
                "hidden_size": width, "members": {"left": left, "right": right},
                "scales": {"left": layer.left_scale, "right": layer.right_scale},
            },
        )
        lm, rm = dst + "mixer.left.", dst + "mixer.right."
        q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        rq, rv = b.heads * b.dim, b.heads * b.vdim
        rules += [
            WeightRule(src + "norm1", dst + "norm_input.weight"),
            WeightRule(src + "canon1", dst + "mixer_filter.weight"),
            WeightRule(src + "mix.left.q", lm + "in_weight", 0, q),
            WeightRule(src + "mix.left.k", lm + "in_weight", q, k),
            WeightRule(src + "mix.left.v", lm + "in_weight", q + k, v),
            WeightRule(src + "mix.left.g", lm + "in_weight", q + k + v, a.heads),
            WeightRule(src + "mix.left.q.b", lm + "in_bias", 0, q),
            WeightRule(src + "mix.left.k.b", lm + "in_bias", q, k),
            WeightRule(src + "mix.left.v.b", lm + "in_bias", q + k, v),
            WeightRule(src + "mix.left.q.norm", lm + "q_norm_weight"),
            WeightRule(src + "mix.left.k.norm", lm + "k_norm_weight"),
            WeightRule(src + "mix.left.temp", lm + "head_scale"),
            WeightRule(src + "mix.left.sink", lm + "sinks"),
            WeightRule(src + "mix.left.o", lm + "o_weight"),
            WeightRule(src + "mix.right.q", rm + "in_weight", 0, rq),
            WeightRule(src + "mix.right.k", rm + "in_weight", rq, rq),
            WeightRule(src + "mix.right.v", rm + "in_weight", 2 * rq, rv),
            WeightRule(src + "mix.right.g", rm + "in_weight", 2 * rq + rv, rv),
            WeightRule(src + "mix.right.a1", rm + "in_weight", 2 * rq + 2 * rv, rank),
            WeightRule(src + "mix.right.a2", rm + "decay_weight"),
            WeightRule(src + "mix.right.a2.b", rm + "decay_bias"),
            WeightRule(src + "mix.right.norm", rm + "norm_weight"),
            WeightRule(src + "mix.right.o", rm + "o_weight"),
        ]
        feed_forward = None
        if layer.ff is not None:
            feed_forward = PartSpec("swiglu", {"hidden_size": width, "intermediate_size": layer.ff})
            ff = dst + "feed_forward."
            if layer.ff % 2 == 0:
                # gate and up rows woven in pairs: the product's epilogue then holds a gate sum beside its up sum
                rules += [
                    WeightRule(src + "mlp.gate", ff + "gate_up_weight", 0, layer.ff, block=2, period=4),
                    WeightRule(src + "mlp.up", ff + "gate_up_weight", 2, layer.ff, block=2, period=4),
                ]
            else:  # an odd size cannot be woven: the gating runs behind the product
                rules += [
                    WeightRule(src + "mlp.gate", ff + "gate_up_weight", 0, layer.ff),
                    WeightRule(src + "mlp.up", ff + "gate_up_weight", layer.ff, layer.ff),
                ]
            rules.append(WeightRule(src + "mlp.down", ff + "down_weight"))
        layers.append(
            LayerSpec(
                block="parallel", mixer=mixer, feed_forward=feed_forward, norms={"input": norm},
                mixer_filter=PartSpec("causal_conv", {"width": width, "taps": config.canon_taps}),
            )
        )
    rules += [WeightRule("final.norm", "final_norm.weight"), WeightRule("head", "head.weight")]
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        hidden_size=width,
        max_position_embeddings=_NO_POSITION_LIMIT,
        layers=tuple(layers),
        order=tuple(OrderEntry(i) for i in config.layer_runs()),  # every run of a layer is a site of its own
        final_norm=norm,
        tie_word_embeddings=False,
        weight_rules=tuple(rules),
        embedding_scale=config.embedding_scale,
    )


register_architecture(
    VobisunConfig.architecture, VobisunConfig, vobisun_spec, replace=True,
    with_shapes=lambda config, shapes: config.with_shapes(shapes),
)
