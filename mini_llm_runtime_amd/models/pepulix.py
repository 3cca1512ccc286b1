"""The Pepulix decoder as a list of parts.

A decoder whose config.json lists the layers one by one.  The layers keep several residual streams
(`hyper_connections`; without `streams` in the config one stream with plain additions, `pre_norm`), mix tokens
by attention with sigmoid weights (`sigmoid_attention`), by softmax attention over cached latents with the
queries through a latent of their own (`latent_attention`), or by a matrix memory with exponential gates
(`matrix_memory`), and have a dense gated feed-forward with biases, a mixture of gated experts among which
some hand their input on, or none.  The head is the embedding table; the logits are capped.

Checkpoint tensors: `embed`, `final.norm`, and per layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.hc{1,2}.{in,out,mix}`,
`l<i>.mix.{q,k,v}` with `.b` biases and `.{vmix,pb,g,o}` (attention), `l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}`
(latent attention), `l<i>.mix.{q,k,v,g,o,norm,i,f}` with `i.b`, `f.b` (memory), `l<i>.mlp.{gate,up,down}` with `.b`
biases (dense) or `l<i>.mlp.{router,correction}` and `l<i>.mlp.e<j>.{gate,up,down}` (experts); linear weights are
stored [out, in].
"""

from __future__ import annotations

from ..config.pepulix import PepulixAttention, PepulixConfig, PepulixLatentAttention, PepulixMemory
from ..parts.spec import LayerSpec, ModelSpec, OrderEntry, PartSpec, WeightRule
from .registry import register_architecture

# positions are only limited by what a rotation can tell apart
_NO_POSITION_LIMIT = 1 << 30


def _rotary(rot, part_dim: int, interleaved: bool = False) -> PartSpec:
    scaling = None
    if rot.scaling is not None:
        s = rot.scaling
        scaling = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    params = {"head_dim": part_dim, "theta": rot.base, "rotary_dim": rot.dims, "scaling": scaling}
    if interleaved:
        params["interleaved"] = True
    return PartSpec("rotary", params)


def pepulix_spec(config: PepulixConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps
    norm = PartSpec("rms_norm", {"size": width, "eps": eps})
    streams = config.streams
    layers: list[LayerSpec] = []
    rules: list[WeightRule] = [WeightRule("embed", "embed.weight")]
    values_kept = False  # whether an earlier layer keeps its values for later ones to mix in
    for i, layer in enumerate(config.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        m = layer.mixer
        mix = dst + "mixer."
        if isinstance(m, PepulixAttention):
            source = None
            if m.v_mix:
                source = "mixed" if values_kept else "first"
                values_kept = True
            mixer = PartSpec(
                "sigmoid_attention",
                {
                    "hidden_size": width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                    "value_dim": m.vdim, "scale": m.scale, "norm_eps": eps, "value_source": source,
                    "position": None if m.rot is None else _rotary(m.rot, m.dim),
                },
            )
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            rules += [
                WeightRule(src + "mix.q", mix + "in_weight", 0, q),
                WeightRule(src + "mix.k", mix + "in_weight", q, k),
                WeightRule(src + "mix.v", mix + "in_weight", q + k, v),
                WeightRule(src + "mix.g", mix + "in_weight", q + k + v, m.heads),
                WeightRule(src + "mix.q.b", mix + "qkv_bias_vec", 0, q),
                WeightRule(src + "mix.k.b", mix + "qkv_bias_vec", q, k),
                WeightRule(src + "mix.v.b", mix + "qkv_bias_vec", q + k, v),
                WeightRule(src + "mix.pb", mix + "score_bias"),
                WeightRule(src + "mix.o", mix + "o_weight"),
            ]
            if source is not None:
                rules.append(WeightRule(src + "mix.vmix", mix + "value_mix"))
        elif isinstance(m, PepulixLatentAttention):
            mixer = PartSpec(
                "latent_attention",
                {
                    "hidden_size": width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
                    "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale, "norm_eps": eps,
                    "position": _rotary(m.rot, m.rot_dim, interleaved=True), "sink": False, "output_gate": False,
                    "q_rank": m.q_rank,
                },
            )
            rules += [
                WeightRule(src + "mix.dq", mix + "dq_weight"),
                WeightRule(src + "mix.dq.norm", mix + "q_norm_weight"),
                WeightRule(src + "mix.uq", mix + "uq_weight"),
                WeightRule(src + "mix.dkv", mix + "in_weight"),
                WeightRule(src + "mix.dkv.norm", mix + "latent_norm_weight"),
                WeightRule(src + "mix.uk", mix + "uk_weight"),
                WeightRule(src + "mix.uv", mix + "uv_weight"),
                WeightRule(src + "mix.o", mix + "o_weight"),
            ]
        elif isinstance(m, PepulixMemory):
            mixer = PartSpec(
                "matrix_memory",
                {
                    "hidden_size": width, "num_heads": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                    "gate_cap": m.gate_cap, "norm_eps": eps,
                },
            )
            qk, vg = m.heads * m.dim, m.heads * m.vdim
            rules += [
                WeightRule(src + "mix.q", mix + "in_weight", 0, qk),
                WeightRule(src + "mix.k", mix + "in_weight", qk, qk),
                WeightRule(src + "mix.v", mix + "in_weight", 2 * qk, vg),
                WeightRule(src + "mix.g", mix + "in_weight", 2 * qk + vg, vg),
                WeightRule(src + "mix.i", mix + "in_weight", 2 * qk + 2 * vg, m.heads),
                WeightRule(src + "mix.f", mix + "in_weight", 2 * qk + 2 * vg + m.heads, m.heads),
                WeightRule(src + "mix.i.b", mix + "gate_bias", 0, m.heads),
                WeightRule(src + "mix.f.b", mix + "gate_bias", m.heads, m.heads),
                WeightRule(src + "mix.norm", mix + "head_norm_weight"),
                WeightRule(src + "mix.o", mix + "o_weight"),
            ]
        else:
            raise TypeError(f"layer {i}: unknown mixer configuration {type(m).__name__}")
        norms = {"input": norm}
        rules.append(WeightRule(src + "norm1", dst + "norm_input.weight"))
        hyper = [("hc1", "mixer")]
        feed_forward = None
        f = layer.mlp
        if f is not None:
            norms["post_mixer"] = norm
            rules.append(WeightRule(src + "norm2", dst + "norm_post_mixer.weight"))
            hyper.append(("hc2", "ff"))
            ff = dst + "feed_forward."
            if f.kind == "dense":
                feed_forward = PartSpec("swiglu", {"hidden_size": width, "intermediate_size": f.ff, "bias": True})
                rules += [
                    WeightRule(src + "mlp.gate", ff + "gate_up_weight", 0, f.ff),
                    WeightRule(src + "mlp.up", ff + "gate_up_weight", f.ff, f.ff),
                    WeightRule(src + "mlp.gate.b", ff + "gate_up_bias", 0, f.ff),
                    WeightRule(src + "mlp.up.b", ff + "gate_up_bias", f.ff, f.ff),
                    WeightRule(src + "mlp.down", ff + "down_weight"),
                    WeightRule(src + "mlp.down.b", ff + "down_bias"),
                ]
            else:
                feed_forward = PartSpec(
                    "routed_experts",
                    {
                        "hidden_size": width, "intermediate_size": f.ff, "experts": f.experts, "top": f.top,
                        "activation": "swiglu", "scores": "softmax", "normalise": True, "identity": f.identity,
                    },
                )
                rules += [WeightRule(src + "mlp.router", ff + "router_weight"), WeightRule(src + "mlp.correction", ff + "correction")]
                for e in range(f.experts):
                    rules += [
                        WeightRule(f"{src}mlp.e{e}.gate", ff + "up_weight", 2 * e * f.ff, f.ff),
                        WeightRule(f"{src}mlp.e{e}.up", ff + "up_weight", (2 * e + 1) * f.ff, f.ff),
                        WeightRule(f"{src}mlp.e{e}.down", ff + "down_weight", e * width, width),
                    ]
        if streams is not None:
            for stored, own in hyper:
                rules += [
                    WeightRule(f"{src}{stored}.in", f"{dst}{own}_read"),
                    WeightRule(f"{src}{stored}.out", f"{dst}{own}_write"),
                    WeightRule(f"{src}{stored}.mix", f"{dst}{own}_mix"),
                ]
        layers.append(
            LayerSpec(
                block="hyper_connections" if streams is not None else "pre_norm", mixer=mixer, feed_forward=feed_forward,
                norms=norms,
            )
        )
    rules.append(WeightRule("final.norm", "final_norm.weight"))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        hidden_size=width,
        max_position_embeddings=_NO_POSITION_LIMIT,
        layers=tuple(layers),
        order=tuple(OrderEntry(i) for i in range(len(layers))),
        final_norm=norm,
        tie_word_embeddings=True,
        weight_rules=tuple(rules),
        logit_softcap=config.logit_softcap,
        residual_streams=streams or 0,
    )


register_architecture(PepulixConfig.architecture, PepulixConfig, pepulix_spec, replace=True)
