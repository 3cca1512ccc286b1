"""A plain, slow implementation of the Vobisun decoder: whole sequences, no cache, no carried
state, float64, one function per mechanism.  It shares no code with the engine; the tests compare
the engine with it.

The model is given as a config dictionary (the keys of config.json) and a dictionary of tensors by
checkpoint name (`embed`, `l<i>.norm1`, `l<i>.canon1`, `l<i>.mix.left.*`, `l<i>.mix.right.*`,
`l<i>.mlp.*`, `final.norm`, `head`), linear weights stored [out, in].
"""

from __future__ import annotations

import torch

F64 = torch.float64
_ROUND = False


class rounded:
    """Within this context every product's input is rounded to bfloat16 first (the weights are bfloat16 anyway):
    what rounding alone does to a row, as a yardstick for rows on which the engine's bfloat16 and the exact
    result differ much (a head's norm of a near-zero output is a sign function)."""

    def __enter__(self):
        global _ROUND
        self.before, _ROUND = _ROUND, True

    def __exit__(self, *exc):
        global _ROUND
        _ROUND = self.before


def _mm(x, w):
    """x times w transposed."""
    if _ROUND:
        x = x.to(torch.bfloat16).to(F64)
    return x @ w.T


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last dimension (weight None: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def causal_conv(h, taps_weight):
    """h [T, W], taps_weight [W, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before t = 0."""
    T, W = h.shape
    taps = taps_weight.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += taps_weight[:, j] * h[: T - back]
    return out


def rotate_interleaved(x, positions, dims, base, factor):
    """x [T, heads, d]: the pairs (2i, 2i + 1), i < dims / 2, turn by position * base^(-2i/dims) / factor."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F64)
    freq = base ** (-2.0 * i / dims) / factor
    angle = positions.to(F64)[:, None] * freq[None, :]  # [T, dims/2]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def pooled_window_attention(q, k, v, *, window, pool, scale, temp, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence (positions 0..T-1).

    Query i sees the tokens j with 0 <= i - j < window, and one pooled key and value (the means over
    the block) for every block b of `pool` tokens with b * pool + pool - 1 <= i - window.  One
    softmax over both, whose denominator also holds exp(sink_h)."""
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    per = H // G
    out = torch.zeros((T, H, dv), dtype=F64)
    blocks = T // pool
    pk = k[: blocks * pool].reshape(blocks, pool, G, d).mean(1) if blocks else k[:0]
    pv = v[: blocks * pool].reshape(blocks, pool, G, dv).mean(1) if blocks else v[:0]
    for i in range(T):
        lo = max(0, i - window + 1)
        seen = 0
        if i - window >= 0:
            seen = (i - window + 1) // pool  # blocks b with (b + 1) * pool - 1 <= i - window
        for h in range(H):
            g = h // per
            keys = torch.cat([pk[:seen, g], k[lo : i + 1, g]])
            vals = torch.cat([pv[:seen, g], v[lo : i + 1, g]])
            s = (keys @ q[i, h]) * scale * temp[h]
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * vals).sum(0) / (e.sum() + torch.exp(sink[h] - m))
    return out


def left_mixer(h, w, p, cfg, eps, positions):
    """The softmax half: biased projections, one norm over all of q and all of k, interleaved
    partial rotation, window with pooled blocks, sink, a gate per head, output projection."""
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = _mm(h, w[p + "q"]) + w[p + "q.b"]
    k = _mm(h, w[p + "k"]) + w[p + "k.b"]
    v = _mm(h, w[p + "v"]) + w[p + "v.b"]
    q = rms_norm(q, w[p + "q.norm"], eps).view(T, H, d)
    k = rms_norm(k, w[p + "k.norm"], eps).view(T, G, d)
    v = v.view(T, G, dv)
    rot = cfg["rot"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    q = rotate_interleaved(q, positions, rot["dims"], rot["base"], factor)
    k = rotate_interleaved(k, positions, rot["dims"], rot["base"], factor)
    a = pooled_window_attention(
        q, k, v, window=cfg["mask"]["size"], pool=cfg["mask"]["pool"], scale=cfg["scale"],
        temp=w[p + "temp"], sink=w[p + "sink"],
    )
    gate = torch.sigmoid(_mm(h, w[p + "g"]))  # [T, H]
    a = a * gate[:, :, None]
    return _mm(a.reshape(T, H * dv), w[p + "o"])


def gated_linear_attention(q, k, v, alpha):
    """q, k, alpha [T, H, d], v [T, H, dv]: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, d = q.shape
    dv = v.shape[2]
    S = torch.zeros((H, d, dv), dtype=F64)
    out = torch.zeros((T, H, dv), dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def right_mixer(h, w, p, cfg, eps):
    """The recurrent half: a decay per key channel from a two-step projection, the recurrence, a norm
    per head with one shared weight, a silu gate, output projection."""
    H, d, dv, tau = cfg["heads"], cfg["dim"], cfg["vdim"], cfg["tau"]
    T = h.shape[0]
    q = (_mm(h, w[p + "q"]) * d ** -0.5).view(T, H, d)
    k = (_mm(h, w[p + "k"])).view(T, H, d)
    v = (_mm(h, w[p + "v"])).view(T, H, dv)
    z = _mm(h, w[p + "a1"]) @ w[p + "a2"].T + w[p + "a2.b"]  # the second product stays exact: it enters the recurrence
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(T, H, d)
    o = gated_linear_attention(q, k, v, alpha)
    o = rms_norm(o, w[p + "norm"], eps).reshape(T, H * dv)
    g = _mm(h, w[p + "g"])
    return _mm(o * g * torch.sigmoid(g), w[p + "o"])


def dense_feed_forward(h, w, p):
    g = _mm(h, w[p + "gate"])
    return _mm(g * torch.sigmoid(g) * _mm(h, w[p + "up"]), w[p + "down"])


def layer(x, w, i, cfg, config, positions):
    """One parallel layer: h = norm(x); x + mixer(h + conv(h)) + feed_forward(h)."""
    eps = config["norm"]["eps"]
    p = f"l{i}."
    h = rms_norm(x, w[p + "norm1"], eps)
    m = h + causal_conv(h, w[p + "canon1"])
    mix = cfg["mixer"]
    y = mix["left_scale"] * left_mixer(m, w, p + "mix.left.", mix["left"], eps, positions)
    y = y + mix["right_scale"] * right_mixer(m, w, p + "mix.right.", mix["right"], eps)
    if cfg.get("mlp") is not None:
        y = y + dense_feed_forward(h, w, p + "mlp.")
    return x + y


def layer_runs(config):
    """The layers in the order they run: start .. stop - 1 `times` times in a row."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config, weights, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (and the stream after every layer run)."""
    w = {k: v.to(F64) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = w["embed"][tokens] * config["embedding"]["scale"]
    streams = []
    for i in layer_runs(config):
        x = layer(x, w, i, config["layers"][i], config, positions)
        streams.append(x)
    logits = _mm(rms_norm(x, w["final.norm"], config["norm"]["eps"]), w["head"])
    return (logits, torch.stack(streams)) if return_layers else logits

