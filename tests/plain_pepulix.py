"""The Pepulix decoder, plainly: whole sequences, no cache, no carried state, float64, one function per
mechanism.  It shares no code with the engine and exists to be compared with it.

`config` is the decoder's config.json as a dict, `weights` a dict of float64 tensors under the
checkpoint's own names.  The `round_to` argument of `forward` makes the yardstick for ill-conditioned rows:
the same arithmetic with every product's inputs rounded to bfloat16.
"""

from __future__ import annotations

import math
from typing import Mapping, Optional

import torch

F64 = torch.float64


def _r(x, round_to):
    return x if round_to is None else x.to(round_to).to(F64)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---- rotations ------------------------------------------------------------------------------------------

def rotary_frequencies(rot: Mapping) -> tuple[torch.Tensor, float]:
    """Turning rates of the dims/2 pairs and the amplitude of cos and sin."""
    dims = int(rot["dims"])
    base = float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return f, 1.0
    factor = float(scaling["factor"])

    def pair_of(turns: float) -> float:
        return dims * math.log(float(scaling["original"]) / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: Mapping, layout: str) -> torch.Tensor:
    """x [T, heads, d]: the first rot.dims dims of every head turn, the rest pass.  layout "halves": dim i
    with i + dims/2; "pairs": dim 2i with 2i + 1."""
    dims = int(rot["dims"])
    f, amplitude = rotary_frequencies(rot)
    angle = positions.to(F64)[:, None] * f[None, :]  # [T, dims/2]
    cos = (torch.cos(angle) * amplitude)[:, None, :]
    sin = (torch.sin(angle) * amplitude)[:, None, :]
    out = x.clone()
    if layout == "halves":
        u, v = x[..., : dims // 2], x[..., dims // 2 : dims]
        out[..., : dims // 2] = u * cos - v * sin
        out[..., dims // 2 : dims] = v * cos + u * sin
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---- mixers ---------------------------------------------------------------------------------------------

def sigmoid_attention(w, p: str, m: Mapping, h: torch.Tensor, eps: float, shared: dict, round_to=None) -> torch.Tensor:
    """Grouped heads, biased projections, rotation of halves, unit norms of q, k and v, sigmoid weights."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    hr = _r(h, round_to)
    q = (hr @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = (hr @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = (hr @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    pos = torch.arange(T)
    if m.get("rot"):
        q = rotate(q, pos, m["rot"], "halves")
        k = rotate(k, pos, m["rot"], "halves")
    q, k, v = unit_rms(q, eps), unit_rms(k, eps), unit_rms(v, eps)
    if m.get("v_mix"):
        if "first_values" in shared:
            lam = w[p + "vmix"]
            v = (1.0 - lam) * v + lam * shared["first_values"]
        else:
            shared["first_values"] = v
    q, k, v = _r(q, round_to), _r(k, round_to), _r(v, round_to)
    out = torch.zeros(T, H, dv, dtype=F64)
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for head in range(H):
        g = head // (H // G)
        score = (q[:, head] @ k[:, g].T) * float(m["scale"]) + w[p + "pb"][head]
        weight = torch.sigmoid(score) * seen
        out[:, head] = weight @ v[:, g]
    gate = torch.sigmoid(hr @ w[p + "g"].T)  # [T, H]
    out = out * gate[:, :, None]
    return _r(out.reshape(T, H * dv), round_to) @ w[p + "o"].T


def latent_attention(w, p: str, m: Mapping, h: torch.Tensor, eps: float, round_to=None) -> torch.Tensor:
    """Queries through a normed latent; keys and values from one normed latent per token beside one rotated
    key part that all heads share; softmax."""
    T = h.shape[0]
    H, d, r, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    hr = _r(h, round_to)
    cq = rms_norm(hr @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (_r(cq, round_to) @ w[p + "uq"].T).view(T, H, d + r)
    down = hr @ w[p + "dkv"].T
    c = _r(rms_norm(down[:, :R], w[p + "dkv.norm"], eps), round_to)
    pos = torch.arange(T)
    key_rot = rotate(down[:, None, R:], pos, m["rot"], "pairs")[:, 0]  # [T, r]
    q_rot = rotate(q[..., d:], pos, m["rot"], "pairs")
    k_plain = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    hidden = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    for head in range(H):
        score = (q[:, head, :d] @ k_plain[:, head].T + q_rot[:, head] @ key_rot.T) * float(m["scale"])
        score = score.masked_fill(hidden, -math.inf)
        out[:, head] = torch.softmax(score, -1) @ v[:, head]
    return _r(out.reshape(T, H * dv), round_to) @ w[p + "o"].T


def mlstm(w, p: str, m: Mapping, h: torch.Tensor, eps: float, round_to=None) -> torch.Tensor:
    """Matrix memory with exponential input gate, sigmoid forget gate and a running maximum that starts at 0."""
    T = h.shape[0]
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    hr = _r(h, round_to)
    q = (hr @ w[p + "q"].T).view(T, H, d) * d**-0.5
    k = (hr @ w[p + "k"].T).view(T, H, d)
    v = (hr @ w[p + "v"].T).view(T, H, dv)
    log_in = cap * torch.tanh((hr @ w[p + "i"].T + w[p + "i.b"]) / cap)  # [T, H]
    log_keep = torch.nn.functional.logsigmoid(cap * torch.tanh((hr @ w[p + "f"].T + w[p + "f.b"]) / cap))
    out = torch.zeros(T, H, dv, dtype=F64)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        n = torch.zeros(d, dtype=F64)
        top = 0.0
        for t in range(T):
            f, i = float(log_keep[t, head]), float(log_in[t, head])
            new_top = max(f + top, i)
            S = math.exp(f + top - new_top) * S + math.exp(i - new_top) * torch.outer(k[t, head], v[t, head])
            n = math.exp(f + top - new_top) * n + math.exp(i - new_top) * k[t, head]
            top = new_top
            denominator = max(abs(float(n @ q[t, head])), math.exp(-top)) + 1e-6
            out[t, head] = (S.T @ q[t, head]) / denominator
    out = unit_rms(out, eps).reshape(T, H * dv) * w[p + "norm"]
    out = out * torch.sigmoid(hr @ w[p + "g"].T)
    return _r(out, round_to) @ w[p + "o"].T


# ---- feed-forwards --------------------------------------------------------------------------------------

def dense_ff(w, p: str, h: torch.Tensor, round_to=None) -> torch.Tensor:
    hr = _r(h, round_to)
    inner = silu(hr @ w[p + "gate"].T + w[p + "gate.b"]) * (hr @ w[p + "up"].T + w[p + "up.b"])
    return _r(inner, round_to) @ w[p + "down"].T + w[p + "down.b"]


def route(w, p: str, mlp: Mapping, h: torch.Tensor, notes: Optional[dict] = None):
    """ids [T, top] and weights [T, top] of the chosen experts.  `notes["margins"]` receives, per token, by how
    much the last chosen expert's choice score leads the first one left out (a close call is a coin flip once
    anything is rounded)."""
    top = int(mlp["router"]["top"])
    s = torch.softmax(h @ w[p + "router"].T, -1)
    choice = s + w[p + "correction"]
    ids = torch.topk(choice, top, dim=-1).indices
    if notes is not None and choice.shape[-1] > top:
        ranked = choice.sort(-1, descending=True).values
        notes.setdefault("margins", []).append(ranked[:, top - 1] - ranked[:, top])
    chosen = torch.gather(s, 1, ids)
    return ids, chosen / (chosen.sum(-1, keepdim=True) + 1e-20)


def expert_ff(w, p: str, h: torch.Tensor, round_to=None) -> torch.Tensor:
    inner = silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)
    return _r(inner, round_to) @ w[p + "down"].T


def moe_ff(w, p: str, mlp: Mapping, h: torch.Tensor, round_to=None, notes: Optional[dict] = None) -> torch.Tensor:
    real = int(mlp["router"]["experts"])
    hr = _r(h, round_to)
    ids, weights = route(w, p, mlp, hr, notes)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), weights[t]):
            out[t] += a * (hr[t] if e >= real else expert_ff(w, f"{p}e{e}.", hr[t : t + 1], round_to)[0])
    return out


def feed_forward(w, p: str, mlp: Mapping, h: torch.Tensor, round_to=None, notes: Optional[dict] = None) -> torch.Tensor:
    return dense_ff(w, p, h, round_to) if mlp["kind"] == "dense" else moe_ff(w, p, mlp, h, round_to, notes)


# ---- the model ------------------------------------------------------------------------------------------

def forward(
    config: Mapping, weights: Mapping[str, torch.Tensor], tokens, round_to: Optional[torch.dtype] = None,
    notes: Optional[dict] = None,
):
    """logits [T, vocab] and the stream after every layer [layers, T, width] (the sum of the streams).  `notes`
    (a dict) receives what a comparison may want to know besides (see `route`)."""
    w = weights
    eps = float(config["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    streams = config.get("streams")
    xs = [x0.clone() for _ in range(int(streams) if streams else 1)]
    shared: dict = {}
    after = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        for q, what in ((1, layer["type"]), (2, layer.get("mlp"))):
            if what is None:
                continue
            if streams:
                u = sum(w[f"{p}hc{q}.in"][s] * xs[s] for s in range(len(xs)))
            else:
                u = xs[0]
            h = rms_norm(u, w[f"{p}norm{q}"], eps)
            if q == 2:
                y = feed_forward(w, p + "mlp.", what, h, round_to, notes)
            elif what == "attention":
                y = sigmoid_attention(w, p + "mix.", layer["mixer"], h, eps, shared, round_to)
            elif what == "latent_attention":
                y = latent_attention(w, p + "mix.", layer["mixer"], h, eps, round_to)
            elif what == "mlstm":
                y = mlstm(w, p + "mix.", layer["mixer"], h, eps, round_to)
            else:
                raise ValueError(f"unknown mixer {what!r}")
            if streams:
                mix, out = w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"]
                xs = [sum(mix[s, t] * xs[s] for s in range(len(xs))) + out[t] * y for t in range(len(xs))]
            else:
                xs = [xs[0] + y]
        after.append(sum(xs))
    x = rms_norm(sum(xs), w["final.norm"], eps)
    logits = _r(x, round_to) @ w["embed"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits, torch.stack(after)
