"""The Pepulix decoder's configuration.

Its config.json is nested and lists the layers one by one, each with a mixer of its own kind and sizes and a
feed-forward of its own kind (or none):

    {"architecture": "Pepulix", "vocab": V, "width": W, "norm": {"eps": e}, "streams": S, "logit_softcap": c,
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": c, "v_mix": true,
                           "rot": {"base": b, "dims": r}},
                 "mlp": {"kind": "dense", "ff": F}},
                {"type": "latent_attention",
                 "mixer": {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": R, "q_rank": Q, "scale": c,
                           "rot": {"base": b, "dims": r, "scaling": {"factor": f, "original": n, "fast": a, "slow": z}}},
                 "mlp": {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "identity": I, "top": k}}},
                {"type": "mlstm", "mixer": {"heads": H, "dim": d, "vdim": dv, "gate_cap": c}, "mlp": null}, ...]}

`streams` (optional) is the number of residual streams the layers keep; `logit_softcap` (optional) caps the
logits.  Nothing here is a size of one particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Mapping, Optional

from .bubitar import Rotary, _mapping
from .model_config import ConfigError, ModelConfig, positive_float, positive_int, require_keys


def _optional_int(data: Mapping[str, Any], key: str, where: str, least: int = 0) -> Optional[int]:
    value = data.get(key)
    if value is None:
        return None
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise ConfigError(f"{where}: {key!r} must be an integer >= {least} or absent, found {value!r}")
    return int(value)


@dataclass(frozen=True)
class PepulixAttention:
    """Grouped heads, biased projections, unit norms of q, k and v per head, sigmoid weights, a gate per head."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotary] = None
    v_mix: bool = False

    kind: ClassVar[str] = "attention"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "PepulixAttention":
        require_keys(data, ("heads", "dim", "vdim", "scale"), where)
        rot = data.get("rot")
        out = cls(
            heads=positive_int(data, "heads"),
            kv_heads=positive_int(data, "kv_heads") if data.get("kv_heads") is not None else positive_int(data, "heads"),
            dim=positive_int(data, "dim"),
            vdim=positive_int(data, "vdim"),
            scale=positive_float(data, "scale"),
            rot=None if rot is None else Rotary.from_dict(_mapping(data, "rot", where), where + ".rot"),
            v_mix=bool(data.get("v_mix", False)),
        )
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads are no multiple of {out.kv_heads} kv_heads")
        if out.rot is not None and out.rot.dims > out.dim:
            raise ConfigError(f"{where}: more rotated dimensions than a head has")
        if out.rot is not None and out.rot.scaling is not None:
            raise ConfigError(f"{where}: this mixer's rotation has no scaling")
        return out

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
        }
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.v_mix:
            out["v_mix"] = True
        return out


@dataclass(frozen=True)
class PepulixLatentAttention:
    """Queries through a latent of their own; keys and values from one cached latent per token."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Rotary

    kind: ClassVar[str] = "latent_attention"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "PepulixLatentAttention":
        require_keys(data, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot"), where)
        out = cls(
            heads=positive_int(data, "heads"),
            dim=positive_int(data, "dim"),
            rot_dim=positive_int(data, "rot_dim"),
            vdim=positive_int(data, "vdim"),
            kv_rank=positive_int(data, "kv_rank"),
            q_rank=positive_int(data, "q_rank"),
            scale=positive_float(data, "scale"),
            rot=Rotary.from_dict(_mapping(data, "rot", where), where + ".rot"),
        )
        if out.rot.dims > out.rot_dim:
            raise ConfigError(f"{where}: more rotated dimensions than the rotated part has")
        return out

    def to_dict(self) -> dict[str, Any]:
        return {
            "heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
            "q_rank": self.q_rank, "scale": self.scale, "rot": self.rot.to_dict(),
        }


@dataclass(frozen=True)
class PepulixMemory:
    """A matrix memory per head with exponential gates."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    kind: ClassVar[str] = "mlstm"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "PepulixMemory":
        require_keys(data, ("heads", "dim", "vdim", "gate_cap"), where)
        return cls(
            heads=positive_int(data, "heads"), dim=positive_int(data, "dim"), vdim=positive_int(data, "vdim"),
            gate_cap=positive_float(data, "gate_cap"),
        )

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


_MIXERS = {c.kind: c for c in (PepulixAttention, PepulixLatentAttention, PepulixMemory)}


@dataclass(frozen=True)
class PepulixFeedForward:
    """kind "dense": down(silu(gate(x)) * up(x)) with biases, inner size `ff`.  kind "moe": `experts` such
    feed-forwards of inner size `ff` without biases and `identity` more that hand their input on, of which a
    token uses `top`."""

    kind: str
    ff: int
    experts: int = 0
    identity: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "PepulixFeedForward":
        require_keys(data, ("kind",), where)
        if data["kind"] == "dense":
            require_keys(data, ("ff",), where)
            return cls("dense", positive_int(data, "ff"))
        if data["kind"] != "moe":
            raise ConfigError(f"{where}: kind must be 'dense' or 'moe', found {data['kind']!r}")
        require_keys(data, ("expert", "router"), where)
        expert = _mapping(data, "expert", where)
        router = _mapping(data, "router", where)
        require_keys(expert, ("ff",), where + ".expert")
        require_keys(router, ("experts", "top"), where + ".router")
        out = cls(
            "moe", positive_int(expert, "ff"), experts=positive_int(router, "experts"),
            identity=_optional_int(router, "identity", where + ".router") or 0, top=positive_int(router, "top"),
        )
        if out.top > out.experts + out.identity:
            raise ConfigError(f"{where}: a token uses more experts than there are")
        return out

    def to_dict(self) -> dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router: dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.identity:
            router["identity"] = self.identity
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": router}


@dataclass(frozen=True)
class PepulixLayer:
    mixer: Any  # one of the three mixer configurations
    mlp: Optional[PepulixFeedForward]

    def to_dict(self) -> dict[str, Any]:
        return {"type": self.mixer.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class PepulixConfig(ModelConfig):
    architecture: ClassVar[str] = "Pepulix"
    model_type: ClassVar[str] = "pepulix"

    vocab: int
    width: int
    norm_eps: float
    layers: tuple[PepulixLayer, ...]
    streams: Optional[int] = None  # None: one residual stream with plain additions
    logit_softcap: Optional[float] = None

    def __post_init__(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("PepulixConfig: vocab and width must be > 0")
        if not self.layers:
            raise ConfigError("PepulixConfig: a model needs at least one layer")
        if not self.norm_eps >= 0:
            raise ConfigError("PepulixConfig: norm.eps must be >= 0")
        if self.streams is not None and not 0 < self.streams <= 16:
            raise ConfigError("PepulixConfig: streams must be within 1..16 or absent")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError("PepulixConfig: logit_softcap must be > 0 or absent")
        shared = {
            (layer.mixer.kv_heads, layer.mixer.vdim)
            for layer in self.layers
            if isinstance(layer.mixer, PepulixAttention) and layer.mixer.v_mix
        }
        if len(shared) > 1:
            raise ConfigError("PepulixConfig: layers that mix values must agree in kv_heads and vdim")

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "PepulixConfig":
        require_keys(data, ("vocab", "width", "norm", "layers"), "PepulixConfig")
        norm = _mapping(data, "norm", "PepulixConfig")
        require_keys(norm, ("eps",), "PepulixConfig.norm")
        eps = norm["eps"]
        if isinstance(eps, bool) or not isinstance(eps, (int, float)) or not eps >= 0:
            raise ConfigError(f"norm.eps must be a number >= 0, found {eps!r}")
        listed = data["layers"]
        if not isinstance(listed, (list, tuple)):
            raise ConfigError("PepulixConfig: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{where} must be an object")
            require_keys(entry, ("type", "mixer"), where)
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}: unknown mixer type {entry['type']!r}; known: {', '.join(sorted(_MIXERS))}")
            mixer = _MIXERS[entry["type"]].from_dict(_mapping(entry, "mixer", where), where + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None and not isinstance(mlp, Mapping):
                raise ConfigError(f"{where}: 'mlp' must be an object or null")
            layers.append(PepulixLayer(mixer, None if mlp is None else PepulixFeedForward.from_dict(mlp, where + ".mlp")))
        cap = data.get("logit_softcap")
        if cap is not None and (isinstance(cap, bool) or not isinstance(cap, (int, float)) or not cap > 0):
            raise ConfigError(f"logit_softcap must be a number > 0 or absent, found {cap!r}")
        return cls(
            vocab=positive_int(data, "vocab"),
            width=positive_int(data, "width"),
            norm_eps=float(eps),
            layers=tuple(layers),
            streams=_optional_int(data, "streams", "PepulixConfig", least=1),
            logit_softcap=None if cap is None else float(cap),
        )

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.streams is not None:
            out["streams"] = self.streams
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out
