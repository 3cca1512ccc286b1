"""The Vobisun decoder's configuration.

Its config.json is nested and lists the layers one by one; a span of layers may run several times
in a row with the same weights:

    {"architecture": "Vobisun", "vocab": V, "width": W, "norm": {"eps": e},
     "embedding": {"scale": s}, "canon": {"taps": k},
     "loop": {"start": a, "stop": b, "times": n},
     "layers": [{"type": "parallel",
                 "mixer": {"left": {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": c,
                                    "mask": {"size": w, "pool": P},
                                    "rot": {"base": b, "dims": r, "scaling": {"factor": f}}},
                           "left_scale": x,
                           "right": {"heads": H, "dim": d, "vdim": dv, "tau": t},
                           "right_scale": y},
                 "mlp": {"kind": "dense", "ff": F} | null}, ...]}

Nothing here is a size of one particular model.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Mapping, Optional

from .model_config import ConfigError, ModelConfig, positive_float, positive_int, require_keys


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where}: {key!r} must be an object, found {value!r}")
    return value


def _number(data: Mapping[str, Any], key: str, where: str) -> float:
    value = data.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"{where}: {key!r} must be a number, found {value!r}")
    return float(value)


@dataclass(frozen=True)
class VobisunRotary:
    """Pairs (2i, 2i + 1) of the first `dims` dimensions of a head turn by position * base^(-2i/dims) / factor."""

    base: float
    dims: int
    factor: float = 1.0

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "VobisunRotary":
        require_keys(data, ("base", "dims"), where)
        factor = 1.0
        scaling = data.get("scaling")
        if scaling is not None:
            if not isinstance(scaling, Mapping):
                raise ConfigError(f"{where}: 'scaling' must be an object or null")
            require_keys(scaling, ("factor",), where + ".scaling")
            factor = positive_float(scaling, "factor")
        dims = data["dims"]
        if isinstance(dims, bool) or not isinstance(dims, int) or dims < 0 or dims % 2:
            raise ConfigError(f"{where}: dims must be an even integer >= 0 (0: nothing turns), found {dims!r}")
        return cls(base=positive_float(data, "base"), dims=int(dims), factor=factor)

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            out["scaling"] = {"factor": self.factor}
        return out


@dataclass(frozen=True)
class VobisunLeft:
    """The softmax half of a layer's mixer: a window of tokens and, before it, pooled blocks."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    pool: int
    rot: VobisunRotary

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "VobisunLeft":
        require_keys(data, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"), where)
        mask = _mapping(data, "mask", where)
        require_keys(mask, ("size", "pool"), where + ".mask")
        out = cls(
            heads=positive_int(data, "heads"),
            kv_heads=positive_int(data, "kv_heads"),
            dim=positive_int(data, "dim"),
            vdim=positive_int(data, "vdim"),
            scale=positive_float(data, "scale"),
            window=positive_int(mask, "size"),
            pool=positive_int(mask, "pool"),
            rot=VobisunRotary.from_dict(_mapping(data, "rot", where), where + ".rot"),
        )
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
        if out.rot.dims > out.dim:
            raise ConfigError(f"{where}: rot.dims {out.rot.dims} exceeds dim {out.dim}")
        return out

    def to_dict(self) -> dict[str, Any]:
        return {
            "heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
            "mask": {"size": self.window, "pool": self.pool}, "rot": self.rot.to_dict(),
        }


@dataclass(frozen=True)
class VobisunRight:
    """The recurrent half: linear attention with a decay per key channel, sigmoid(z)^(1/tau)."""

    heads: int
    dim: int
    vdim: int
    tau: float
    # numbers between the two products that make the decay: no config.json key, the shape of the stored
    # tensor `mix.right.a1` [rank, width] (see `VobisunConfig.with_shapes`)
    rank: int = 16

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "VobisunRight":
        require_keys(data, ("heads", "dim", "vdim", "tau"), where)
        return cls(
            heads=positive_int(data, "heads"), dim=positive_int(data, "dim"), vdim=positive_int(data, "vdim"),
            tau=positive_float(data, "tau"),
        )

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


@dataclass(frozen=True)
class VobisunLayer:
    left: VobisunLeft
    right: VobisunRight
    left_scale: float
    right_scale: float
    ff: Optional[int]  # None: the layer has no feed-forward

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "VobisunLayer":
        require_keys(data, ("type", "mixer"), where)
        if data["type"] != "parallel":
            raise ConfigError(f"{where}: unknown mixer type {data['type']!r}; known: parallel")
        mixer = _mapping(data, "mixer", where)
        require_keys(mixer, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
        ff = None
        mlp = data.get("mlp")
        if mlp is not None:
            if not isinstance(mlp, Mapping):
                raise ConfigError(f"{where}: 'mlp' must be an object or null")
            require_keys(mlp, ("kind", "ff"), where + ".mlp")
            if mlp["kind"] != "dense":
                raise ConfigError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; known: dense")
            ff = positive_int(mlp, "ff")
        return cls(
            left=VobisunLeft.from_dict(_mapping(mixer, "left", where), where + ".mixer.left"),
            right=VobisunRight.from_dict(_mapping(mixer, "right", where), where + ".mixer.right"),
            left_scale=_number(mixer, "left_scale", where + ".mixer"),
            right_scale=_number(mixer, "right_scale", where + ".mixer"),
            ff=ff,
        )

    def to_dict(self) -> dict[str, Any]:
        return {
            "type": "parallel",
            "mixer": {
                "left": self.left.to_dict(), "left_scale": self.left_scale,
                "right": self.right.to_dict(), "right_scale": self.right_scale,
            },
            "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff},
        }


@dataclass(frozen=True)
class VobisunConfig(ModelConfig):
    architecture: ClassVar[str] = "Vobisun"
    model_type: ClassVar[str] = "vobisun"

    vocab: int = 0
    width: int = 0
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    canon_taps: int = 1
    layers: tuple[VobisunLayer, ...] = ()
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "VobisunConfig":
        where = "Vobisun"
        require_keys(data, ("vocab", "width", "norm", "embedding", "canon", "layers"), where)
        norm = _mapping(data, "norm", where)
        require_keys(norm, ("eps",), where + ".norm")
        embedding = _mapping(data, "embedding", where)
        require_keys(embedding, ("scale",), where + ".embedding")
        canon = _mapping(data, "canon", where)
        require_keys(canon, ("taps",), where + ".canon")
        layers = data["layers"]
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        start = stop = 0
        times = 1
        loop = data.get("loop")
        if loop is not None:
            if not isinstance(loop, Mapping):
                raise ConfigError(f"{where}: 'loop' must be an object or null")
            require_keys(loop, ("start", "stop", "times"), where + ".loop")
            start, stop, times = loop["start"], loop["stop"], loop["times"]
            for name, value in (("start", start), ("stop", stop), ("times", times)):
                if isinstance(value, bool) or not isinstance(value, int) or value < 0:
                    raise ConfigError(f"{where}.loop: {name!r} must be an integer >= 0, found {value!r}")
            if not (start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"{where}.loop: needs start <= stop <= number of layers and times >= 1")
        return cls(
            vocab=positive_int(data, "vocab"),
            width=positive_int(data, "width"),
            norm_eps=positive_float(norm, "eps"),
            embedding_scale=_number(embedding, "scale", where + ".embedding"),
            canon_taps=positive_int(canon, "taps"),
            layers=tuple(VobisunLayer.from_dict(layer, f"layers[{i}]") for i, layer in enumerate(layers)),
            loop_start=int(start),
            loop_stop=int(stop),
            loop_times=int(times),
        )

    def with_shapes(self, shapes: Mapping[str, tuple]) -> "VobisunConfig":
        """The configuration with the sizes that only the stored tensors give (name -> shape)."""
        from dataclasses import replace

        layers = []
        for i, layer in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.right.a1")
            if shape is not None and len(shape) == 2 and shape[0] != layer.right.rank:
                layer = replace(layer, right=replace(layer.right, rank=int(shape[0])))
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def layer_runs(self) -> list[int]:
        """The layers in the order they run: start .. stop - 1 `times` times in a row."""
        n = len(self.layers)
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))

    def to_dict(self) -> dict[str, Any]:
        return {
            "architecture": self.architecture,
            "vocab": self.vocab,
            "width": self.width,
            "norm": {"eps": self.norm_eps},
            "embedding": {"scale": self.embedding_scale},
            "canon": {"taps": self.canon_taps},
            "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times},
            "layers": [layer.to_dict() for layer in self.layers],
        }
