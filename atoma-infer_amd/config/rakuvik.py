"""Typed configuration of the Rakuvik decoder.

config.json of this design is nested: ``layers`` lists every layer with its ``type`` (which mixer it has: ``attention``
or ``mingru``), the mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``: ``kind`` ``dense`` or
``moe``; null for a layer without one); ``norm.eps``, ``vocab`` and ``width`` stand at the top, and ``architecture``
names the design.  Every layer may have sizes of its own.  The design has no largest position; ``max_positions``
(not a key of the design) bounds a request's length for the engine and defaults to 2^20.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, as_float, as_int, as_positive_int, key, optional, parse_fields


def _obj(cls, where: str):
    def conv(v: Any):
        return cls.from_json(v, where)
    return conv


@dataclasses.dataclass(frozen=True)
class LinearScaling:
    """Every frequency of the rotation divided by ``factor``."""
    factor: float = key(convert=as_float)

    @classmethod
    def from_json(cls, obj, where="scaling"):
        s = cls(**parse_fields(cls, obj, where))
        if not s.factor > 0:
            raise ConfigError(f"{where}: factor must be positive")
        return s


@dataclasses.dataclass(frozen=True)
class HalfRotation:
    """Rotation of the first ``dims`` columns of a score map, column c paired with column c + dims/2."""
    base: float = key(convert=as_float)
    dims: int = key(convert=as_int)
    scaling: Optional[LinearScaling] = key(default=None, convert=optional(_obj(LinearScaling, "scaling")))

    @classmethod
    def from_json(cls, obj, where="rot"):
        r = cls(**parse_fields(cls, obj, where))
        if r.dims < 0 or r.dims % 2 or not r.base > 0:
            raise ConfigError(f"{where}: dims must be even and not negative, base positive")
        return r

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = {"factor": self.scaling.factor}
        return d


@dataclasses.dataclass(frozen=True)
class DifferentialMixer:
    """Attention whose heads put out the difference of two softmax maps over one set of values."""
    kind = "attention"
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)
    diff: float = key(convert=as_float)
    rot: Optional[HalfRotation] = key(default=None, convert=optional(_obj(HalfRotation, "rot")))
    kv_from: Optional[int] = key(default=None, convert=optional(as_int))

    @classmethod
    def from_json(cls, obj, where="mixer"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.heads % m.kv_heads:
            p.append(f"heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        if m.rot is not None and m.rot.dims > m.dim:
            p.append(f"dim {m.dim} cannot hold the {m.rot.dims} rotated columns")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "scale": self.scale,
             "diff": self.diff}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d

    def cache_shape(self):
        """What two layers must agree in for one to read the other's keys and values."""
        return (self.dim, self.kv_heads, self.vdim, self.rot)


@dataclasses.dataclass(frozen=True)
class MinGruMixer:
    """A gated recurrence of ``width`` channels whose gates read the current token only."""
    kind = "mingru"
    width: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mixer"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"width": self.width}


MIXERS = {c.kind: c for c in (DifferentialMixer, MinGruMixer)}


@dataclasses.dataclass(frozen=True)
class DenseFeedForward:
    kind = "dense"
    ff: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mlp"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class Router:
    experts: int = key(convert=as_positive_int)
    top: int = key(convert=as_positive_int)
    scale: float = key(default=1.0, convert=as_float)

    @classmethod
    def from_json(cls, obj, where="router"):
        r = cls(**parse_fields(cls, obj, where))
        if r.top > r.experts:
            raise ConfigError(f"{where}: top {r.top} exceeds the {r.experts} experts")
        return r


@dataclasses.dataclass(frozen=True)
class ExpertSize:
    ff: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="expert"):
        return cls(**parse_fields(cls, obj, where))


@dataclasses.dataclass(frozen=True)
class ExpertsFeedForward:
    kind = "moe"
    expert: ExpertSize = key(convert=_obj(ExpertSize, "expert"))
    router: Router = key(convert=_obj(Router, "router"))
    shared: Optional[ExpertSize] = key(default=None, convert=optional(_obj(ExpertSize, "shared")))

    @classmethod
    def from_json(cls, obj, where="mlp"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        d = {"kind": "moe", "expert": {"ff": self.expert.ff},
             "router": {"experts": self.router.experts, "scale": self.router.scale, "top": self.router.top}}
        if self.shared is not None:
            d["shared"] = {"ff": self.shared.ff}
        return d


FEED_FORWARDS = {c.kind: c for c in (DenseFeedForward, ExpertsFeedForward)}


@dataclasses.dataclass(frozen=True)
class RakuvikLayer:
    type: str
    mixer: Union[DifferentialMixer, MinGruMixer]
    mlp: Union[DenseFeedForward, ExpertsFeedForward, None]

    @classmethod
    def from_json(cls, obj, where):
        if not isinstance(obj, dict) or "type" not in obj or "mixer" not in obj:
            raise ConfigError(f"{where}: a layer needs 'type' and 'mixer'")
        if obj["type"] not in MIXERS:
            raise ConfigError(f"{where}: layer type {obj['type']!r} is not supported (known: {', '.join(sorted(MIXERS))})")
        mlp = obj.get("mlp")
        if mlp is not None:
            if not isinstance(mlp, dict) or mlp.get("kind") not in FEED_FORWARDS:
                raise ConfigError(f"{where}.mlp: kind must be one of {', '.join(sorted(FEED_FORWARDS))}")
            mlp = FEED_FORWARDS[mlp["kind"]].from_json(mlp, where + ".mlp")
        return cls(obj["type"], MIXERS[obj["type"]].from_json(obj["mixer"], where + ".mixer"), mlp)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


def _layers(v: Any) -> Tuple[RakuvikLayer, ...]:
    if not isinstance(v, list) or not v:
        raise ConfigError("layers: expected a list with at least one layer")
    return tuple(RakuvikLayer.from_json(x, f"layers[{i}]") for i, x in enumerate(v))


def _eps(v: Any) -> float:
    if not isinstance(v, dict) or "eps" not in v:
        raise ConfigError("norm: expected an object with 'eps'")
    eps = as_float(v["eps"])
    if not eps > 0:
        raise ConfigError("norm.eps must be positive")
    return eps


@dataclasses.dataclass(frozen=True)
class RakuvikConfig(ModelConfig):
    architectures = ("Rakuvik",)

    layers: Tuple[RakuvikLayer, ...] = key(convert=_layers)
    norm_eps: float = key("norm", convert=_eps)
    vocab: int = key(convert=as_positive_int)
    width: int = key(convert=as_positive_int)
    max_positions: int = key(default=1 << 20, convert=as_positive_int)

    def validate(self, where: str) -> None:
        p = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if not isinstance(m, DifferentialMixer) or m.kv_from is None:
                continue
            j = m.kv_from
            if not 0 <= j < i or not isinstance(self.layers[j].mixer, DifferentialMixer) \
                    or self.layers[j].mixer.kv_from is not None:
                p.append(f"layers[{i}]: kv_from {j} must name an earlier attention layer with keys and values of its own")
            elif self.layers[j].mixer.cache_shape() != m.cache_shape():
                p.append(f"layers[{i}]: its key and value sizes or rotation differ from layer {j}'s, whose cache it reads")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": "Rakuvik", "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "vocab": self.vocab, "width": self.width}
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        return d
