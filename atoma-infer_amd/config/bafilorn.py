"""Typed configuration of the Bafilorn decoder.

config.json of this design is nested: ``layers`` lists every layer with its ``type`` (which mixer it has:
``latent_attention``, ``lightning`` or ``parallel``), the mixer's sizes and constants (``mixer``) and its feed-forward
(``mlp``, null for a layer without one); ``loop`` names a run of layers that is gone through several times;
``embedding`` holds the embedding's scale and the constants of its table of token pairs; ``streams`` the number of
copies the residual stream is kept in; ``norm.eps``, ``vocab`` and ``width`` stand at the top, and ``architecture``
names the design.  Every layer may have sizes of its own.  The design has no largest position (rotation angles are
worked out from the position); ``max_positions`` (not a key of the design) bounds a request's length for the engine
and defaults to 2^20.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, as_float, as_int, as_positive_int, key, optional, parse_fields
from .morulix import DenseFeedForward, LayerLoop, _eps, _obj


@dataclasses.dataclass(frozen=True)
class ChunkMask:
    """A token sees the keys of its own chunk of ``size`` positions, chunks counted from position 0."""
    size: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mask"):
        return cls(**parse_fields(cls, obj, where))


@dataclasses.dataclass(frozen=True)
class WaveScaling:
    """Slowing the rotation's long waves down (see ``parts.attention.rotation_frequencies``)."""
    factor: float = key(convert=as_float)
    original: float = key(convert=as_float)
    fast: float = key(convert=as_float)
    slow: float = key(convert=as_float)

    @classmethod
    def from_json(cls, obj, where="scaling"):
        s = cls(**parse_fields(cls, obj, where))
        if not (s.factor > 0 and s.original > 0 and s.fast > 0 and s.slow > 0):
            raise ConfigError(f"{where}: factor, original, fast and slow must be positive")
        return s

    def to_dict(self):
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclasses.dataclass(frozen=True)
class Rotation:
    """Rotation of the first ``dims`` columns of a head (or of a head's rotated part)."""
    base: float = key(convert=as_float)
    dims: int = key(convert=as_int)
    scaling: Optional[WaveScaling] = key(default=None, convert=optional(_obj(WaveScaling, "scaling")))

    @classmethod
    def from_json(cls, obj, where="rot"):
        r = cls(**parse_fields(cls, obj, where))
        if r.dims < 0 or r.dims % 2 or not r.base > 0 or r.base == 1.0:
            raise ConfigError(f"{where}: dims must be even and not negative, base positive and not 1")
        return r

    def to_dict(self):
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclasses.dataclass(frozen=True)
class LatentMixer:
    """Attention over a cached latent with a rotated key part shared by the heads and queries through a latent."""
    kind = "latent_attention"
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_rank: int = key(convert=as_positive_int)
    q_rank: int = key(convert=as_positive_int)
    rot_dim: int = key(convert=as_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)
    rot: Optional[Rotation] = key(default=None, convert=optional(_obj(Rotation, "rot")))

    @classmethod
    def from_json(cls, obj, where="mixer"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.rot_dim < 0:
            p.append("rot_dim must not be negative")
        if m.rot is not None and m.rot.dims > m.rot_dim:
            p.append(f"rot_dim {m.rot_dim} cannot hold the {m.rot.dims} rotated columns")
        if m.rot is not None and m.rot.scaling is not None:
            p.append("the rotation of latent attention has no scaling")
        if m.kv_rank + m.rot_dim > 256:
            p.append(f"a cached key of {m.kv_rank + m.rot_dim} columns is more than the attention kernels' 256")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
             "rot_dim": self.rot_dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


def _decays(v: Any) -> Tuple[float, ...]:
    if not isinstance(v, list) or not v:
        raise TypeError("expected a list of one decay per head")
    out = tuple(as_float(x) for x in v)
    if any(not 0.0 <= d <= 1.0 for d in out):
        raise ValueError("decays lie between 0 and 1")
    return out


@dataclasses.dataclass(frozen=True)
class LightningMixer:
    """Linear attention with a fixed decay per head."""
    kind = "lightning"
    decay: Tuple[float, ...] = key(convert=_decays)
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mixer"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if len(m.decay) != m.heads:
            p.append(f"{len(m.decay)} decays for {m.heads} heads")
        if m.dim > 256:
            p.append("dim beyond 256 is not supported")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclasses.dataclass(frozen=True)
class TiedAttentionBranch:
    """Grouped attention whose values are its keys, in chunks, with a sink of score zero."""
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)
    mask: Optional[ChunkMask] = key(default=None, convert=optional(_obj(ChunkMask, "mask")))
    rot: Optional[Rotation] = key(default=None, convert=optional(_obj(Rotation, "rot")))

    @classmethod
    def from_json(cls, obj, where="left"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.heads % m.kv_heads:
            p.append(f"heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        if m.vdim != m.dim:
            p.append(f"values are the keys: vdim {m.vdim} must equal dim {m.dim}")
        if m.rot is not None and m.rot.dims > m.dim:
            p.append(f"dim {m.dim} cannot hold the {m.rot.dims} rotated columns")
        if m.dim > 256:
            p.append("dim beyond 256 is not supported")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim,
                             "scale": self.scale}
        if self.mask is not None:
            d["mask"] = {"size": self.mask.size}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclasses.dataclass(frozen=True)
class RecurrentBranch:
    """A gated linear recurrence per channel behind a short convolution."""
    blocks: int = key(convert=as_positive_int)
    conv: int = key(convert=as_positive_int)
    width: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="right"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.width % m.blocks:
            p.append(f"blocks {m.blocks} does not divide width {m.width}")
        if m.conv > 64:
            p.append("convolutions of more than 64 taps are not supported")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        return {"blocks": self.blocks, "conv": self.conv, "width": self.width}


@dataclasses.dataclass(frozen=True)
class ParallelMixerConfig:
    """Two mixers side by side: attention on the left, a recurrence on the right."""
    kind = "parallel"
    left: TiedAttentionBranch = key(convert=_obj(TiedAttentionBranch, "left"))
    right: RecurrentBranch = key(convert=_obj(RecurrentBranch, "right"))

    @classmethod
    def from_json(cls, obj, where="mixer"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


MIXERS = {c.kind: c for c in (LatentMixer, LightningMixer, ParallelMixerConfig)}


@dataclasses.dataclass(frozen=True)
class BafilornLayer:
    type: str
    mixer: Union[LatentMixer, LightningMixer, ParallelMixerConfig]
    mlp: Optional[DenseFeedForward]

    @classmethod
    def from_json(cls, obj, where):
        if not isinstance(obj, dict) or "type" not in obj or "mixer" not in obj:
            raise ConfigError(f"{where}: a layer needs 'type' and 'mixer'")
        if obj["type"] not in MIXERS:
            raise ConfigError(f"{where}: layer type {obj['type']!r} is not supported (known: {', '.join(sorted(MIXERS))})")
        mlp = obj.get("mlp")
        return cls(obj["type"], MIXERS[obj["type"]].from_json(obj["mixer"], where + ".mixer"),
                   DenseFeedForward.from_json(mlp, where + ".mlp") if mlp is not None else None)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclasses.dataclass(frozen=True)
class PairTable:
    """The second embedding table: row (previous token * mul_prev + token * mul_cur) mod buckets."""
    buckets: int = key(convert=as_positive_int)
    mul_cur: int = key(convert=as_int)
    mul_prev: int = key(convert=as_int)

    @classmethod
    def from_json(cls, obj, where="bigram"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"buckets": self.buckets, "mul_cur": self.mul_cur, "mul_prev": self.mul_prev}


@dataclasses.dataclass(frozen=True)
class EmbeddingConfig:
    scale: float = key(default=1.0, convert=as_float)
    bigram: Optional[PairTable] = key(default=None, convert=optional(_obj(PairTable, "bigram")))

    @classmethod
    def from_json(cls, obj, where="embedding"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        d: Dict[str, Any] = {"scale": self.scale}
        if self.bigram is not None:
            d["bigram"] = self.bigram.to_dict()
        return d


def _layers(v: Any) -> Tuple[BafilornLayer, ...]:
    if not isinstance(v, list) or not v:
        raise ConfigError("layers: expected a list with at least one layer")
    return tuple(BafilornLayer.from_json(x, f"layers[{i}]") for i, x in enumerate(v))


@dataclasses.dataclass(frozen=True)
class BafilornConfig(ModelConfig):
    architectures = ("Bafilorn",)

    layers: Tuple[BafilornLayer, ...] = key(convert=_layers)
    norm_eps: float = key("norm", convert=_eps)
    vocab: int = key(convert=as_positive_int)
    width: int = key(convert=as_positive_int)
    embedding: EmbeddingConfig = key(default=EmbeddingConfig(), convert=_obj(EmbeddingConfig, "embedding"))
    #: copies of the residual stream; None (the key absent): one stream and no connection tensors
    streams: Optional[int] = key(default=None, convert=optional(as_positive_int))
    loop: Optional[LayerLoop] = key(default=None, convert=optional(_obj(LayerLoop, "loop")))
    max_positions: int = key(default=1 << 20, convert=as_positive_int)

    def validate(self, where: str) -> None:
        if self.loop is not None and not 0 <= self.loop.start < self.loop.stop <= len(self.layers):
            raise ConfigError(f"{where}: loop {self.loop.start}..{self.loop.stop} does not lie within the "
                              f"{len(self.layers)} layers")
        if self.streams is not None and self.streams > 8:
            raise ConfigError(f"{where}: more than 8 copies of the stream are not supported")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": "Bafilorn", "embedding": self.embedding.to_dict(),
                             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                             "vocab": self.vocab, "width": self.width}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        return d
