"""Typed configuration of the Morulix decoder.

config.json of this design is nested: ``layers`` lists every layer with its ``type`` (which mixer it has:
``attention``, ``latent_attention`` or ``mamba2``), the mixer's sizes and constants (``mixer``) and its feed-forward
(``mlp``, null for a layer without one); ``loop`` names a run of layers that is gone through several times;
``norm.eps``, ``vocab`` and ``width`` stand at the top, and ``architecture`` names the design.  Every layer may have
sizes of its own.  The design has no largest position; ``max_positions`` (not a key of the design) bounds a request's
length for the engine and the table of rotation angles, and defaults to 2^17.
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
class WindowMask:
    """A token sees the last ``size`` keys, its own among them."""
    size: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mask"):
        return cls(**parse_fields(cls, obj, where))


@dataclasses.dataclass(frozen=True)
class BandScaling:
    """Rescaling of the rotation's frequencies by wavelength: kept below ``original / high``, divided by ``factor``
    above ``original / low``, blended between."""
    factor: float = key(convert=as_float)
    low: float = key(convert=as_float)
    high: float = key(convert=as_float)
    original: float = key(convert=as_float)

    @classmethod
    def from_json(cls, obj, where="scaling"):
        s = cls(**parse_fields(cls, obj, where))
        if not (s.factor > 0 and s.original > 0 and s.high > s.low >= 0):
            raise ConfigError(f"{where}: factor and original must be positive and high above low")
        return s

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclasses.dataclass(frozen=True)
class HalfRotation:
    """Rotation of the first ``dims`` columns of a head, column i paired with column i + dims/2."""
    base: float = key(convert=as_float)
    dims: int = key(convert=as_int)
    scaling: Optional[BandScaling] = key(default=None, convert=optional(_obj(BandScaling, "scaling")))

    @classmethod
    def from_json(cls, obj, where="rot"):
        r = cls(**parse_fields(cls, obj, where))
        if r.dims < 0 or r.dims % 2 or not r.base > 0:
            raise ConfigError(f"{where}: dims must be even and not negative, base positive")
        return r

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclasses.dataclass(frozen=True)
class AttentionMixer:
    """Grouped attention with a window and rotated queries and keys."""
    kind = "attention"
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)
    mask: Optional[WindowMask] = key(default=None, convert=optional(_obj(WindowMask, "mask")))
    rot: Optional[HalfRotation] = key(default=None, convert=optional(_obj(HalfRotation, "rot")))

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
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "scale": self.scale}
        if self.mask is not None:
            d["mask"] = {"size": self.mask.size}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclasses.dataclass(frozen=True)
class LatentMixer:
    """Attention whose keys and values are made from one small vector per token."""
    kind = "latent_attention"
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_rank: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)

    @classmethod
    def from_json(cls, obj, where="mixer"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "vdim": self.vdim, "scale": self.scale}


@dataclasses.dataclass(frozen=True)
class StateSpaceMixer:
    """A selective state-space recurrence with a scalar decay per head."""
    kind = "mamba2"
    conv: int = key(convert=as_positive_int)
    groups: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    norm_groups: int = key(convert=as_positive_int)
    state: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mixer"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.heads % m.groups:
            p.append(f"heads {m.heads} is not a multiple of groups {m.groups}")
        if (m.heads * m.vdim) % m.norm_groups:
            p.append(f"norm_groups {m.norm_groups} does not divide the inner width {m.heads * m.vdim}")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


MIXERS = {c.kind: c for c in (AttentionMixer, LatentMixer, StateSpaceMixer)}


@dataclasses.dataclass(frozen=True)
class DenseFeedForward:
    kind: str = key(convert=str)
    ff: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mlp"):
        m = cls(**parse_fields(cls, obj, where))
        if m.kind != "dense":
            raise ConfigError(f"{where}: kind {m.kind!r} is not supported (known: dense)")
        return m

    def to_dict(self):
        return {"kind": self.kind, "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class MorulixLayer:
    type: str
    mixer: Union[AttentionMixer, LatentMixer, StateSpaceMixer]
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
class LayerLoop:
    """Layers ``start`` .. ``stop - 1`` run ``times`` times in a row with the same weights."""
    start: int = key(convert=as_int)
    stop: int = key(convert=as_int)
    times: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="loop"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"start": self.start, "stop": self.stop, "times": self.times}


def _layers(v: Any) -> Tuple[MorulixLayer, ...]:
    if not isinstance(v, list) or not v:
        raise ConfigError("layers: expected a list with at least one layer")
    return tuple(MorulixLayer.from_json(x, f"layers[{i}]") for i, x in enumerate(v))


def _eps(v: Any) -> float:
    if not isinstance(v, dict) or "eps" not in v:
        raise ConfigError("norm: expected an object with 'eps'")
    eps = as_float(v["eps"])
    if not eps > 0:
        raise ConfigError("norm.eps must be positive")
    return eps


@dataclasses.dataclass(frozen=True)
class MorulixConfig(ModelConfig):
    architectures = ("Morulix",)

    layers: Tuple[MorulixLayer, ...] = key(convert=_layers)
    norm_eps: float = key("norm", convert=_eps)
    vocab: int = key(convert=as_positive_int)
    width: int = key(convert=as_positive_int)
    loop: Optional[LayerLoop] = key(default=None, convert=optional(_obj(LayerLoop, "loop")))
    max_positions: int = key(default=1 << 17, convert=as_positive_int)

    def validate(self, where: str) -> None:
        if self.loop is not None and not 0 <= self.loop.start < self.loop.stop <= len(self.layers):
            raise ConfigError(f"{where}: loop {self.loop.start}..{self.loop.stop} does not lie within the "
                              f"{len(self.layers)} layers")

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": "Morulix", "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.max_positions != 1 << 17:
            d["max_positions"] = self.max_positions
        return d
