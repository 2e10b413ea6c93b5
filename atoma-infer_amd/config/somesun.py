"""Typed configuration of the Somesun decoder.

config.json of this design is nested: ``layers`` lists every layer with its ``type`` (which mixer it has), the
mixer's sizes and constants (``mixer``) and its feed-forward (``mlp``, null for a layer without one); ``norm.eps``,
``vocab`` and ``width`` stand at the top, and ``architecture`` names the design.  Every layer may have sizes of its
own.  The design has no largest position; ``max_positions`` (not a key of the design) bounds a request's length for the
engine and defaults to 2^20.

The sizes that config.json does not give (the inner sizes of the recurrent mixer's two low-rank maps) are the
checkpoint's; ``decay_rank`` / ``gate_rank`` may name them for the random-weights mode.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, as_float, as_int, as_positive_int, key, optional, parse_fields


def _obj(cls, where: str):
    def conv(v: Any):
        return cls.from_json(v, where)
    return conv


@dataclasses.dataclass(frozen=True)
class ChunkMask:
    size: int = key(convert=as_positive_int)

    @classmethod
    def from_json(cls, obj, where="mask"):
        return cls(**parse_fields(cls, obj, where))


@dataclasses.dataclass(frozen=True)
class PairRotation:
    base: float = key(convert=as_float)
    dims: int = key(convert=as_int)       # 0: nothing is rotated

    @classmethod
    def from_json(cls, obj, where="rot"):
        r = cls(**parse_fields(cls, obj, where))
        if r.dims < 0 or r.dims % 2 or not r.base > 0:
            raise ConfigError(f"{where}: dims must be even and not negative, base positive")
        return r


@dataclasses.dataclass(frozen=True)
class LeftMixer:
    """The attention branch: chunked mask, a sink per head, values tied to the keys."""
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    scale: float = key(convert=as_float)
    mask: ChunkMask = key(convert=_obj(ChunkMask, "mask"))
    rot: PairRotation = key(convert=_obj(PairRotation, "rot"))

    @classmethod
    def from_json(cls, obj, where="left"):
        m = cls(**parse_fields(cls, obj, where))
        p = []
        if m.heads % m.kv_heads:
            p.append(f"heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        if m.vdim != m.dim:
            p.append(f"vdim {m.vdim} differs from dim {m.dim}, but the values are the keys")
        if m.dim % 2 or m.rot.dims > m.dim:
            p.append(f"dim {m.dim} must be even and hold the {m.rot.dims} rotated columns")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))
        return m

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim,
                "scale": self.scale, "mask": {"size": self.mask.size},
                "rot": {"base": self.rot.base, "dims": self.rot.dims}}


@dataclasses.dataclass(frozen=True)
class RightMixer:
    """The recurrent branch: gated delta rule behind short convolutions."""
    dim: int = key(convert=as_positive_int)
    heads: int = key(convert=as_positive_int)
    kv_heads: int = key(convert=as_positive_int)
    vdim: int = key(convert=as_positive_int)
    conv: int = key(convert=as_positive_int)
    decay_rank: Optional[int] = key(default=None, convert=optional(as_positive_int))
    gate_rank: Optional[int] = key(default=None, convert=optional(as_positive_int))

    @classmethod
    def from_json(cls, obj, where="right"):
        m = cls(**parse_fields(cls, obj, where))
        if m.heads % m.kv_heads:
            raise ConfigError(f"{where}: heads {m.heads} is not a multiple of kv_heads {m.kv_heads}")
        return m

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "conv": self.conv}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            d["gate_rank"] = self.gate_rank
        return d


@dataclasses.dataclass(frozen=True)
class ParallelMixerConfig:
    left: LeftMixer = key(convert=_obj(LeftMixer, "left"))
    right: RightMixer = key(convert=_obj(RightMixer, "right"))
    left_scale: float = key(convert=as_float)
    right_scale: float = key(convert=as_float)

    @classmethod
    def from_json(cls, obj, where="mixer"):
        return cls(**parse_fields(cls, obj, where))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclasses.dataclass(frozen=True)
class ExpertsConfig:
    kind: str = key(convert=str)
    ff: int = key(default=0)
    experts: int = key(default=0)
    top: int = key(default=0)

    @classmethod
    def from_json(cls, obj, where="mlp"):
        if not isinstance(obj, dict):
            raise ConfigError(f"{where}: expected a JSON object")
        if obj.get("kind") != "moe":
            raise ConfigError(f"{where}: kind {obj.get('kind')!r} is not supported (known: moe)")
        try:
            ff = as_positive_int(obj["expert"]["ff"])
            experts = as_positive_int(obj["router"]["experts"])
            top = as_positive_int(obj["router"]["top"])
        except (KeyError, TypeError, ValueError) as e:
            raise ConfigError(f"{where}: expert.ff, router.experts and router.top are needed ({e})") from None
        if top > experts:
            raise ConfigError(f"{where}: top {top} exceeds the {experts} experts")
        return cls("moe", ff, experts, top)

    def to_dict(self):
        return {"kind": self.kind, "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclasses.dataclass(frozen=True)
class SomesunLayer:
    type: str
    mixer: ParallelMixerConfig
    mlp: Optional[ExpertsConfig]

    @classmethod
    def from_json(cls, obj, where):
        if not isinstance(obj, dict) or "type" not in obj or "mixer" not in obj:
            raise ConfigError(f"{where}: a layer needs 'type' and 'mixer'")
        if obj["type"] != "parallel":
            raise ConfigError(f"{where}: layer type {obj['type']!r} is not supported (known: parallel)")
        mlp = obj.get("mlp")
        return cls("parallel", ParallelMixerConfig.from_json(obj["mixer"], where + ".mixer"),
                   ExpertsConfig.from_json(mlp, where + ".mlp") if mlp is not None else None)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


def _layers(v: Any) -> Tuple[SomesunLayer, ...]:
    if not isinstance(v, list) or not v:
        raise ConfigError("layers: expected a list with at least one layer")
    return tuple(SomesunLayer.from_json(x, f"layers[{i}]") for i, x in enumerate(v))


def _eps(v: Any) -> float:
    if not isinstance(v, dict) or "eps" not in v:
        raise ConfigError("norm: expected an object with 'eps'")
    eps = as_float(v["eps"])
    if not eps > 0:
        raise ConfigError("norm.eps must be positive")
    return eps


@dataclasses.dataclass(frozen=True)
class SomesunConfig(ModelConfig):
    architectures = ("Somesun",)

    layers: Tuple[SomesunLayer, ...] = key(convert=_layers)
    norm_eps: float = key("norm", convert=_eps)
    vocab: int = key(convert=as_positive_int)
    width: int = key(convert=as_positive_int)
    max_positions: int = key(default=1 << 20, convert=as_positive_int)

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": "Somesun", "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "vocab": self.vocab, "width": self.width}
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        return d
