"""Zepolix configuration: a nested ``config.json`` that lists the layers one by one.

Top level: ``architecture`` ("Zepolix"), ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` (the short convolution in
front of every mixer; absent: none) and ``layers``.  A layer entry gives ``type`` (its mixer), ``mixer`` (the mixer's
sizes and constants) and ``mlp`` (its feed-forward, or null).  Nothing here is a default of the design: every size and
constant comes from the file.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, UnsupportedModelError, field

MIXERS = ("latent_attention",)
FEED_FORWARDS = ("moe",)


def _number(where: str, raw: Mapping[str, Any], key: str, kind=int):
    if not isinstance(raw, Mapping) or key not in raw:
        raise ConfigError(f"config.json: {where} must give {key!r}")
    value = raw[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or (kind is int and not isinstance(value, int)):
        raise ConfigError(f"config.json: {where}.{key} must be {'an integer' if kind is int else 'a number'}, got {value!r}")
    return kind(value)


@dataclasses.dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int            # unrotated query/key dimensions of a head
    rot_dim: int        # rotated ones
    vdim: int           # value size of a head
    kv_rank: int        # size of the latent
    scale: float
    rot_base: float
    rot_dims: int

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "LatentAttentionSizes":
        rot = raw.get("rot") if isinstance(raw, Mapping) else None
        sizes = cls(*(_number(where, raw, key) for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank")),
                    _number(where, raw, "scale", float), _number(where + ".rot", rot, "base", float), _number(where + ".rot", rot, "dims"))
        for name in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot_dims"):
            if getattr(sizes, name) <= 0:
                raise ConfigError(f"config.json: {where}.{name} must be positive")
        if sizes.rot_dims % 2 or sizes.rot_dims > sizes.rot_dim:
            raise ConfigError(f"config.json: {where}: {sizes.rot_dims} of {sizes.rot_dim} rotated dimensions turn; that must be an even number of them")
        return sizes

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclasses.dataclass(frozen=True)
class ExpertsSizes:
    ff: int
    experts: int
    top: int

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "ExpertsSizes":
        sizes = cls(_number(where + ".expert", raw.get("expert"), "ff"), _number(where + ".router", raw.get("router"), "experts"),
                    _number(where + ".router", raw.get("router"), "top"))
        if sizes.ff <= 0 or not 1 <= sizes.top <= sizes.experts:
            raise ConfigError(f"config.json: {where}: ff {sizes.ff}, {sizes.top} of {sizes.experts} experts")
        return sizes

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclasses.dataclass(frozen=True)
class ZepolixLayer:
    type: str
    mixer: LatentAttentionSizes
    mlp: Optional[ExpertsSizes]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclasses.dataclass(frozen=True)
class ZepolixConfig(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "Zepolix"

    vocab: int = field("vocab", int)
    width: int = field("width", int)
    norm: object = field("norm", object)
    layers_raw: object = field("layers", object)
    canon: object = field("canon", object, None)
    layers: Tuple[ZepolixLayer, ...] = ()
    norm_eps: float = 0.0
    canon_taps: int = 0          # 0: no convolution in front of the mixers

    def resolve(self, raw: Mapping[str, Any]) -> "ZepolixConfig":
        if not isinstance(self.layers_raw, (list, tuple)) or not self.layers_raw:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        layers = []
        for index, entry in enumerate(self.layers_raw):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping) or not isinstance(entry.get("type"), str):
                raise ConfigError(f"config.json: {where} must be an object with a 'type'")
            if entry["type"] not in MIXERS:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the mixer {entry['type']!r}; built: {', '.join(MIXERS)}")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") not in FEED_FORWARDS:
                    kind = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                    raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the feed-forward {kind!r}; built: {', '.join(FEED_FORWARDS)}")
                mlp = ExpertsSizes.read(where + ".mlp", mlp)
            layers.append(ZepolixLayer(entry["type"], LatentAttentionSizes.read(where + ".mixer", entry.get("mixer")), mlp))
        taps = _number("canon", self.canon, "taps") if self.canon is not None else 0
        return dataclasses.replace(self, layers=tuple(layers), norm_eps=_number("norm", self.norm, "eps", float), canon_taps=taps)

    def validate(self, raw: Mapping[str, Any]) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"vocab and width must be positive: {self.vocab}, {self.width}")
        if self.norm_eps <= 0.0:
            raise ConfigError(f"norm.eps must be positive: {self.norm_eps}")
        if self.canon is not None and self.canon_taps < 1:
            raise ConfigError(f"canon.taps must be at least 1: {self.canon_taps}")
        for index, layer in enumerate(self.layers):
            row = layer.mixer.kv_rank + layer.mixer.rot_dim
            if row > 256:
                raise UnsupportedModelError(
                    f"Model type {self.MODEL_TYPE!r}: layers[{index}] caches {row} numbers a token (kv_rank + rot_dim); the attention "
                    "kernels take rows of up to 256")

    # what the rest of the package asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def to_dict(self) -> dict:
        out = {"architecture": self.MODEL_TYPE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        return out
