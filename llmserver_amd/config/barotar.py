"""Barotar configuration: a nested ``config.json`` that lists the layers one by one.

Top level: ``architecture`` ("Barotar"), ``vocab``, ``width``, ``norm.eps`` and ``layers``.  A layer entry gives
``type`` (its mixer: ``gla`` or ``parallel``), ``mixer`` (the mixer's sizes and constants) and ``mlp`` (``kind``
``dense`` or ``moe`` with its sizes, or null).  Nothing here is a default of the design: every size and constant comes
from the file.  The inner ranks of the decays' low-rank maps are no keys of the file: the checkpoint's tensors have
them; a configuration may name one (``low``) for folders of random weights.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping, Optional, Tuple, Union

from .base import ConfigError, ModelConfig, UnsupportedModelError, field
from .zepolix import _number

MIXERS = ("gla", "parallel")
FEED_FORWARDS = ("dense", "moe")
DEFAULT_LOW_RANK = 16      # what random weights draw where neither the file nor a checkpoint says


def _mapping(where: str, raw, key: str) -> Mapping[str, Any]:
    value = raw.get(key) if isinstance(raw, Mapping) else None
    if not isinstance(value, Mapping):
        raise ConfigError(f"config.json: {where} must give an object {key!r}")
    return value


def _low(where: str, raw: Mapping[str, Any]) -> Optional[int]:
    if "low" not in raw or raw["low"] is None:
        return None
    low = _number(where, raw, "low")
    if low <= 0:
        raise ConfigError(f"config.json: {where}.low must be positive")
    return low


def _positive(where: str, sizes, names) -> None:
    for name in names:
        if getattr(sizes, name) <= 0:
            raise ConfigError(f"config.json: {where}.{name} must be positive")


@dataclasses.dataclass(frozen=True)
class GLASizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    low: Optional[int] = None

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "GLASizes":
        sizes = cls(_number(where, raw, "heads"), _number(where, raw, "dim"), _number(where, raw, "vdim"),
                    _number(where, raw, "tau", float), _low(where, raw))
        _positive(where, sizes, ("heads", "dim", "vdim", "tau"))
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.low is not None:
            out["low"] = self.low
        return out


@dataclasses.dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    rot_base: float
    rot_dims: int
    scale: float
    softcap: float

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "WindowAttentionSizes":
        rot, mask = _mapping(where, raw, "rot"), _mapping(where, raw, "mask")
        sizes = cls(_number(where, raw, "heads"), _number(where, raw, "kv_heads"), _number(where, raw, "dim"), _number(where, raw, "vdim"),
                    _number(where + ".mask", mask, "size"), _number(where + ".rot", rot, "base", float), _number(where + ".rot", rot, "dims"),
                    _number(where, raw, "scale", float), _number(where, raw, "softcap", float))
        _positive(where, sizes, ("heads", "kv_heads", "dim", "vdim", "window", "rot_base", "softcap"))
        if sizes.heads % sizes.kv_heads:
            raise ConfigError(f"config.json: {where}: {sizes.heads} query heads are no multiple of {sizes.kv_heads} key/value heads")
        if sizes.rot_dims < 0 or sizes.rot_dims % 2 or sizes.rot_dims > sizes.dim:
            raise ConfigError(f"config.json: {where}.rot.dims must be an even number up to dim {sizes.dim}, got {sizes.rot_dims}")
        return sizes

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "mask": {"size": self.window},
                "rot": {"base": self.rot_base, "dims": self.rot_dims}, "scale": self.scale, "softcap": self.softcap}


@dataclasses.dataclass(frozen=True)
class TimeMixSizes:
    heads: int
    dim: int
    low: Optional[int] = None

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "TimeMixSizes":
        sizes = cls(_number(where, raw, "heads"), _number(where, raw, "dim"), _low(where, raw))
        _positive(where, sizes, ("heads", "dim"))
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim}
        if self.low is not None:
            out["low"] = self.low
        return out


@dataclasses.dataclass(frozen=True)
class ParallelSizes:
    left: WindowAttentionSizes
    right: TimeMixSizes
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "ParallelSizes":
        return cls(WindowAttentionSizes.read(where + ".left", _mapping(where, raw, "left")),
                   TimeMixSizes.read(where + ".right", _mapping(where, raw, "right")),
                   _number(where, raw, "left_scale", float), _number(where, raw, "right_scale", float))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale, "right_scale": self.right_scale}


@dataclasses.dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class GroupedExpertsSizes:
    ff: int
    limit: float
    experts: int
    top: int
    groups: int
    keep: int

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "GroupedExpertsSizes":
        expert, router = _mapping(where, raw, "expert"), _mapping(where, raw, "router")
        groups = _mapping(where + ".router", router, "groups")
        sizes = cls(_number(where + ".expert", expert, "ff"), _number(where + ".expert", expert, "limit", float),
                    _number(where + ".router", router, "experts"), _number(where + ".router", router, "top"),
                    _number(where + ".router.groups", groups, "count"), _number(where + ".router.groups", groups, "keep"))
        _positive(where, sizes, ("ff", "limit", "experts", "top", "groups", "keep"))
        if sizes.experts % sizes.groups or sizes.keep > sizes.groups:
            raise ConfigError(f"config.json: {where}: {sizes.experts} experts in {sizes.groups} equal groups of which {sizes.keep} are kept")
        if sizes.top > sizes.keep * (sizes.experts // sizes.groups):
            raise ConfigError(f"config.json: {where}: a token uses {sizes.top} experts, the kept groups hold {sizes.keep * (sizes.experts // sizes.groups)}")
        return sizes

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}


@dataclasses.dataclass(frozen=True)
class BarotarLayer:
    type: str
    mixer: Union[GLASizes, ParallelSizes]
    mlp: Union[None, DenseSizes, GroupedExpertsSizes]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclasses.dataclass(frozen=True)
class BarotarConfig(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "Barotar"

    vocab: int = field("vocab", int)
    width: int = field("width", int)
    norm: object = field("norm", object)
    layers_raw: object = field("layers", object)
    layers: Tuple[BarotarLayer, ...] = ()
    norm_eps: float = 0.0

    def resolve(self, raw: Mapping[str, Any]) -> "BarotarConfig":
        if not isinstance(self.layers_raw, (list, tuple)) or not self.layers_raw:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        layers = []
        for index, entry in enumerate(self.layers_raw):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping) or not isinstance(entry.get("type"), str):
                raise ConfigError(f"config.json: {where} must be an object with a 'type'")
            kind = entry["type"]
            if kind not in MIXERS:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the mixer {kind!r}; built: {', '.join(MIXERS)}")
            sizes = _mapping(where, entry, "mixer")
            mixer = GLASizes.read(where + ".mixer", sizes) if kind == "gla" else ParallelSizes.read(where + ".mixer", sizes)
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") not in FEED_FORWARDS:
                    named = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                    raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the feed-forward {named!r}; built: {', '.join(FEED_FORWARDS)}")
                if mlp["kind"] == "dense":
                    mlp = DenseSizes(_number(where + ".mlp", mlp, "ff"))
                    if mlp.ff <= 0:
                        raise ConfigError(f"config.json: {where}.mlp.ff must be positive")
                else:
                    mlp = GroupedExpertsSizes.read(where + ".mlp", mlp)
            layers.append(BarotarLayer(kind, mixer, mlp))
        return dataclasses.replace(self, layers=tuple(layers), norm_eps=_number("norm", self.norm, "eps", float))

    def validate(self, raw: Mapping[str, Any]) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"vocab and width must be positive: {self.vocab}, {self.width}")
        if self.norm_eps <= 0.0:
            raise ConfigError(f"norm.eps must be positive: {self.norm_eps}")
        for index, layer in enumerate(self.layers):
            if isinstance(layer.mixer, ParallelSizes) and max(layer.mixer.left.dim, layer.mixer.left.vdim) > 256:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] has attention heads of "
                                            f"{layer.mixer.left.dim} / {layer.mixer.left.vdim}; the attention kernels take heads of up to 256")

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
        return {"architecture": self.MODEL_TYPE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "layers": [layer.to_dict() for layer in self.layers]}
