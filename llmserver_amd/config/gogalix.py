"""Gogalix configuration: a nested ``config.json`` that lists the layers one by one.

Top level: ``architecture`` ("Gogalix"), ``vocab``, ``width``, ``norm.eps``, ``layers`` and, optional, ``embedding.scale``
(what the embedding rows are multiplied by).  A layer entry gives ``type`` (its mixer: ``attention``, ``delta`` or
``channel_delta``), ``mixer`` (the mixer's sizes and constants) and ``mlp`` (``kind`` ``dense`` with ``ff``, ``kind``
``moe`` with ``expert.ff`` and ``router.{experts, top}``, or null).  An attention mixer gives ``heads``, ``kv_heads``,
``dim``, ``vdim``, ``scale``, ``diff``, ``mask.size`` (absent: every earlier key is seen) and possibly ``kv_from``, the layer
whose keys and values it reads instead of having its own.  A delta mixer gives ``heads``, ``kv_heads``, ``dim``,
``vdim`` and ``conv`` (the taps of its short convolutions).  The inner sizes of the low-rank maps of ``channel_delta``
are no keys of the file: the checkpoint's tensors have them (``low`` and ``gate_low`` may name them for folders of random
weights).  Nothing here is a default of the design: what the file does not name is not there.
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping, Optional, Tuple, Union

from .barotar import _mapping, _positive
from .base import ConfigError, ModelConfig, UnsupportedModelError, field
from .kerudra import _window
from .zepolix import _number

MIXERS = ("attention", "delta", "channel_delta")
FEED_FORWARDS = ("dense", "moe")
MOST_HEAD = 256             # the widest head the attention kernels take, and the most key channels of the delta kernels


def _optional_number(where: str, raw: Mapping[str, Any], key: str) -> Optional[int]:
    if key not in raw or raw[key] is None:
        return None
    value = _number(where, raw, key)
    if value <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be positive")
    return value


def _grouped(where: str, heads: int, kv_heads: int) -> None:
    if heads % kv_heads:
        raise ConfigError(f"config.json: {where}: {heads} heads are no multiple of {kv_heads} key heads")


@dataclasses.dataclass(frozen=True)
class DifferentialAttentionSizes:
    """Two softmax maps a head over the same values, their difference normed per head; windowed, unrotated."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: Optional[int]
    kv_from: Optional[int]

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "DifferentialAttentionSizes":
        heads = _number(where, raw, "heads")
        kv_from = None
        if raw.get("kv_from") is not None:
            kv_from = _number(where, raw, "kv_from")
        sizes = cls(heads, _number(where, raw, "kv_heads") if "kv_heads" in raw else heads, _number(where, raw, "dim"),
                    _number(where, raw, "vdim"), _number(where, raw, "scale", float), _number(where, raw, "diff", float),
                    _window(where, raw), kv_from)
        _positive(where, sizes, ("heads", "kv_heads", "dim", "vdim"))
        _grouped(where, sizes.heads, sizes.kv_heads)
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale, "diff": self.diff}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclasses.dataclass(frozen=True)
class DeltaSizes:
    """A gated delta rule; ``per_channel``: the decay is one number per head and key channel (through a low-rank map)
    and the output gate a sigmoid of a low-rank map, instead of one decay per head and a silu gate."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int
    per_channel: bool = False
    low: Optional[int] = None
    gate_low: Optional[int] = None

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any], per_channel: bool) -> "DeltaSizes":
        heads = _number(where, raw, "heads")
        sizes = cls(heads, _number(where, raw, "kv_heads") if "kv_heads" in raw else heads, _number(where, raw, "dim"),
                    _number(where, raw, "vdim"), _number(where, raw, "conv"), per_channel,
                    _optional_number(where, raw, "low"), _optional_number(where, raw, "gate_low"))
        _positive(where, sizes, ("heads", "kv_heads", "dim", "vdim", "taps"))
        _grouped(where, sizes.heads, sizes.kv_heads)
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.taps}
        if self.low is not None:
            out["low"] = self.low
        if self.gate_low is not None:
            out["gate_low"] = self.gate_low
        return out


@dataclasses.dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class RoutedSizes:
    ff: int
    experts: int
    top: int

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclasses.dataclass(frozen=True)
class GogalixLayer:
    type: str
    mixer: Union[DifferentialAttentionSizes, DeltaSizes]
    mlp: Union[DenseSizes, RoutedSizes, None]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclasses.dataclass(frozen=True)
class GogalixConfig(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "Gogalix"

    vocab: int = field("vocab", int)
    width: int = field("width", int)
    norm: object = field("norm", object)
    layers_raw: object = field("layers", object)
    embedding: object = field("embedding", object, None)
    layers: Tuple[GogalixLayer, ...] = ()
    norm_eps: float = 0.0
    embedding_scale: float = 1.0

    def resolve(self, raw: Mapping[str, Any]) -> "GogalixConfig":
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
            if kind == "attention":
                mixer = DifferentialAttentionSizes.read(where + ".mixer", sizes)
            else:
                mixer = DeltaSizes.read(where + ".mixer", sizes, kind == "channel_delta")
            layers.append(GogalixLayer(kind, mixer, self._feed_forward(where, entry.get("mlp"))))
        scale = 1.0
        if self.embedding is not None:
            if not isinstance(self.embedding, Mapping):
                raise ConfigError("config.json: 'embedding' must be an object")
            if "scale" in self.embedding:
                scale = _number("embedding", self.embedding, "scale", float)
        return dataclasses.replace(self, layers=tuple(layers), norm_eps=_number("norm", self.norm, "eps", float), embedding_scale=scale)

    def _feed_forward(self, where: str, mlp):
        if mlp is None:
            return None
        if not isinstance(mlp, Mapping) or mlp.get("kind") not in FEED_FORWARDS:
            named = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
            raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the feed-forward {named!r}; built: {', '.join(FEED_FORWARDS)}")
        if mlp["kind"] == "dense":
            sizes = DenseSizes(_number(where + ".mlp", mlp, "ff"))
            _positive(where + ".mlp", sizes, ("ff",))
            return sizes
        router = _mapping(where + ".mlp", mlp, "router")
        sizes = RoutedSizes(_number(where + ".mlp.expert", _mapping(where + ".mlp", mlp, "expert"), "ff"),
                            _number(where + ".mlp.router", router, "experts"), _number(where + ".mlp.router", router, "top"))
        _positive(where + ".mlp", sizes, ("ff", "experts", "top"))
        if sizes.top > sizes.experts:
            raise ConfigError(f"config.json: {where}.mlp: a token cannot use {sizes.top} of {sizes.experts} experts")
        return sizes

    def validate(self, raw: Mapping[str, Any]) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"vocab and width must be positive: {self.vocab}, {self.width}")
        if self.norm_eps <= 0.0:
            raise ConfigError(f"norm.eps must be positive: {self.norm_eps}")
        for index, layer in enumerate(self.layers):
            sizes = layer.mixer
            if isinstance(sizes, DifferentialAttentionSizes):
                if max(sizes.dim, sizes.vdim) > MOST_HEAD:
                    raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] has attention heads of {sizes.dim} / "
                                                f"{sizes.vdim}; the attention kernels take heads of up to {MOST_HEAD}")
                if sizes.window is not None and sizes.window <= 0:
                    raise ConfigError(f"config.json: layers[{index}].mixer.mask.size must be positive")
                if sizes.kv_from is not None:
                    source = self.layers[sizes.kv_from].mixer if 0 <= sizes.kv_from < index else None
                    if not isinstance(source, DifferentialAttentionSizes) or source.kv_from is not None:
                        raise ConfigError(f"config.json: layers[{index}].mixer.kv_from must name an earlier attention layer with keys and "
                                          f"values of its own, got {sizes.kv_from}")
                    if (source.kv_heads, source.dim, source.vdim) != (sizes.kv_heads, sizes.dim, sizes.vdim):
                        raise ConfigError(f"config.json: layers[{index}] reads the keys and values of layers[{sizes.kv_from}], whose heads differ")
            elif sizes.dim > MOST_HEAD:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] has delta heads of {sizes.dim} key channels; "
                                            f"the kernels take up to {MOST_HEAD}")

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
                "embedding": {"scale": self.embedding_scale}, "layers": [layer.to_dict() for layer in self.layers]}
