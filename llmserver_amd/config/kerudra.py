"""Kerudra configuration: a nested ``config.json`` that lists the layers one by one.

Top level: ``architecture`` ("Kerudra"), ``vocab``, ``width``, ``norm.eps``, ``layers`` and, each optional,
``embedding.scale`` (what the embedding rows are multiplied by), ``logit_scale``, ``residual_mult`` (what every
sublayer's result is multiplied by before it joins the stream), ``streams`` (the number of residual streams that
hyper-connections keep; absent: one plain stream) and ``loop`` (``start``, ``stop``, ``times``: the layers ``start`` to
``stop - 1`` run ``times`` times in a row with the same weights).  A layer entry gives ``type`` (its mixer: ``attention``,
``latent_attention`` or ``mlstm``), ``mixer`` (the mixer's sizes and constants) and ``mlp`` (``kind`` ``dense`` with its
size, or null).  Nothing here is a default of the design: what the file does not name is not there (no window, no
rotation, no loop, a scale of one).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Mapping, Optional, Tuple, Union

from .barotar import _mapping, _positive
from .base import ConfigError, ModelConfig, UnsupportedModelError, field
from .zepolix import _number

MIXERS = ("attention", "latent_attention", "mlstm")
FEED_FORWARDS = ("dense",)
MOST_STREAMS = 8            # what the stream kernels are built for (csrc/stream.hip)


def _optional_mapping(where: str, raw: Mapping[str, Any], key: str) -> Optional[Mapping[str, Any]]:
    if key not in raw or raw[key] is None:
        return None
    return _mapping(where, raw, key)


def _rotation(where: str, raw: Mapping[str, Any], most: int) -> Tuple[int, float]:
    """``(dims, base)`` of ``raw["rot"]``; no such key: nothing turns."""
    rot = _optional_mapping(where, raw, "rot")
    if rot is None:
        return 0, 1.0
    dims, base = _number(where + ".rot", rot, "dims"), _number(where + ".rot", rot, "base", float)
    if dims < 0 or dims % 2 or dims > most or base <= 0:
        raise ConfigError(f"config.json: {where}.rot: an even number of up to {most} dimensions turns, with a positive base; got {dims}, {base}")
    return dims, base


def _window(where: str, raw: Mapping[str, Any]) -> Optional[int]:
    mask = _optional_mapping(where, raw, "mask")
    if mask is None:
        return None
    size = _number(where + ".mask", mask, "size")
    if size <= 0:
        raise ConfigError(f"config.json: {where}.mask.size must be positive")
    return size


def _rotation_dict(dims: int, base: float) -> dict:
    return {"rot": {"base": base, "dims": dims}} if dims else {}


@dataclasses.dataclass(frozen=True)
class SharedValueAttentionSizes:
    """Softmax attention with grouped key/value heads without value weights: the unrotated key rows serve as values."""
    heads: int
    kv_heads: int
    dim: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int]

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "SharedValueAttentionSizes":
        heads, dim = _number(where, raw, "heads"), _number(where, raw, "dim")
        kv_heads = _number(where, raw, "kv_heads") if "kv_heads" in raw else heads
        sizes = cls(heads, kv_heads, dim, _number(where, raw, "scale", float), *_rotation(where, raw, dim), _window(where, raw))
        _positive(where, sizes, ("heads", "kv_heads", "dim"))
        if sizes.heads % sizes.kv_heads:
            raise ConfigError(f"config.json: {where}: {sizes.heads} query heads are no multiple of {sizes.kv_heads} key/value heads")
        if "vdim" in raw and _number(where, raw, "vdim") != dim:
            raise ConfigError(f"config.json: {where}: the values are the keys, so vdim must be dim ({dim})")
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.dim, "scale": self.scale,
               **_rotation_dict(self.rot_dims, self.rot_base)}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclasses.dataclass(frozen=True)
class WindowedLatentSizes:
    """Attention over a shared low-rank latent with a rotated key part, gated per channel, possibly windowed."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int]

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "WindowedLatentSizes":
        rot_dim = _number(where, raw, "rot_dim")
        sizes = cls(_number(where, raw, "heads"), _number(where, raw, "dim"), rot_dim, _number(where, raw, "vdim"), _number(where, raw, "kv_rank"),
                    _number(where, raw, "scale", float), *_rotation(where, raw, rot_dim), _window(where, raw))
        _positive(where, sizes, ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        return sizes

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank, "scale": self.scale,
               **_rotation_dict(self.rot_dims, self.rot_base)}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclasses.dataclass(frozen=True)
class MatrixMemorySizes:
    """A matrix memory per head with exponential gates (mLSTM)."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def read(cls, where: str, raw: Mapping[str, Any]) -> "MatrixMemorySizes":
        sizes = cls(_number(where, raw, "heads"), _number(where, raw, "dim"), _number(where, raw, "vdim"), _number(where, raw, "gate_cap", float))
        _positive(where, sizes, ("heads", "dim", "vdim", "gate_cap"))
        return sizes

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


MIXER_SIZES = {"attention": SharedValueAttentionSizes, "latent_attention": WindowedLatentSizes, "mlstm": MatrixMemorySizes}


@dataclasses.dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class KerudraLayer:
    type: str
    mixer: Union[SharedValueAttentionSizes, WindowedLatentSizes, MatrixMemorySizes]
    mlp: Optional[DenseSizes]

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclasses.dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclasses.dataclass(frozen=True)
class KerudraConfig(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "Kerudra"

    vocab: int = field("vocab", int)
    width: int = field("width", int)
    norm: object = field("norm", object)
    layers_raw: object = field("layers", object)
    embedding: object = field("embedding", object, None)
    loop_raw: object = field("loop", object, None)
    logit_scale: float = field("logit_scale", float, 1.0)
    residual_mult: float = field("residual_mult", float, 1.0)
    streams: int = field("streams", int, 0)          # 0: one plain residual stream, no hyper-connections
    layers: Tuple[KerudraLayer, ...] = ()
    loop: Optional[Loop] = None
    norm_eps: float = 0.0
    embedding_scale: float = 1.0

    def resolve(self, raw: Mapping[str, Any]) -> "KerudraConfig":
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
            mixer = MIXER_SIZES[kind].read(where + ".mixer", _mapping(where, entry, "mixer"))
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") not in FEED_FORWARDS:
                    named = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                    raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {where} has the feed-forward {named!r}; built: {', '.join(FEED_FORWARDS)}")
                mlp = DenseSizes(_number(where + ".mlp", mlp, "ff"))
                if mlp.ff <= 0:
                    raise ConfigError(f"config.json: {where}.mlp.ff must be positive")
            layers.append(KerudraLayer(kind, mixer, mlp))
        loop = None
        if self.loop_raw is not None:
            loop = Loop(*(_number("loop", self.loop_raw, key) for key in ("start", "stop", "times")))
        scale = 1.0
        if self.embedding is not None:
            if not isinstance(self.embedding, Mapping):
                raise ConfigError("config.json: 'embedding' must be an object")
            if "scale" in self.embedding:
                scale = _number("embedding", self.embedding, "scale", float)
        return dataclasses.replace(self, layers=tuple(layers), loop=loop, norm_eps=_number("norm", self.norm, "eps", float),
                                   embedding_scale=scale)

    def validate(self, raw: Mapping[str, Any]) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"vocab and width must be positive: {self.vocab}, {self.width}")
        if self.norm_eps <= 0.0:
            raise ConfigError(f"norm.eps must be positive: {self.norm_eps}")
        if self.streams < 0:
            raise ConfigError(f"streams must not be negative: {self.streams}")
        if self.streams > MOST_STREAMS:
            raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: {self.streams} residual streams; the stream kernels take up to {MOST_STREAMS}")
        if self.loop is not None and not (0 <= self.loop.start <= self.loop.stop <= len(self.layers) and self.loop.times >= 1):
            raise ConfigError(f"loop: layers {self.loop.start} to {self.loop.stop - 1} of {len(self.layers)}, {self.loop.times} times")
        for index, layer in enumerate(self.layers):
            sizes = layer.mixer
            if isinstance(sizes, SharedValueAttentionSizes) and sizes.dim > 256:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] has attention heads of {sizes.dim}; "
                                            "the attention kernels take heads of up to 256")
            if isinstance(sizes, WindowedLatentSizes) and sizes.kv_rank + sizes.rot_dim > 256:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] caches rows of {sizes.kv_rank} + {sizes.rot_dim}; "
                                            "the attention kernels take rows of up to 256")
            if isinstance(sizes, MatrixMemorySizes) and sizes.dim > 512:
                raise UnsupportedModelError(f"Model type {self.MODEL_TYPE!r}: layers[{index}] has memory heads of {sizes.dim} key channels; "
                                            "the recurrence kernels take up to 512")

    def layer_runs(self) -> Tuple[int, ...]:
        """The layers in the order they run, a looped layer once for every pass."""
        indices = tuple(range(len(self.layers)))
        if self.loop is None:
            return indices
        return indices[:self.loop.start] + indices[self.loop.start:self.loop.stop] * self.loop.times + indices[self.loop.stop:]

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
               "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale, "residual_mult": self.residual_mult,
               "layers": [layer.to_dict() for layer in self.layers]}
        if self.streams:
            out["streams"] = self.streams
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out
