"""Typed configuration of the Siditar decoder, read from its config.json.

The file names the model as ``"architecture": "Siditar"`` and gives, beside ``vocab``, ``width``, ``streams``,
``norm.eps`` and ``loop``, a list ``layers`` whose entries hold the sizes and constants of that layer's mixer and
feed-forward. Two sizes are in no key: the rows of an attention's table of distance biases and the rank of a
linear attention's decay projection. They are the shapes of tensors, so a configuration read from a folder is
completed from the file's header (``with_tensor_shapes``); one made in code names them itself.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from . import fields
from .fields import ConfigError

PARALLEL = "parallel"
DENSE = "dense"


def _object(source: Mapping[str, Any], key: str, optional: bool = False) -> Optional[Mapping[str, Any]]:
    value = source.get(key)
    if value is None:
        if optional:
            return None
        raise ConfigError(f"config is missing {key}")
    if not isinstance(value, dict):
        raise ConfigError(f"config key {key} must be an object, got {value!r}")
    return value


def _positive(value, what: str):
    if value is None or value <= 0:
        raise ConfigError(f"{what} must be positive, got {value!r}")
    return value


@dataclass(frozen=True)
class BiasAttentionConfig:
    """The softmax attention of a parallel mixer: a bias by distance bucket, a sink, a query factor by position."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    temp_coef: float
    temp_every: int
    bias_rows: Optional[int] = None     # rows of the bias table: the tensor's shape says

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "BiasAttentionConfig":
        temp = _object(source, "q_temp")
        config = cls(heads=fields.integer(source, "heads"), kv_heads=fields.integer(source, "kv_heads"),
                     dim=fields.integer(source, "dim"), vdim=fields.integer(source, "vdim"),
                     scale=fields.number(source, "scale"), bias_max=fields.integer(source, "bias_max"),
                     temp_coef=fields.number(temp, "coef"), temp_every=fields.integer(temp, "every"),
                     bias_rows=fields.integer(source, "bias_rows", None))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim", "bias_max", "temp_every"):
            _positive(getattr(self, name), f"left.{name}")
        if self.heads % self.kv_heads != 0:
            raise ConfigError("left.heads must be a multiple of left.kv_heads")
        if self.bias_rows is not None and (self.bias_rows < 2 or self.bias_max <= self.bias_rows // 2):
            raise ConfigError("left.bias_max must lie beyond the distances that have a bucket of their own")

    def to_dict(self) -> Dict[str, Any]:
        return {"bias_max": self.bias_max, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "q_temp": {"coef": self.temp_coef, "every": self.temp_every}, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class LinearAttentionConfig:
    """The gated linear attention of a parallel mixer."""
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int] = None    # inner size of the decay's two projections: the tensors' shapes say

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "LinearAttentionConfig":
        config = cls(heads=fields.integer(source, "heads"), dim=fields.integer(source, "dim"),
                     vdim=fields.integer(source, "vdim"), tau=fields.number(source, "tau"),
                     decay_rank=fields.integer(source, "decay_rank", None))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "dim", "vdim", "tau"):
            _positive(getattr(self, name), f"right.{name}")

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: BiasAttentionConfig
    right: LinearAttentionConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ParallelMixerConfig":
        return cls(left=BiasAttentionConfig.from_dict(_object(source, "left")),
                   right=LinearAttentionConfig.from_dict(_object(source, "right")),
                   left_scale=fields.number(source, "left_scale"), right_scale=fields.number(source, "right_scale"))

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "DenseMlpConfig":
        kind = fields.string(source, "kind")
        if kind != DENSE:
            raise ConfigError(f"unknown feed-forward kind {kind!r}; this design has {DENSE!r}")
        return cls(ff=_positive(fields.integer(source, "ff"), "mlp.ff"), limit=_positive(fields.number(source, "limit"), "mlp.limit"))

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": DENSE, "limit": self.limit}


@dataclass(frozen=True)
class SiditarLayerConfig:
    type: str
    mixer: ParallelMixerConfig
    mlp: Optional[DenseMlpConfig]

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "SiditarLayerConfig":
        kind = fields.string(source, "type")
        if kind != PARALLEL:
            raise ConfigError(f"unknown layer type {kind!r}; this design has {PARALLEL!r}")
        mlp = _object(source, "mlp", optional=True)
        return cls(type=kind, mixer=ParallelMixerConfig.from_dict(_object(source, "mixer")),
                   mlp=DenseMlpConfig.from_dict(mlp) if mlp is not None else None)

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class LoopConfig:
    """Layers ``start`` to ``stop - 1`` run ``times`` times in a row, with the same weights."""
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class SiditarConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[SiditarLayerConfig, ...]
    streams: Optional[int] = None       # None: one residual stream with a plain sum
    loop: Optional[LoopConfig] = None
    architecture: str = "Siditar"

    # what the engine's generic code asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "SiditarConfig":
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(layer, dict) for layer in layers):
            raise ConfigError("config key layers must be a list of objects with at least one entry")
        loop_source = _object(source, "loop", optional=True)
        loop = None
        if loop_source is not None:
            loop = LoopConfig(fields.integer(loop_source, "start"), fields.integer(loop_source, "stop"),
                              fields.integer(loop_source, "times"))
        config = cls(vocab=fields.integer(source, "vocab"), width=fields.integer(source, "width"),
                     norm_eps=fields.number(_object(source, "norm"), "eps"),
                     layers=tuple(SiditarLayerConfig.from_dict(layer) for layer in layers),
                     streams=fields.integer(source, "streams", None), loop=loop,
                     architecture=fields.string(source, "architecture", "Siditar"))
        config.validate()
        return config

    def validate(self) -> None:
        _positive(self.vocab, "vocab")
        _positive(self.width, "width")
        _positive(self.norm_eps, "norm.eps")
        if self.streams is not None and not 1 <= self.streams <= 8:
            raise ConfigError("streams must lie between 1 and 8")
        if self.loop is not None:
            if not 0 <= self.loop.start < self.loop.stop <= len(self.layers) or self.loop.times < 1:
                raise ConfigError("loop must name a non-empty range of layers and run it at least once")

    def run_order(self) -> Tuple[int, ...]:
        """The layer of every run, in order: the looped range as often as it says, in a row."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(range(count))
        inner = list(range(self.loop.start, self.loop.stop)) * self.loop.times
        return tuple(list(range(self.loop.start)) + inner + list(range(self.loop.stop, count)))

    # ---- sizes that only tensors give ---------------------------------------------------------------------
    def with_tensor_shapes(self, shapes: Mapping[str, Sequence[int]]) -> "SiditarConfig":
        """The same configuration with the bias tables' rows and the decays' ranks read from the files' header."""
        layers = []
        for index, layer in enumerate(self.layers):
            left, right = layer.mixer.left, layer.mixer.right
            rel, low = shapes.get(f"l{index}.mix.left.rel"), shapes.get(f"l{index}.mix.right.a1")
            if left.bias_rows is None and rel is not None and len(rel) == 2:
                left = dataclasses.replace(left, bias_rows=int(rel[0]))
                left.validate()
            if right.decay_rank is None and low is not None and len(low) == 2:
                right = dataclasses.replace(right, decay_rank=int(low[0]))
            layers.append(dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, left=left, right=right)))
        return dataclasses.replace(self, layers=tuple(layers))

    # ---- writing ------------------------------------------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
                               "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        if self.streams is not None:
            out["streams"] = self.streams
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1, sort_keys=True)
