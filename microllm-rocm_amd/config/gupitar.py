"""Typed configuration of the Gupitar decoder, read from its config.json.

The file names the model as ``"architecture": "Gupitar"`` and gives ``vocab``, ``width``, ``norm.eps`` and a list
``layers``. Every entry has a ``type`` (which mixer the layer has: ``latent_attention`` or ``rglru``), the mixer's
sizes and constants under ``mixer`` and its feed-forward under ``mlp`` (``dense``, ``moe`` or null for none). Every
size and constant is a key of the file; nothing has to be read from a tensor's shape.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

from . import fields
from .fields import ConfigError

LATENT_ATTENTION = "latent_attention"
RGLRU = "rglru"
DENSE = "dense"
MOE = "moe"


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
class LatentAttentionConfig:
    """Attention whose keys and values are projected up from one cached latent vector a token."""
    heads: int
    dim: int            # unrotated query/key dims a head
    rot_dim: int        # rotated query/key dims a head; the keys' rotated part is shared by all heads
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int         # a query sees itself and the window - 1 tokens before it
    rot_base: float
    rot_dims: int
    kv_from: Optional[int] = None   # the layer whose cached latents this layer reads instead of making its own

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "LatentAttentionConfig":
        rot = _object(source, "rot")
        config = cls(heads=fields.integer(source, "heads"), dim=fields.integer(source, "dim"),
                     rot_dim=fields.integer(source, "rot_dim"), vdim=fields.integer(source, "vdim"),
                     q_rank=fields.integer(source, "q_rank"), kv_rank=fields.integer(source, "kv_rank"),
                     scale=fields.number(source, "scale"), window=fields.integer(_object(source, "mask"), "size"),
                     rot_base=fields.number(rot, "base"), rot_dims=fields.integer(rot, "dims"),
                     kv_from=fields.integer(source, "kv_from", None))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "window", "rot_base", "rot_dims"):
            _positive(getattr(self, name), f"mixer.{name}")
        if self.rot_dims != self.rot_dim:
            raise ConfigError("mixer.rot.dims must equal mixer.rot_dim: the rotated part turns whole")
        if self.rot_dims % 2 != 0:
            raise ConfigError("mixer.rot.dims must be even")
        if self.kv_from is not None and self.kv_from < 0:
            raise ConfigError("mixer.kv_from names an earlier layer")

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "mask": {"size": self.window},
                               "q_rank": self.q_rank, "rot": {"base": self.rot_base, "dims": self.rot_dims},
                               "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class RglruConfig:
    """A recurrent block: a gated branch beside a short convolution and a gated linear recurrence."""
    width: int
    blocks: int
    conv: int           # taps of the convolution

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "RglruConfig":
        config = cls(width=fields.integer(source, "width"), blocks=fields.integer(source, "blocks"),
                     conv=fields.integer(source, "conv"))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("width", "blocks", "conv"):
            _positive(getattr(self, name), f"mixer.{name}")
        if self.width % self.blocks != 0:
            raise ConfigError("mixer.width must divide into mixer.blocks equal parts")

    def to_dict(self) -> Dict[str, Any]:
        return {"blocks": self.blocks, "conv": self.conv, "width": self.width}


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": DENSE}


@dataclass(frozen=True)
class MoeMlpConfig:
    experts: int
    top: int
    expert_ff: int
    shared_ff: Optional[int] = None     # None: no shared expert

    def validate(self) -> None:
        _positive(self.experts, "mlp.router.experts")
        _positive(self.top, "mlp.router.top")
        _positive(self.expert_ff, "mlp.expert.ff")
        if self.top > self.experts:
            raise ConfigError("mlp.router.top cannot exceed mlp.router.experts")
        if self.shared_ff is not None:
            _positive(self.shared_ff, "mlp.shared.ff")

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"expert": {"ff": self.expert_ff}, "kind": MOE,
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _mlp_from_dict(source: Optional[Mapping[str, Any]]) -> Union[None, DenseMlpConfig, MoeMlpConfig]:
    if source is None:
        return None
    kind = fields.string(source, "kind")
    if kind == DENSE:
        return DenseMlpConfig(ff=_positive(fields.integer(source, "ff"), "mlp.ff"))
    if kind == MOE:
        router = _object(source, "router")
        shared = _object(source, "shared", optional=True)
        config = MoeMlpConfig(experts=fields.integer(router, "experts"), top=fields.integer(router, "top"),
                              expert_ff=fields.integer(_object(source, "expert"), "ff"),
                              shared_ff=fields.integer(shared, "ff") if shared is not None else None)
        config.validate()
        return config
    raise ConfigError(f"unknown feed-forward kind {kind!r}; this design has {DENSE!r} and {MOE!r}")


@dataclass(frozen=True)
class GupitarLayerConfig:
    type: str
    mixer: Union[LatentAttentionConfig, RglruConfig]
    mlp: Union[None, DenseMlpConfig, MoeMlpConfig]

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "GupitarLayerConfig":
        kind = fields.string(source, "type")
        mixer = _object(source, "mixer")
        if kind == LATENT_ATTENTION:
            mixer_config = LatentAttentionConfig.from_dict(mixer)
        elif kind == RGLRU:
            mixer_config = RglruConfig.from_dict(mixer)
        else:
            raise ConfigError(f"unknown layer type {kind!r}; this design has {LATENT_ATTENTION!r} and {RGLRU!r}")
        return cls(type=kind, mixer=mixer_config, mlp=_mlp_from_dict(_object(source, "mlp", optional=True)))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class GupitarConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[GupitarLayerConfig, ...]
    architecture: str = "Gupitar"

    # what the engine's generic code asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "GupitarConfig":
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(layer, dict) for layer in layers):
            raise ConfigError("config key layers must be a list of objects with at least one entry")
        config = cls(vocab=fields.integer(source, "vocab"), width=fields.integer(source, "width"),
                     norm_eps=fields.number(_object(source, "norm"), "eps"),
                     layers=tuple(GupitarLayerConfig.from_dict(layer) for layer in layers),
                     architecture=fields.string(source, "architecture", "Gupitar"))
        config.validate()
        return config

    def validate(self) -> None:
        _positive(self.vocab, "vocab")
        _positive(self.width, "width")
        _positive(self.norm_eps, "norm.eps")
        for index, layer in enumerate(self.layers):
            mixer = layer.mixer
            if not isinstance(mixer, LatentAttentionConfig) or mixer.kv_from is None:
                continue
            if not 0 <= mixer.kv_from < index:
                raise ConfigError(f"layer {index}: kv_from must name an earlier layer")
            source = self.layers[mixer.kv_from].mixer
            if not isinstance(source, LatentAttentionConfig) or source.kv_from is not None:
                raise ConfigError(f"layer {index}: kv_from names layer {mixer.kv_from}, which makes no latents of its own")
            if (source.kv_rank, source.rot_dim, source.rot_base, source.rot_dims) != (mixer.kv_rank, mixer.rot_dim, mixer.rot_base, mixer.rot_dims):
                raise ConfigError(f"layer {index}: its latent size and rotation must equal those of layer {mixer.kv_from}")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1, sort_keys=True)
