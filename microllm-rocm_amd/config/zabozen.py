"""Typed configuration of the Zabozen decoder, read from its config.json.

The file names the model as ``"architecture": "Zabozen"`` and gives ``vocab``, ``width``, ``norm.eps``,
``residual_mult`` (the factor on what every sublayer adds to the residual stream), ``logit_softcap`` (absent or null:
none) and a list ``layers``. Every entry has a ``type`` (which mixer the layer has: ``latent_attention``, ``attention``
or ``delta``), the mixer's sizes and constants under ``mixer`` and its feed-forward under ``mlp`` (``dense``, or null
for none). Every size and constant is a key of the file; nothing has to be read from a tensor's shape.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

from . import fields
from .fields import ConfigError

LATENT_ATTENTION = "latent_attention"
ATTENTION = "attention"
DELTA = "delta"
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
class LatentAttentionConfig:
    """Causal attention whose keys and values are projected up from one cached latent vector a token; the queries come
    straight from the input, the heads' results pass a gate of one number a head."""
    heads: int
    dim: int            # unrotated query/key dims a head
    rot_dim: int        # rotated query/key dims a head; the keys' rotated part is shared by all heads
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "LatentAttentionConfig":
        rot = _object(source, "rot")
        config = cls(heads=fields.integer(source, "heads"), dim=fields.integer(source, "dim"),
                     rot_dim=fields.integer(source, "rot_dim"), vdim=fields.integer(source, "vdim"),
                     kv_rank=fields.integer(source, "kv_rank"), scale=fields.number(source, "scale"),
                     rot_base=fields.number(rot, "base"), rot_dims=fields.integer(rot, "dims"))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot_base", "rot_dims"):
            _positive(getattr(self, name), f"mixer.{name}")
        if self.rot_dims != self.rot_dim:
            raise ConfigError("mixer.rot.dims must equal mixer.rot_dim: the rotated part turns whole")
        if self.rot_dims % 2 != 0:
            raise ConfigError("mixer.rot.dims must be even")

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": {"base": self.rot_base, "dims": self.rot_dims},
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class WindowAttentionConfig:
    """Softmax attention over a sliding window with grouped key/value heads, biases on its projections, queries and
    keys of unit root mean square, and a slope a head times the distance taken off the scores."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int         # a query sees itself and the window - 1 tokens before it
    kv_from: Optional[int] = None   # the layer whose cached keys and values this layer reads instead of making its own

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "WindowAttentionConfig":
        config = cls(heads=fields.integer(source, "heads"), kv_heads=fields.integer(source, "kv_heads"),
                     dim=fields.integer(source, "dim"), vdim=fields.integer(source, "vdim"), scale=fields.number(source, "scale"),
                     window=fields.integer(_object(source, "mask"), "size"), kv_from=fields.integer(source, "kv_from", None))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim", "window"):
            _positive(getattr(self, name), f"mixer.{name}")
        if self.heads % self.kv_heads != 0:
            raise ConfigError("mixer.heads must divide into mixer.kv_heads groups")
        if self.kv_from is not None and self.kv_from < 0:
            raise ConfigError("mixer.kv_from names an earlier layer")

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "mask": {"size": self.window},
                               "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class DeltaConfig:
    """The gated delta rule behind short convolutions."""
    heads: int
    kv_heads: int       # heads of queries and keys
    dim: int
    vdim: int
    conv: int           # taps of the convolutions

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "DeltaConfig":
        config = cls(heads=fields.integer(source, "heads"), kv_heads=fields.integer(source, "kv_heads"),
                     dim=fields.integer(source, "dim"), vdim=fields.integer(source, "vdim"), conv=fields.integer(source, "conv"))
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim", "conv"):
            _positive(getattr(self, name), f"mixer.{name}")
        if self.heads % self.kv_heads != 0:
            raise ConfigError("mixer.heads must divide into mixer.kv_heads groups")

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"ff": self.ff, "kind": DENSE}


def _mlp_from_dict(source: Optional[Mapping[str, Any]]) -> Optional[DenseMlpConfig]:
    if source is None:
        return None
    kind = fields.string(source, "kind")
    if kind != DENSE:
        raise ConfigError(f"unknown feed-forward kind {kind!r}; this design has {DENSE!r}")
    return DenseMlpConfig(ff=_positive(fields.integer(source, "ff"), "mlp.ff"))


MixerConfig = Union[LatentAttentionConfig, WindowAttentionConfig, DeltaConfig]
_MIXERS = {LATENT_ATTENTION: LatentAttentionConfig, ATTENTION: WindowAttentionConfig, DELTA: DeltaConfig}


@dataclass(frozen=True)
class ZabozenLayerConfig:
    type: str
    mixer: MixerConfig
    mlp: Optional[DenseMlpConfig]

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ZabozenLayerConfig":
        kind = fields.string(source, "type")
        if kind not in _MIXERS:
            raise ConfigError(f"unknown layer type {kind!r}; this design has {', '.join(sorted(_MIXERS))}")
        return cls(type=kind, mixer=_MIXERS[kind].from_dict(_object(source, "mixer")),
                   mlp=_mlp_from_dict(_object(source, "mlp", optional=True)))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class ZabozenConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[ZabozenLayerConfig, ...]
    logit_softcap: Optional[float] = None
    architecture: str = "Zabozen"

    # what the engine's generic code asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ZabozenConfig":
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(layer, dict) for layer in layers):
            raise ConfigError("config key layers must be a list of objects with at least one entry")
        config = cls(vocab=fields.integer(source, "vocab"), width=fields.integer(source, "width"),
                     norm_eps=fields.number(_object(source, "norm"), "eps"), residual_mult=fields.number(source, "residual_mult", 1.0),
                     layers=tuple(ZabozenLayerConfig.from_dict(layer) for layer in layers),
                     logit_softcap=fields.number(source, "logit_softcap", None),
                     architecture=fields.string(source, "architecture", "Zabozen"))
        config.validate()
        return config

    def validate(self) -> None:
        _positive(self.vocab, "vocab")
        _positive(self.width, "width")
        _positive(self.norm_eps, "norm.eps")
        if self.logit_softcap is not None:
            _positive(self.logit_softcap, "logit_softcap")
        for index, layer in enumerate(self.layers):
            mixer = layer.mixer
            if not isinstance(mixer, WindowAttentionConfig) or mixer.kv_from is None:
                continue
            if not 0 <= mixer.kv_from < index:
                raise ConfigError(f"layer {index}: kv_from must name an earlier layer")
            source = self.layers[mixer.kv_from].mixer
            if not isinstance(source, WindowAttentionConfig) or source.kv_from is not None:
                raise ConfigError(f"layer {index}: kv_from names layer {mixer.kv_from}, which makes no keys and values of its own")
            if (source.kv_heads, source.dim, source.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                raise ConfigError(f"layer {index}: its key/value heads and their sizes must equal those of layer {mixer.kv_from}")

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1, sort_keys=True)
