"""Typed configuration of the Kalevik decoder, read from its config.json.

The file names the model as ``"architecture": "Kalevik"`` and gives ``vocab``, ``width``, ``norm.eps``,
``embedding.scale`` (the factor on the embedding's rows; absent: 1), ``loop`` (``start``, ``stop``, ``times``: the
layers ``start .. stop - 1`` run ``times`` times in a row with the same weights; absent: every layer once) and a list
``layers``. Every entry has a ``type`` (``latent_attention`` or ``parallel``), the mixer's sizes and constants under
``mixer`` and its feed-forward under ``mlp`` (``dense``, ``moe``, or null for none). Every size and constant is a key of
the file; nothing has to be read from a tensor's shape.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

from . import fields
from .fields import ConfigError

LATENT_ATTENTION = "latent_attention"
PARALLEL = "parallel"
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
    """Causal attention whose keys and values are projected up from one cached latent vector a token; the queries come
    straight from the input; the rotated parts turn with neighbouring channels paired."""
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
class ChunkAttentionConfig:
    """The left member of a parallel mixer: softmax attention inside chunks of positions, grouped key/value heads, a
    norm of queries and keys, a partial rotation with stretched positions, one added to the softmax's denominator, a
    gate a head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int              # mask.size
    rot_base: float
    rot_dims: int
    rot_factor: float = 1.0     # rot.scaling.factor: every rate is divided by it

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ChunkAttentionConfig":
        rot = _object(source, "rot")
        scaling = _object(rot, "scaling", optional=True)
        config = cls(heads=fields.integer(source, "heads"), kv_heads=fields.integer(source, "kv_heads"),
                     dim=fields.integer(source, "dim"), vdim=fields.integer(source, "vdim"), scale=fields.number(source, "scale"),
                     chunk=fields.integer(_object(source, "mask"), "size"), rot_base=fields.number(rot, "base"),
                     rot_dims=fields.integer(rot, "dims"),
                     rot_factor=fields.number(scaling, "factor") if scaling is not None else 1.0)
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "kv_heads", "dim", "vdim", "chunk", "rot_base", "rot_dims", "rot_factor"):
            _positive(getattr(self, name), f"mixer.left.{name}")
        if self.heads % self.kv_heads != 0:
            raise ConfigError("mixer.left.heads must divide into mixer.left.kv_heads groups")
        if self.rot_dims % 2 != 0 or self.rot_dims > self.dim:
            raise ConfigError("mixer.left.rot.dims must be even and at most mixer.left.dim")

    def to_dict(self) -> Dict[str, Any]:
        rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_factor != 1.0:
            rot["scaling"] = {"factor": self.rot_factor}
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "mask": {"size": self.chunk}, "rot": rot,
                "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class RetentionConfig:
    """The right member: linear attention with one fixed decay a head."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "RetentionConfig":
        decay = source.get("decay")
        if not isinstance(decay, list) or not decay:
            raise ConfigError("mixer.right.decay must be a list with one number a head")
        values = tuple(fields.number({"decay": value}, "decay") for value in decay)
        config = cls(heads=fields.integer(source, "heads"), dim=fields.integer(source, "dim"), vdim=fields.integer(source, "vdim"),
                     decay=values)
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("heads", "dim", "vdim"):
            _positive(getattr(self, name), f"mixer.right.{name}")
        if len(self.decay) != self.heads:
            raise ConfigError("mixer.right.decay must hold one number a head")
        if any(not 0.0 <= value <= 1.0 for value in self.decay):
            raise ConfigError("mixer.right.decay must lie between 0 and 1")

    def to_dict(self) -> Dict[str, Any]:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelConfig:
    left: ChunkAttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "ParallelConfig":
        return cls(left=ChunkAttentionConfig.from_dict(_object(source, "left")), right=RetentionConfig.from_dict(_object(source, "right")),
                   left_scale=fields.number(source, "left_scale"), right_scale=fields.number(source, "right_scale"))

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(), "right_scale": self.right_scale}


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
    groups: int = 1             # router.groups.count; 1: every expert can be chosen
    keep_groups: int = 1        # router.groups.keep
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "MoeMlpConfig":
        router = _object(source, "router")
        groups = _object(router, "groups", optional=True)
        shared = _object(source, "shared", optional=True)
        config = cls(experts=fields.integer(router, "experts"), top=fields.integer(router, "top"),
                     expert_ff=fields.integer(_object(source, "expert"), "ff"),
                     groups=fields.integer(groups, "count") if groups is not None else 1,
                     keep_groups=fields.integer(groups, "keep") if groups is not None else 1,
                     shared_ff=fields.integer(shared, "ff") if shared is not None else None)
        config.validate()
        return config

    def validate(self) -> None:
        for name in ("experts", "top", "expert_ff", "groups", "keep_groups"):
            _positive(getattr(self, name), f"mlp.{name}")
        if self.shared_ff is not None:
            _positive(self.shared_ff, "mlp.shared.ff")
        if self.top > self.experts:
            raise ConfigError("mlp.router.top cannot exceed mlp.router.experts")
        if self.experts % self.groups != 0 or self.keep_groups > self.groups:
            raise ConfigError("mlp.router.groups: equal groups of experts, of which at most all are kept")
        if self.keep_groups * (self.experts // self.groups) < self.top:
            raise ConfigError("mlp.router.groups: the kept groups hold fewer experts than a token takes")

    def to_dict(self) -> Dict[str, Any]:
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.groups != 1:
            router["groups"] = {"count": self.groups, "keep": self.keep_groups}
        out: Dict[str, Any] = {"expert": {"ff": self.expert_ff}, "kind": MOE, "router": router}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


MlpConfig = Union[DenseMlpConfig, MoeMlpConfig]


def _mlp_from_dict(source: Optional[Mapping[str, Any]]) -> Optional[MlpConfig]:
    if source is None:
        return None
    kind = fields.string(source, "kind")
    if kind == DENSE:
        return DenseMlpConfig(ff=_positive(fields.integer(source, "ff"), "mlp.ff"))
    if kind == MOE:
        return MoeMlpConfig.from_dict(source)
    raise ConfigError(f"unknown feed-forward kind {kind!r}; this design has {DENSE!r} and {MOE!r}")


MixerConfig = Union[LatentAttentionConfig, ParallelConfig]
_MIXERS = {LATENT_ATTENTION: LatentAttentionConfig, PARALLEL: ParallelConfig}


@dataclass(frozen=True)
class KalevikLayerConfig:
    type: str
    mixer: MixerConfig
    mlp: Optional[MlpConfig]

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "KalevikLayerConfig":
        kind = fields.string(source, "type")
        if kind not in _MIXERS:
            raise ConfigError(f"unknown layer type {kind!r}; this design has {', '.join(sorted(_MIXERS))}")
        return cls(type=kind, mixer=_MIXERS[kind].from_dict(_object(source, "mixer")),
                   mlp=_mlp_from_dict(_object(source, "mlp", optional=True)))

    def to_dict(self) -> Dict[str, Any]:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class KalevikConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[KalevikLayerConfig, ...]
    embedding_scale: float = 1.0
    loop: Optional[LoopConfig] = None
    architecture: str = "Kalevik"

    # what the engine's generic code asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "KalevikConfig":
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(layer, dict) for layer in layers):
            raise ConfigError("config key layers must be a list of objects with at least one entry")
        loop_source = _object(source, "loop", optional=True)
        loop = None
        if loop_source is not None:
            loop = LoopConfig(fields.integer(loop_source, "start"), fields.integer(loop_source, "stop"),
                              fields.integer(loop_source, "times"))
        embedding = _object(source, "embedding", optional=True)
        config = cls(vocab=fields.integer(source, "vocab"), width=fields.integer(source, "width"),
                     norm_eps=fields.number(_object(source, "norm"), "eps"),
                     layers=tuple(KalevikLayerConfig.from_dict(layer) for layer in layers),
                     embedding_scale=fields.number(embedding, "scale", 1.0) if embedding is not None else 1.0, loop=loop,
                     architecture=fields.string(source, "architecture", "Kalevik"))
        config.validate()
        return config

    def validate(self) -> None:
        _positive(self.vocab, "vocab")
        _positive(self.width, "width")
        _positive(self.norm_eps, "norm.eps")
        if self.loop is not None:
            if not 0 <= self.loop.start < self.loop.stop <= len(self.layers) or self.loop.times < 1:
                raise ConfigError("loop must name a non-empty range of layers and run it at least once")

    def run_order(self) -> Tuple[Tuple[int, bool], ...]:
        """``(layer, whether the embedding's output joins the stream right before it)`` for every run, in order: the
        looped range as often as it says, in a row; every pass but the first begins with the embedding's output."""
        count = len(self.layers)
        if self.loop is None:
            return tuple((index, False) for index in range(count))
        order = [(index, False) for index in range(self.loop.start)]
        for turn in range(self.loop.times):
            order += [(index, turn > 0 and index == self.loop.start) for index in range(self.loop.start, self.loop.stop)]
        return tuple(order + [(index, False) for index in range(self.loop.stop, count)])

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                               "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
                               "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1, sort_keys=True)
