"""Typed configuration of the Dafidra architecture, read from its config.json.

The file names every size and every constant that may differ between models of the design:
``vocab``, ``width``, ``norm.eps``, ``residual_mult`` and a list ``layers`` whose entries give
the layer's ``type`` (which mixer it has), the mixer's sizes (``mixer``) and its feed-forward
(``mlp``, or null for none).  Nothing here has a default that a model could contradict, except
where a whole feature may be left out (no window, no query temperature, experts in one group).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from ..errors import ConfigError, UnsupportedModelError
from .base import ConfigReader

DEFAULT_MAX_POSITIONS = 1 << 20      # the design has no position table: a bound for the block tables only


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    temp_coef: float
    temp_every: int

    @classmethod
    def read(cls, r: ConfigReader) -> "SinkAttentionConfig":
        mask, temp = r.mapping("mask"), r.mapping("q_temp")
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  scale=r.number("scale"), window=mask.integer("size") if mask is not None else None,
                  temp_coef=temp.number("coef", positive=False) if temp is not None else 0.0,
                  temp_every=temp.integer("every") if temp is not None else 1)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{r.where}: heads ({cfg.heads}) must be a multiple of kv_heads ({cfg.kv_heads})")
        return cfg

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.temp_coef:
            d["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        return d


@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def read(cls, r: ConfigReader) -> "MatrixMemoryConfig":
        return cls(heads=r.integer("heads"), dim=r.integer("dim"), vdim=r.integer("vdim"), gate_cap=r.number("gate_cap"))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                  # "dense" or "moe"
    ff: int                    # dense: its width; moe: one expert's width
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1

    @classmethod
    def read(cls, r: ConfigReader) -> "FeedForwardConfig":
        kind = r.string("kind")
        if kind == "dense":
            return cls(kind, r.integer("ff"))
        if kind == "moe":
            expert, router = r.mapping("expert"), r.mapping("router")
            if expert is None or router is None:
                raise ConfigError(f"{r.where}: a 'moe' feed-forward needs 'expert' and 'router'")
            groups = router.mapping("groups")
            cfg = cls(kind, expert.integer("ff"), experts=router.integer("experts"), top=router.integer("top"),
                      groups=groups.integer("count") if groups is not None else 1,
                      keep=groups.integer("keep") if groups is not None else 1)
            if cfg.top > cfg.experts or cfg.experts % cfg.groups or cfg.keep > cfg.groups:
                raise ConfigError(f"{r.where}: {cfg.top} of {cfg.experts} experts in {cfg.groups} groups ({cfg.keep} kept) is not possible")
            return cfg
        raise UnsupportedModelError(f"{r.where}: feed-forward kind '{kind}' is not known (dense, moe)")

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}


@dataclass(frozen=True)
class DafidraLayer:
    type: str                                  # the mixer: "parallel"
    left: SinkAttentionConfig
    right: MatrixMemoryConfig
    mlp: Optional[FeedForwardConfig]

    @classmethod
    def read(cls, r: ConfigReader) -> "DafidraLayer":
        kind = r.string("type")
        if kind != "parallel":
            raise UnsupportedModelError(f"{r.where}: layer type '{kind}' is not known (parallel)")
        mixer = r.mapping("mixer")
        if mixer is None:
            raise ConfigError(f"{r.where}: required key 'mixer' is missing")
        left, right = mixer.mapping("left"), mixer.mapping("right")
        if left is None or right is None:
            raise ConfigError(f"{mixer.where}: a parallel mixer needs 'left' and 'right'")
        mlp = r.mapping("mlp")
        return cls(kind, SinkAttentionConfig.read(left), MatrixMemoryConfig.read(right),
                   FeedForwardConfig.read(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": {"left": self.left.to_dict(), "right": self.right.to_dict()},
                "mlp": self.mlp.to_dict() if self.mlp is not None else None}


@dataclass(frozen=True)
class DafidraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[DafidraLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str = "config.json") -> "DafidraConfig":
        r = ConfigReader(raw, where)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError(f"{where}: required key 'norm' is missing")
        entries = raw.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = tuple(DafidraLayer.read(ConfigReader(e, f"{where}:layers[{i}]")) for i, e in enumerate(entries))
        return cls(architecture=r.string("architecture", "Dafidra"), vocab=r.integer("vocab"), width=r.integer("width"),
                   norm_eps=norm.number("eps"), residual_mult=r.number("residual_mult", positive=False), layers=layers,
                   max_positions=r.integer("max_positions", DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # what the engine's front ends ask of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width
