"""Typed configuration of the Rorevik architecture, read from its config.json.

The file names every size and every constant that may differ between models of the design:
``vocab``, ``width``, ``max_positions`` (rows of the learned position table), ``embedding.scale``,
``norm.eps``, a list ``layers`` whose entries give the layer's ``type`` (which mixer it has), the
mixer's sizes (``mixer``) and its feed-forward (``mlp``, or null for none), and ``loop``: the
layers ``start .. stop - 1`` run ``times`` times in a row before the rest follow.  Nothing here
has a default that a model could contradict, except where a whole feature may be left out (no
loop, no rotation, no cap on the scores).
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping, Optional, Tuple, Union

from ..errors import ConfigError, UnsupportedModelError
from .base import ConfigReader


@dataclass(frozen=True)
class SoftcapAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]
    rot_dims: int                 # 0: no rotation
    rot_base: float

    @classmethod
    def read(cls, r: ConfigReader) -> "SoftcapAttentionConfig":
        rot = r.mapping("rot")
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  scale=r.number("scale"), softcap=r.number("softcap") if r.has("softcap") else None,
                  rot_dims=rot.integer("dims", minimum=0) if rot is not None else 0,
                  rot_base=rot.number("base") if rot is not None else 1.0)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{r.where}: heads ({cfg.heads}) must be a multiple of kv_heads ({cfg.kv_heads})")
        if cfg.rot_dims % 2 or cfg.rot_dims > cfg.dim:
            raise ConfigError(f"{r.where}: rot.dims ({cfg.rot_dims}) must be even and at most dim ({cfg.dim})")
        return cfg

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return d


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @classmethod
    def read(cls, r: ConfigReader) -> "StateSpaceConfig":
        cfg = cls(heads=r.integer("heads"), vdim=r.integer("vdim"), state=r.integer("state"), groups=r.integer("groups"),
                  norm_groups=r.integer("norm_groups"), conv=r.integer("conv"))
        if cfg.heads % cfg.groups:
            raise ConfigError(f"{r.where}: heads ({cfg.heads}) must be a multiple of groups ({cfg.groups})")
        if (cfg.heads * cfg.vdim) % cfg.norm_groups:
            raise ConfigError(f"{r.where}: heads * vdim ({cfg.heads * cfg.vdim}) must be a multiple of norm_groups ({cfg.norm_groups})")
        return cfg

    def to_dict(self) -> dict:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: SoftcapAttentionConfig
    right: StateSpaceConfig
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, r: ConfigReader) -> "ParallelMixerConfig":
        left, right = r.mapping("left"), r.mapping("right")
        if left is None or right is None:
            raise ConfigError(f"{r.where}: a parallel mixer needs 'left' and 'right'")
        return cls(SoftcapAttentionConfig.read(left), StateSpaceConfig.read(right),
                   r.number("left_scale", positive=False), r.number("right_scale", positive=False))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # The inner sizes of the two low-rank projections (decays, output gate).  A model folder's
    # config.json need not name them: they are then the row counts of the tensors ``a1`` and ``g1``
    # (``RorevikConfig.with_tensor_shapes``).  A bare configuration, which has no tensors, names them.
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None

    @classmethod
    def read(cls, r: ConfigReader) -> "ChannelDeltaConfig":
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  conv=r.integer("conv"), decay_rank=r.integer("decay_rank") if r.has("decay_rank") else None,
                  gate_rank=r.integer("gate_rank") if r.has("gate_rank") else None)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{r.where}: heads ({cfg.heads}) must be a multiple of kv_heads ({cfg.kv_heads})")
        return cfg

    def to_dict(self) -> dict:
        d = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            d["gate_rank"] = self.gate_rank
        return d


@dataclass(frozen=True)
class ClampedGluConfig:
    kind: str
    ff: int
    limit: float

    @classmethod
    def read(cls, r: ConfigReader) -> "ClampedGluConfig":
        kind = r.string("kind")
        if kind != "dense":
            raise UnsupportedModelError(f"{r.where}: feed-forward kind '{kind}' is not known (dense)")
        return cls(kind, r.integer("ff"), r.number("limit"))

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": self.kind, "limit": self.limit}


MIXER_CONFIGS = {"parallel": ParallelMixerConfig, "channel_delta": ChannelDeltaConfig}


@dataclass(frozen=True)
class RorevikLayer:
    type: str
    mixer: Union[ParallelMixerConfig, ChannelDeltaConfig]
    mlp: Optional[ClampedGluConfig]

    @classmethod
    def read(cls, r: ConfigReader) -> "RorevikLayer":
        kind = r.string("type")
        if kind not in MIXER_CONFIGS:
            raise UnsupportedModelError(f"{r.where}: layer type '{kind}' is not known ({', '.join(sorted(MIXER_CONFIGS))})")
        mixer = r.mapping("mixer")
        if mixer is None:
            raise ConfigError(f"{r.where}: required key 'mixer' is missing")
        mlp = r.mapping("mlp")
        return cls(kind, MIXER_CONFIGS[kind].read(mixer), ClampedGluConfig.read(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class RorevikConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[RorevikLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str = "config.json") -> "RorevikConfig":
        r = ConfigReader(raw, where)
        norm, emb, loop = r.mapping("norm"), r.mapping("embedding"), r.mapping("loop")
        if norm is None or emb is None:
            raise ConfigError(f"{where}: required keys 'norm' and 'embedding' are objects")
        entries = raw.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = tuple(RorevikLayer.read(ConfigReader(e, f"{where}:layers[{i}]")) for i, e in enumerate(entries))
        start = stop = 0
        times = 1
        if loop is not None:
            start, stop, times = loop.integer("start", minimum=0), loop.integer("stop", minimum=0), loop.integer("times", minimum=0)
            if not start <= stop <= len(layers):
                raise ConfigError(f"{where}: loop {start} .. {stop} does not lie within the {len(layers)} layers")
        return cls(architecture=r.string("architecture", "Rorevik"), vocab=r.integer("vocab"), width=r.integer("width"),
                   max_positions=r.integer("max_positions"), embedding_scale=emb.number("scale", positive=False),
                   norm_eps=norm.number("eps"), layers=layers, loop_start=start, loop_stop=stop, loop_times=times)

    def with_tensor_shapes(self, shapes) -> "RorevikConfig":
        """The configuration with the sizes that only the tensors give: ``shapes()`` returns the
        folder's tensor shapes by name and is called only if something is left open."""
        open_layers = [i for i, l in enumerate(self.layers)
                       if isinstance(l.mixer, ChannelDeltaConfig) and (l.mixer.decay_rank is None or l.mixer.gate_rank is None)]
        if not open_layers:
            return self
        found = shapes()
        layers = list(self.layers)
        for i in open_layers:
            m, ranks = layers[i].mixer, {}
            for key, name in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                if getattr(m, key) is None:
                    if name not in found or len(found[name]) != 2:
                        raise ConfigError(f"layer {i}: neither the configuration's '{key}' nor a matrix '{name}' gives the size")
                    ranks[key] = int(found[name][0])
            layers[i] = replace(layers[i], mixer=replace(m, **ranks))
        return replace(self, layers=tuple(layers))

    def run_order(self) -> Tuple[int, ...]:
        """Layer indices in the order they run: the looped span repeated in a row, then the rest."""
        n = len(self.layers)
        span = tuple(range(self.loop_start, self.loop_stop))
        return tuple(range(self.loop_start)) + span * self.loop_times + tuple(range(self.loop_stop, n))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
             "layers": [l.to_dict() for l in self.layers], "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
             "vocab": self.vocab, "width": self.width}
        if self.loop_stop > self.loop_start:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return d

    # what the engine's front ends ask of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width
