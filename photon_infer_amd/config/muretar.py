"""Typed configuration of the Muretar architecture, read from its config.json.

The file names every size and every constant that may differ between models of the design:
``vocab``, ``width``, ``norm.eps`` and a list ``layers`` whose entries give the layer's ``type`` (which
mixer it has: ``attention``, ``parallel`` or ``gla``), the mixer's sizes (``mixer``), its feed-forward
(``mlp``: ``kind`` ``dense`` or ``moe``, or null for none) and, optionally, ``weights_of``: the index of
the layer whose tensors this layer runs with a memory of its own.  The inner size of the gated linear
attention's low-rank decay projection is not in the file: it is the row count of the tensor ``a1``
(a bare configuration, which has no tensors, names ``decay_rank``).
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping, Optional, Tuple, Union

from ..errors import ConfigError, UnsupportedModelError
from .base import ConfigReader

DEFAULT_MAX_POSITIONS = 1 << 20      # nothing in the design bounds a position: the rotation is computed, states have no length


def _heads(r: ConfigReader, heads: int, kv_heads: int) -> None:
    if heads % kv_heads:
        raise ConfigError(f"{r.where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")


@dataclass(frozen=True)
class DiffAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float

    @classmethod
    def read(cls, r: ConfigReader) -> "DiffAttentionConfig":
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  scale=r.number("scale"), diff=r.number("diff", positive=False))
        _heads(r, cfg.heads, cfg.kv_heads)
        return cfg

    def to_dict(self) -> dict:
        return {"diff": self.diff, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class RotaryAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int                 # 0: no rotation
    rot_base: float
    rot_factor: Optional[float]   # every frequency divided by it; None: as they are

    @classmethod
    def read(cls, r: ConfigReader) -> "RotaryAttentionConfig":
        rot = r.mapping("rot")
        scaling = rot.mapping("scaling") if rot is not None else None
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  scale=r.number("scale"), rot_dims=rot.integer("dims", minimum=0) if rot is not None else 0,
                  rot_base=rot.number("base") if rot is not None else 1.0,
                  rot_factor=scaling.number("factor") if scaling is not None else None)
        _heads(r, cfg.heads, cfg.kv_heads)
        if cfg.rot_dims % 2 or cfg.rot_dims > cfg.dim:
            raise ConfigError(f"{r.where}: rot.dims ({cfg.rot_dims}) must be even and at most dim ({cfg.dim})")
        return cfg

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_factor is not None:
                d["rot"]["scaling"] = {"factor": self.rot_factor}
        return d


@dataclass(frozen=True)
class GatedDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def read(cls, r: ConfigReader) -> "GatedDeltaConfig":
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"), conv=r.integer("conv"))
        _heads(r, cfg.heads, cfg.kv_heads)
        return cfg

    def to_dict(self) -> dict:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelConfig:
    left: RotaryAttentionConfig
    right: GatedDeltaConfig

    @classmethod
    def read(cls, r: ConfigReader) -> "ParallelConfig":
        left, right = r.mapping("left"), r.mapping("right")
        if left is None or right is None:
            raise ConfigError(f"{r.where}: a parallel mixer needs 'left' and 'right'")
        return cls(RotaryAttentionConfig.read(left), GatedDeltaConfig.read(right))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int] = None     # None: the row count of the tensor ``a1``

    @classmethod
    def read(cls, r: ConfigReader) -> "GlaConfig":
        return cls(heads=r.integer("heads"), dim=r.integer("dim"), vdim=r.integer("vdim"), tau=r.number("tau"),
                   decay_rank=r.integer("decay_rank") if r.has("decay_rank") else None)

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        return d


@dataclass(frozen=True)
class MlpConfig:
    kind: str                      # "dense" or "moe"
    ff: int                        # dense: the gated unit's width; moe: an expert's
    experts: int = 0               # real experts
    identity: int = 0              # identity experts behind them in the router's outputs
    top: int = 0
    shared_ff: Optional[int] = None

    @classmethod
    def read(cls, r: ConfigReader) -> "MlpConfig":
        kind = r.string("kind")
        if kind == "dense":
            return cls(kind, r.integer("ff"))
        if kind != "moe":
            raise UnsupportedModelError(f"{r.where}: feed-forward kind '{kind}' is not known (dense, moe)")
        expert, router, shared = r.mapping("expert"), r.mapping("router"), r.mapping("shared")
        if expert is None or router is None:
            raise ConfigError(f"{r.where}: a mixture of experts needs 'expert' and 'router'")
        cfg = cls(kind, expert.integer("ff"), experts=router.integer("experts"), identity=router.integer("identity", 0, minimum=0),
                  top=router.integer("top"), shared_ff=shared.integer("ff") if shared is not None else None)
        if cfg.top > cfg.experts + cfg.identity:
            raise ConfigError(f"{r.where}: router.top ({cfg.top}) is more than the {cfg.experts + cfg.identity} experts")
        return cfg

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": self.kind}
        d = {"expert": {"ff": self.ff}, "kind": self.kind, "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


MIXER_CONFIGS = {"attention": DiffAttentionConfig, "parallel": ParallelConfig, "gla": GlaConfig}


@dataclass(frozen=True)
class MuretarLayer:
    type: str
    mixer: Union[DiffAttentionConfig, ParallelConfig, GlaConfig]
    mlp: Optional[MlpConfig]
    weights_of: Optional[int] = None

    @classmethod
    def read(cls, r: ConfigReader) -> "MuretarLayer":
        kind = r.string("type")
        if kind not in MIXER_CONFIGS:
            raise UnsupportedModelError(f"{r.where}: layer type '{kind}' is not known ({', '.join(sorted(MIXER_CONFIGS))})")
        mixer = r.mapping("mixer")
        if mixer is None:
            raise ConfigError(f"{r.where}: required key 'mixer' is missing")
        mlp = r.mapping("mlp")
        return cls(kind, MIXER_CONFIGS[kind].read(mixer), MlpConfig.read(mlp) if mlp is not None else None,
                   r.integer("weights_of", minimum=0) if r.has("weights_of") else None)

    def to_dict(self) -> dict:
        d = {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class MuretarConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[MuretarLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str = "config.json") -> "MuretarConfig":
        r = ConfigReader(raw, where)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError(f"{where}: required key 'norm' is an object")
        entries = raw.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = tuple(MuretarLayer.read(ConfigReader(e, f"{where}:layers[{i}]")) for i, e in enumerate(entries))
        cfg = cls(architecture=r.string("architecture", "Muretar"), vocab=r.integer("vocab"), width=r.integer("width"),
                  norm_eps=norm.number("eps"), layers=layers, max_positions=r.integer("max_positions", DEFAULT_MAX_POSITIONS))
        for i in range(len(layers)):
            cfg.owner(i, where)
        return cfg

    def owner(self, i: int, where: str = "config.json") -> int:
        """The layer whose tensors layer i runs: itself, or what its ``weights_of`` leads to."""
        seen = set()
        while self.layers[i].weights_of is not None:
            if i in seen:
                raise ConfigError(f"{where}: the 'weights_of' of layer {i} leads back to itself")
            seen.add(i)
            j = self.layers[i].weights_of
            if not 0 <= j < len(self.layers):
                raise ConfigError(f"{where}: layers[{i}].weights_of names layer {j} of {len(self.layers)}")
            if self.layers[j].type != self.layers[i].type:
                raise ConfigError(f"{where}: layers[{i}] is of type '{self.layers[i].type}' and cannot run the tensors of layer {j} ('{self.layers[j].type}')")
            i = j
        return i

    def with_tensor_shapes(self, shapes) -> "MuretarConfig":
        """The configuration with the sizes that only the tensors give: ``shapes()`` returns the folder's tensor
        shapes by name and is called only if something is left open."""
        open_layers = [i for i, l in enumerate(self.layers) if isinstance(l.mixer, GlaConfig) and l.mixer.decay_rank is None]
        if not open_layers:
            return self
        found = shapes()
        layers = list(self.layers)
        for i in open_layers:
            name = f"l{self.owner(i)}.mix.a1"
            if name not in found or len(found[name]) != 2:
                raise ConfigError(f"layer {i}: neither the configuration's 'decay_rank' nor a matrix '{name}' gives the size")
            layers[i] = replace(layers[i], mixer=replace(layers[i].mixer, decay_rank=int(found[name][0])))
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
             "vocab": self.vocab, "width": self.width}
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
