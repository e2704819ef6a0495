"""Typed configuration of the Dokanex architecture, read from its config.json.

The file names every size and every constant that may differ between models of the design:
``vocab``, ``width``, ``embedding.scale``, ``norm.eps``, ``logit_softcap`` and a list ``layers`` whose
entries give the layer's ``type`` (which mixer it has), the mixer's sizes (``mixer``) and its
feed-forward (``mlp``, or null for none).  Nothing here has a default that a model could
contradict, except where a whole feature may be left out (no chunks, no cap on the scores or on
the logits, no frequency scaling, keys and values of the layer's own).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple, Union

from ..errors import ConfigError, UnsupportedModelError
from .base import ConfigReader

DEFAULT_MAX_POSITIONS = 1 << 20      # the design has no position table: a bound for the block tables only


@dataclass(frozen=True)
class ChunkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float]
    chunk: Optional[int]          # None: every earlier position is seen
    kv_from: Optional[int]        # the layer whose keys and values this one attends over (None: its own)

    @classmethod
    def read(cls, r: ConfigReader) -> "ChunkAttentionConfig":
        mask = r.mapping("mask")
        cfg = cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
                  scale=r.number("scale"), softcap=r.number("softcap") if r.has("softcap") else None,
                  chunk=mask.integer("size") if mask is not None else None,
                  kv_from=r.integer("kv_from", minimum=0) if r.has("kv_from") else None)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{r.where}: heads ({cfg.heads}) must be a multiple of kv_heads ({cfg.kv_heads})")
        return cfg

    def to_dict(self) -> dict:
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        if self.chunk is not None:
            d["mask"] = {"size": self.chunk}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        return d


@dataclass(frozen=True)
class RampScalingConfig:
    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def read(cls, r: ConfigReader) -> "RampScalingConfig":
        return cls(r.number("factor"), r.number("original"), r.number("fast"), r.number("slow"))

    def to_dict(self) -> dict:
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[RampScalingConfig]

    @classmethod
    def read(cls, r: ConfigReader) -> "LatentAttentionConfig":
        rot = r.mapping("rot")
        if rot is None:
            raise ConfigError(f"{r.where}: required key 'rot' is missing")
        scaling = rot.mapping("scaling")
        cfg = cls(heads=r.integer("heads"), dim=r.integer("dim"), rot_dim=r.integer("rot_dim"), vdim=r.integer("vdim"),
                  q_rank=r.integer("q_rank"), kv_rank=r.integer("kv_rank"), scale=r.number("scale"), rot_base=rot.number("base"),
                  rot_dims=rot.integer("dims"), rot_scaling=RampScalingConfig.read(scaling) if scaling is not None else None)
        if cfg.rot_dims != cfg.rot_dim or cfg.rot_dim % 2:
            raise ConfigError(f"{r.where}: rot.dims ({cfg.rot_dims}) must equal rot_dim ({cfg.rot_dim}) and be even")
        return cfg

    def to_dict(self) -> dict:
        rot = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_dict()
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank, "rot": rot,
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class DenseConfig:
    kind: str
    ff: int

    @classmethod
    def read(cls, r: ConfigReader) -> "DenseConfig":
        kind = r.string("kind")
        if kind != "dense":
            raise UnsupportedModelError(f"{r.where}: feed-forward kind '{kind}' is not known (dense)")
        return cls(kind, r.integer("ff"))

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": self.kind}


MIXER_CONFIGS = {"attention": ChunkAttentionConfig, "latent_attention": LatentAttentionConfig}


@dataclass(frozen=True)
class DokanexLayer:
    type: str
    mixer: Union[ChunkAttentionConfig, LatentAttentionConfig]
    mlp: Optional[DenseConfig]

    @classmethod
    def read(cls, r: ConfigReader) -> "DokanexLayer":
        kind = r.string("type")
        if kind not in MIXER_CONFIGS:
            raise UnsupportedModelError(f"{r.where}: layer type '{kind}' is not known ({', '.join(sorted(MIXER_CONFIGS))})")
        mixer = r.mapping("mixer")
        if mixer is None:
            raise ConfigError(f"{r.where}: required key 'mixer' is missing")
        mlp = r.mapping("mlp")
        return cls(kind, MIXER_CONFIGS[kind].read(mixer), DenseConfig.read(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp is not None else None, "type": self.type}


@dataclass(frozen=True)
class DokanexConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    logit_softcap: Optional[float]
    layers: Tuple[DokanexLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str = "config.json") -> "DokanexConfig":
        r = ConfigReader(raw, where)
        norm, emb = r.mapping("norm"), r.mapping("embedding")
        if norm is None or emb is None:
            raise ConfigError(f"{where}: required keys 'norm' and 'embedding' are objects")
        entries = raw.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = tuple(DokanexLayer.read(ConfigReader(e, f"{where}:layers[{i}]")) for i, e in enumerate(entries))
        for i, layer in enumerate(layers):
            m = layer.mixer
            if isinstance(m, ChunkAttentionConfig) and m.kv_from is not None:
                src = layers[m.kv_from].mixer if m.kv_from < i else None
                if not isinstance(src, ChunkAttentionConfig) or src.kv_from is not None:
                    raise ConfigError(f"{where}:layers[{i}]: kv_from {m.kv_from} must name an earlier attention layer with keys and values of its own")
                if (src.kv_heads, src.dim, src.vdim) != (m.kv_heads, m.dim, m.vdim):
                    raise ConfigError(f"{where}:layers[{i}]: kv_heads, dim and vdim must equal those of layer {m.kv_from}, whose keys and values it reads")
        return cls(architecture=r.string("architecture", "Dokanex"), vocab=r.integer("vocab"), width=r.integer("width"),
                   embedding_scale=emb.number("scale", positive=False), norm_eps=norm.number("eps"),
                   logit_softcap=r.number("logit_softcap") if r.has("logit_softcap") else None, layers=layers,
                   max_positions=r.integer("max_positions", DEFAULT_MAX_POSITIONS))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
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
