"""Typed configuration of the Rubasun design: a list of layers, each with a latent-attention
mixer and a dense, routed or absent feed-forward, Dynamic-Tanh norms around every sublayer, a
scaled embedding and a per-layer token input. Every size and every constant that can differ
between models of the design is read from config.json; nothing is defaulted from a known model.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError


def _need(d: Dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or d.get(key) is None:
        raise ConfigError(f"config.json: {where} lacks {key!r}")
    return d[key]


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int               # unrotated query/key entries a head
    rot_dim: int           # rotated entries a head (and of the shared key part)
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int          # entries of the rotated part that turn
    kv_from: Optional[int] # the layer whose latent cache this one reads; None: its own

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "LatentMixerConfig":
        rot = _need(d, "rot", where)
        c = cls(heads=int(_need(d, "heads", where)), dim=int(_need(d, "dim", where)),
                rot_dim=int(_need(d, "rot_dim", where)), vdim=int(_need(d, "vdim", where)),
                kv_rank=int(_need(d, "kv_rank", where)), scale=float(_need(d, "scale", where)),
                rot_base=float(_need(rot, "base", where + ".rot")),
                rot_dims=int(_need(rot, "dims", where + ".rot")),
                kv_from=None if d.get("kv_from") is None else int(d["kv_from"]))
        if min(c.heads, c.vdim, c.kv_rank) <= 0 or c.dim < 0 or c.rot_dim < 0 or c.dim + c.rot_dim <= 0:
            raise ConfigError(f"{where}: sizes must be positive")
        if c.rot_dim % 2 or c.rot_dims % 2 or not 0 <= c.rot_dims <= c.rot_dim:
            raise ConfigError(f"{where}: rot_dim {c.rot_dim} and rot.dims {c.rot_dims} must be even, "
                              "the second at most the first")
        if c.rot_base <= 0:
            raise ConfigError(f"{where}: rot.base must be positive")
        return c


@dataclass(frozen=True)
class ExpertConfig:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d, where) -> "ExpertConfig":
        c = cls(int(_need(d, "ff", where)), float(_need(d, "limit", where)))
        if c.ff <= 0:
            raise ConfigError(f"{where}: ff must be positive")
        return c


@dataclass(frozen=True)
class MlpConfig:
    kind: str                              # "dense" | "moe"
    ff: int = 0                            # dense
    experts: int = 0                       # moe
    top: int = 0
    expert: Optional[ExpertConfig] = None
    shared: Optional[ExpertConfig] = None

    @classmethod
    def from_dict(cls, d, where) -> Optional["MlpConfig"]:
        if d is None:
            return None
        kind = _need(d, "kind", where)
        if kind == "dense":
            ff = int(_need(d, "ff", where))
            if ff <= 0:
                raise ConfigError(f"{where}: ff must be positive")
            return cls("dense", ff=ff)
        if kind == "moe":
            router = _need(d, "router", where)
            c = cls("moe", experts=int(_need(router, "experts", where + ".router")),
                    top=int(_need(router, "top", where + ".router")),
                    expert=ExpertConfig.from_dict(_need(d, "expert", where), where + ".expert"),
                    shared=(ExpertConfig.from_dict(d["shared"], where + ".shared")
                            if d.get("shared") is not None else None))
            if not 0 < c.top <= c.experts:
                raise ConfigError(f"{where}: top {c.top} of {c.experts} experts")
            return c
        raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: 'dense', 'moe')")


@dataclass(frozen=True)
class RubasunLayerConfig:
    mixer: LatentMixerConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class RubasunConfig:
    vocab_size: int
    hidden_size: int
    embedding_scale: float
    norm_eps: float
    token_side_dim: int                    # 0: no per-layer token input
    layers: Tuple[RubasunLayerConfig, ...]
    eos_token_id: Any = None
    initializer_range: float = 0.05
    architectures: Tuple[str, ...] = ("Rubasun",)
    raw: Any = None                        # the dict it was read from (to_dict)

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        e = self.eos_token_id
        if e is None:
            return ()
        return tuple(int(x) for x in e) if isinstance(e, (list, tuple)) else (int(e),)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "RubasunConfig":
        layers = []
        entries = _need(d, "layers", "the model")
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind != "latent_attention":
                raise ConfigError(f"{where}: unknown layer type {kind!r} (known: 'latent_attention')")
            m = LatentMixerConfig.from_dict(_need(e, "mixer", where), where + ".mixer")
            if m.kv_from is not None:
                if not 0 <= m.kv_from < i:
                    raise ConfigError(f"{where}: kv_from {m.kv_from} must name an earlier layer")
                o = layers[m.kv_from].mixer
                if o.kv_from is not None:
                    raise ConfigError(f"{where}: kv_from names layer {m.kv_from}, which has no cache of its own")
                if (o.kv_rank, o.rot_dim, o.rot_base, o.rot_dims) != (m.kv_rank, m.rot_dim, m.rot_base, m.rot_dims):
                    raise ConfigError(f"{where}: kv_rank, rot_dim and rotation differ from layer {m.kv_from}'s")
            layers.append(RubasunLayerConfig(m, MlpConfig.from_dict(e.get("mlp"), where + ".mlp")))
        side = d.get("token_side")
        cfg = cls(vocab_size=int(_need(d, "vocab", "the model")), hidden_size=int(_need(d, "width", "the model")),
                  embedding_scale=float(_need(_need(d, "embedding", "the model"), "scale", "embedding")),
                  norm_eps=float(_need(_need(d, "norm", "the model"), "eps", "norm")),
                  token_side_dim=int(_need(side, "dim", "token_side")) if side else 0,
                  layers=tuple(layers), eos_token_id=d.get("eos_token_id"),
                  initializer_range=float(d.get("initializer_range", 0.05)), raw=dict(d))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or cfg.token_side_dim < 0 or cfg.norm_eps < 0:
            raise ConfigError("vocab and width must be positive, token_side.dim and norm.eps not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)
