"""Typed configuration of the Virusun design: a list of layers, each with one of three mixers
(differential attention; softmax attention and a matrix memory side by side; the gated delta rule)
and a dense feed-forward or none, an RMS norm on every sublayer's output. Every size and every
constant that can differ between models of the design is read from config.json; nothing is
defaulted from a known model.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError
from .rubasun_config import _need


def _positive(where: str, **numbers) -> None:
    for name, v in numbers.items():
        if v <= 0:
            raise ConfigError(f"{where}: {name} must be positive, got {v}")


@dataclass(frozen=True)
class DiffAttentionConfig:
    """Two score maps a head over one set of values, combined by difference."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    kv_from: Optional[int]     # the layer whose keys and values this one reads; None: its own

    @classmethod
    def from_dict(cls, d, where) -> "DiffAttentionConfig":
        c = cls(heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)),
                dim=int(_need(d, "dim", where)), vdim=int(_need(d, "vdim", where)),
                scale=float(_need(d, "scale", where)), diff=float(_need(d, "diff", where)),
                kv_from=None if d.get("kv_from") is None else int(d["kv_from"]))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads are not a multiple of {c.kv_heads} kv_heads")
        return c


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]]      # (factor, original, fast, slow)

    @classmethod
    def from_dict(cls, d, where, head_dim: int) -> "RotationConfig":
        sc = d.get("scaling")
        scaling = None
        if sc is not None:
            scaling = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow"))
            if min(scaling) <= 0:
                raise ConfigError(f"{where}.scaling: factor, original, fast and slow must be positive")
        c = cls(base=float(_need(d, "base", where)), dims=int(_need(d, "dims", where)), scaling=scaling)
        if c.dims < 0 or c.dims % 2 or c.dims > head_dim:
            raise ConfigError(f"{where}: dims {c.dims} must be even and at most the head's {head_dim}")
        if c.base <= 1:
            raise ConfigError(f"{where}: base must be above 1")
        return c

    def scaling_dict(self):
        if self.scaling is None:
            return None
        return dict(zip(("factor", "original", "fast", "slow"), self.scaling))


@dataclass(frozen=True)
class RotaryAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotationConfig

    @classmethod
    def from_dict(cls, d, where) -> "RotaryAttentionConfig":
        dim = int(_need(d, "dim", where))
        c = cls(heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)), dim=dim,
                vdim=int(_need(d, "vdim", where)), scale=float(_need(d, "scale", where)),
                rot=RotationConfig.from_dict(_need(d, "rot", where), where + ".rot", dim))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads are not a multiple of {c.kv_heads} kv_heads")
        return c


@dataclass(frozen=True)
class MatrixMemoryConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, d, where) -> "MatrixMemoryConfig":
        c = cls(heads=int(_need(d, "heads", where)), dim=int(_need(d, "dim", where)),
                vdim=int(_need(d, "vdim", where)), gate_cap=float(_need(d, "gate_cap", where)))
        _positive(where, heads=c.heads, dim=c.dim, vdim=c.vdim, gate_cap=c.gate_cap)
        return c


@dataclass(frozen=True)
class ParallelConfig:
    left: RotaryAttentionConfig
    right: MatrixMemoryConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, d, where) -> "ParallelConfig":
        return cls(left=RotaryAttentionConfig.from_dict(_need(d, "left", where), where + ".left"),
                   right=MatrixMemoryConfig.from_dict(_need(d, "right", where), where + ".right"),
                   left_scale=float(_need(d, "left_scale", where)), right_scale=float(_need(d, "right_scale", where)))


@dataclass(frozen=True)
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d, where) -> "DeltaConfig":
        c = cls(heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)),
                dim=int(_need(d, "dim", where)), vdim=int(_need(d, "vdim", where)), conv=int(_need(d, "conv", where)))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim, conv=c.conv)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads are not a multiple of {c.kv_heads} kv_heads")
        return c


MIXER_CONFIGS = {"attention": DiffAttentionConfig, "parallel": ParallelConfig, "delta": DeltaConfig}


@dataclass(frozen=True)
class VirusunLayerConfig:
    kind: str                  # "attention" | "parallel" | "delta"
    mixer: Any
    ff: int                    # 0: no feed-forward


@dataclass(frozen=True)
class VirusunConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: Tuple[VirusunLayerConfig, ...]
    eos_token_id: Any = None
    initializer_range: float = 0.05
    architectures: Tuple[str, ...] = ("Virusun",)
    raw: Any = None

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
    def from_dict(cls, d: Dict[str, Any]) -> "VirusunConfig":
        layers = []
        for i, e in enumerate(_need(d, "layers", "the model")):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind not in MIXER_CONFIGS:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (known: {sorted(MIXER_CONFIGS)})")
            m = MIXER_CONFIGS[kind].from_dict(_need(e, "mixer", where), where + ".mixer")
            if kind == "attention" and m.kv_from is not None:
                if not 0 <= m.kv_from < i:
                    raise ConfigError(f"{where}: kv_from {m.kv_from} must name an earlier layer")
                o = layers[m.kv_from]
                if o.kind != "attention" or o.mixer.kv_from is not None:
                    raise ConfigError(f"{where}: kv_from names layer {m.kv_from}, which has no keys and "
                                      "values of this kind of its own")
                if (o.mixer.kv_heads, o.mixer.dim, o.mixer.vdim) != (m.kv_heads, m.dim, m.vdim):
                    raise ConfigError(f"{where}: kv_heads, dim and vdim differ from layer {m.kv_from}'s")
            mlp = e.get("mlp")
            ff = 0
            if mlp is not None:
                if _need(mlp, "kind", where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown feed-forward kind {mlp['kind']!r} (known: 'dense')")
                ff = int(_need(mlp, "ff", where + ".mlp"))
                _positive(where + ".mlp", ff=ff)
            layers.append(VirusunLayerConfig(kind, m, ff))
        if not layers:
            raise ConfigError("config.json: 'layers' is empty")
        cfg = cls(vocab_size=int(_need(d, "vocab", "the model")), hidden_size=int(_need(d, "width", "the model")),
                  norm_eps=float(_need(_need(d, "norm", "the model"), "eps", "norm")), layers=tuple(layers),
                  eos_token_id=d.get("eos_token_id"), initializer_range=float(d.get("initializer_range", 0.05)),
                  raw=dict(d))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or cfg.norm_eps < 0:
            raise ConfigError("vocab and width must be positive, norm.eps not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)
