"""Typed configuration of Duvulix (config.json with ``"architecture": "Duvulix"``).

A list of layers, each with a mixer of its own kind and sizes and an optional feed-forward:

    {"architecture": "Duvulix", "vocab": V, "width": W, "norm": {"eps": e},
     "layers": [{"type": "latent_attention" | "attention" | "mamba2", "mixer": {...}, "mlp": {...} | null}, ...]}

mixer of ``latent_attention``: heads, dim, rot_dim, vdim, kv_rank, scale, rot {base, dims}, optional kv_from
(the layer whose latent cache this layer reads); of ``attention``: heads, kv_heads, dim, vdim, scale,
rot {base, dims, optional scaling {factor, original, fast, slow}}, optional mask {size}; of ``mamba2``: heads,
vdim, state, groups, conv, norm_groups.  mlp: {kind: "dense", ff}.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, field_from, require

ARCHITECTURE = "Duvulix"
MIXER_KINDS = ("latent_attention", "attention", "mamba2")


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    # YaRN scaling (factor, original, fast, slow), or None
    scaling: Optional[Tuple[float, int, float, float]] = None

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "Rotation":
        require(isinstance(raw, dict), f"{where}: 'rot' must be an object")
        base, dims = field_from(raw, "base", float, where=where), field_from(raw, "dims", int, where=where)
        require(base > 1.0, f"{where}: rot.base must exceed 1")
        require(dims >= 0 and dims % 2 == 0, f"{where}: rot.dims ({dims}) must be even")
        sc = raw.get("scaling")
        scaling = None
        if sc is not None:
            require(isinstance(sc, dict), f"{where}: rot.scaling must be an object")
            w = where + " rot.scaling"
            scaling = (field_from(sc, "factor", float, where=w), field_from(sc, "original", int, where=w),
                       field_from(sc, "fast", float, where=w), field_from(sc, "slow", float, where=w))
            require(scaling[0] > 0 and scaling[1] > 0 and scaling[2] > 0 and scaling[3] > 0,
                    f"{w}: factor, original, fast and slow must be positive")
        return cls(base, dims, scaling)

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: Rotation
    kv_from: Optional[int] = None

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        c = cls(g("heads"), g("dim"), g("rot_dim"), g("vdim"), g("kv_rank"), field_from(raw, "scale", float, where=where),
                Rotation.from_dict(raw.get("rot"), where), field_from(raw, "kv_from", int, None, where=where))
        require(min(c.heads, c.dim, c.vdim, c.kv_rank) > 0 and c.rot_dim >= 0, f"{where}: sizes must be positive")
        require(c.rot.dims == c.rot_dim, f"{where}: rot.dims ({c.rot.dims}) must equal rot_dim ({c.rot_dim})")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "scale": self.scale, "rot": self.rot.to_dict()}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation
    mask_size: Optional[int] = None

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        mask = raw.get("mask")
        require(mask is None or isinstance(mask, dict), f"{where}: 'mask' must be an object")
        # a configuration that leaves these out means the plain case: a kv head a head, values as wide as keys
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), g("dim"),
                field_from(raw, "vdim", int, g("dim"), where=where), field_from(raw, "scale", float, where=where),
                Rotation.from_dict(raw.get("rot"), where),
                field_from(mask, "size", int, where=where + " mask") if mask is not None else None)
        require(min(c.heads, c.kv_heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.rot.dims <= c.dim, f"{where}: rot.dims ({c.rot.dims}) exceeds dim ({c.dim})")
        require(c.mask_size is None or c.mask_size > 0, f"{where}: mask.size must be positive")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict()}
        if self.mask_size is not None:
            d["mask"] = {"size": self.mask_size}
        return d


@dataclass(frozen=True)
class Mamba2Config:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        c = cls(field_from(raw, "heads", int, where=where), field_from(raw, "vdim", int, where=where),
                field_from(raw, "state", int, where=where), field_from(raw, "groups", int, 1, where=where),
                field_from(raw, "conv", int, where=where), field_from(raw, "norm_groups", int, 1, where=where))
        require(min(c.heads, c.vdim, c.state, c.groups, c.conv, c.norm_groups) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.groups == 0, f"{where}: heads ({c.heads}) must be a multiple of groups ({c.groups})")
        require((c.heads * c.vdim) % c.norm_groups == 0,
                f"{where}: heads * vdim ({c.heads * c.vdim}) must split into norm_groups ({c.norm_groups}) equal parts")
        return c

    def to_dict(self):
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


_MIXER_CONFIGS = {"latent_attention": LatentAttentionConfig, "attention": AttentionConfig, "mamba2": Mamba2Config}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    ff: Optional[int]             # feed-forward width, None: the layer has no feed-forward

    @classmethod
    def from_dict(cls, raw: Any, i: int):
        where = f"config.json layers[{i}]"
        require(isinstance(raw, dict), f"{where}: must be an object")
        kind = field_from(raw, "type", str, where=where)
        if kind not in _MIXER_CONFIGS:
            raise ConfigError(f"{where}: type '{kind}' is not supported (supported: {', '.join(MIXER_KINDS)})")
        require(isinstance(raw.get("mixer"), dict), f"{where}: 'mixer' must be an object")
        mixer = _MIXER_CONFIGS[kind].from_dict(raw["mixer"], where + " mixer")
        mlp = raw.get("mlp")
        ff = None
        if mlp is not None:
            require(isinstance(mlp, dict), f"{where}: 'mlp' must be an object or null")
            mk = field_from(mlp, "kind", str, where=where + " mlp")
            if mk != "dense":
                raise ConfigError(f"{where} mlp: kind '{mk}' is not supported (supported: dense)")
            ff = field_from(mlp, "ff", int, where=where + " mlp")
            require(ff > 0, f"{where} mlp: ff must be positive")
        return cls(kind, mixer, ff)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(),
                "mlp": {"kind": "dense", "ff": self.ff} if self.ff is not None else None}


@dataclass(frozen=True)
class DuvulixConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    eps: float = 1e-6
    layers: Tuple[LayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DuvulixConfig":
        vocab, width = field_from(raw, "vocab", int), field_from(raw, "width", int)
        require(vocab > 0 and width > 0, "config.json: vocab and width must be positive")
        norm = raw.get("norm")
        require(isinstance(norm, dict), "config.json: 'norm' must be an object with 'eps'")
        eps = field_from(norm, "eps", float, where="config.json norm")
        require(eps >= 0, "config.json norm: eps must not be negative")
        layers = raw.get("layers")
        require(isinstance(layers, list) and len(layers) > 0, "config.json: 'layers' must be a non-empty list")
        cfg = cls(ARCHITECTURE, vocab, width, eps, tuple(LayerConfig.from_dict(l, i) for i, l in enumerate(layers)))
        for i, l in enumerate(cfg.layers):
            j = getattr(l.mixer, "kv_from", None)
            if j is None:
                continue
            where = f"config.json layers[{i}] mixer"
            require(0 <= j < i, f"{where}: kv_from ({j}) must name an earlier layer")
            src = cfg.layers[j]
            require(src.type == "latent_attention" and src.mixer.kv_from is None,
                    f"{where}: kv_from names layer {j}, which has no latent cache of its own")
            require((src.mixer.kv_rank, src.mixer.rot_dim, src.mixer.rot) == (l.mixer.kv_rank, l.mixer.rot_dim, l.mixer.rot),
                    f"{where}: kv_rank, rot_dim and rot must equal those of layer {j}, whose cache this layer reads")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [l.to_dict() for l in self.layers]}

    @property
    def vocabulary_size(self) -> int:
        return self.vocab
