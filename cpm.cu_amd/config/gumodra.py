"""Typed configuration of Gumodra (config.json with ``"architecture": "Gumodra"``).

A list of layers, each with a mixer of its own kind and sizes and an optional feed-forward:

    {"architecture": "Gumodra", "vocab": V, "width": W, "norm": {"eps": e}, "embedding": {"scale": s},
     "layers": [{"type": "attention" | "mlstm", "mixer": {...}, "mlp": {...} | null}, ...]}

mixer of ``attention``: heads, kv_heads, dim, vdim (the values are the projected keys, so vdim equals dim),
scale, rot {base, dims}, optional mask {size, keep_first}; of ``mlstm``: heads, dim, vdim, gate_cap.
mlp: {kind: "dense", ff} or {kind: "moe", expert {ff}, router {experts, top, optional groups {count, keep}},
optional shared {ff}}.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, field_from, require

ARCHITECTURE = "Gumodra"
MIXER_KINDS = ("attention", "mlstm")


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int] = None          # None: every earlier token is seen
    keep_first: int = 0                   # tokens at the start of the sequence that stay visible past the window

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        rot = raw.get("rot")
        require(rot is None or isinstance(rot, dict), f"{where}: 'rot' must be an object")
        mask = raw.get("mask")
        require(mask is None or isinstance(mask, dict), f"{where}: 'mask' must be an object")
        rot_dims = field_from(rot, "dims", int, 0, where=where + " rot") if rot is not None else 0
        c = cls(g("heads"), field_from(raw, "kv_heads", int, g("heads"), where=where), g("dim"),
                field_from(raw, "vdim", int, g("dim"), where=where), field_from(raw, "scale", float, where=where),
                field_from(rot, "base", float, where=where + " rot") if rot_dims else 10000.0, rot_dims,
                field_from(mask, "size", int, None, where=where + " mask") if mask is not None else None,
                field_from(mask, "keep_first", int, 0, where=where + " mask") if mask is not None else 0)
        require(min(c.heads, c.kv_heads, c.dim) > 0, f"{where}: sizes must be positive")
        require(c.heads % c.kv_heads == 0, f"{where}: heads ({c.heads}) must be a multiple of kv_heads ({c.kv_heads})")
        require(c.vdim == c.dim, f"{where}: vdim ({c.vdim}) must equal dim ({c.dim}): the values are the projected keys")
        require(c.rot_dims >= 0 and c.rot_dims % 2 == 0 and c.rot_dims <= c.dim,
                f"{where}: rot.dims ({c.rot_dims}) must be even and at most dim ({c.dim})")
        require(c.rot_dims == 0 or c.rot_base > 1.0, f"{where}: rot.base must exceed 1")
        require(c.window is None or c.window > 0, f"{where}: mask.size must be positive")
        require(c.keep_first >= 0, f"{where}: mask.keep_first must not be negative")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return d


@dataclass(frozen=True)
class MLSTMConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str):
        g = lambda k: field_from(raw, k, int, where=where)
        c = cls(g("heads"), g("dim"), field_from(raw, "vdim", int, g("dim"), where=where),
                field_from(raw, "gate_cap", float, where=where))
        require(min(c.heads, c.dim, c.vdim) > 0, f"{where}: sizes must be positive")
        require(c.gate_cap > 0, f"{where}: gate_cap must be positive")
        return c

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                             # 'dense' or 'moe'
    ff: int                               # width of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    groups: Optional[Tuple[int, int]] = None      # (count, keep), None: any expert may be chosen
    shared_ff: Optional[int] = None               # width of the expert every token uses, None: there is none

    @classmethod
    def from_dict(cls, raw: Any, where: str):
        require(isinstance(raw, dict), f"{where}: 'mlp' must be an object or null")
        kind = field_from(raw, "kind", str, where=where)
        if kind == "dense":
            c = cls(kind, field_from(raw, "ff", int, where=where))
            require(c.ff > 0, f"{where}: ff must be positive")
            return c
        if kind != "moe":
            raise ConfigError(f"{where}: kind '{kind}' is not supported (supported: dense, moe)")
        expert, router, shared = raw.get("expert"), raw.get("router"), raw.get("shared")
        require(isinstance(expert, dict), f"{where}: 'expert' must be an object")
        require(isinstance(router, dict), f"{where}: 'router' must be an object")
        require(shared is None or isinstance(shared, dict), f"{where}: 'shared' must be an object")
        groups = router.get("groups")
        require(groups is None or isinstance(groups, dict), f"{where} router: 'groups' must be an object")
        c = cls(kind, field_from(expert, "ff", int, where=where + " expert"),
                field_from(router, "experts", int, where=where + " router"),
                field_from(router, "top", int, where=where + " router"),
                (field_from(groups, "count", int, where=where + " router groups"),
                 field_from(groups, "keep", int, where=where + " router groups")) if groups is not None else None,
                field_from(shared, "ff", int, where=where + " shared") if shared is not None else None)
        require(c.ff > 0 and c.experts > 0, f"{where}: sizes must be positive")
        require(0 < c.top <= c.experts, f"{where} router: top ({c.top}) must lie in 1..experts ({c.experts})")
        if c.groups is not None:
            count, keep = c.groups
            require(count > 0 and c.experts % count == 0,
                    f"{where} router: experts ({c.experts}) must split into groups.count ({count}) equal groups")
            require(0 < keep <= count, f"{where} router: groups.keep ({keep}) must lie in 1..count ({count})")
            require(c.top <= keep * (c.experts // count),
                    f"{where} router: top ({c.top}) exceeds the experts of the {keep} groups that may be chosen from")
        require(c.shared_ff is None or c.shared_ff > 0, f"{where} shared: ff must be positive")
        return c

    def to_dict(self):
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        d: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff}, "router": router}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


_MIXER_CONFIGS = {"attention": WindowAttentionConfig, "mlstm": MLSTMConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    mlp: Optional[FeedForwardConfig]      # None: the layer has no feed-forward

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
        return cls(kind, mixer, FeedForwardConfig.from_dict(mlp, where + " mlp") if mlp is not None else None)

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": self.mlp.to_dict() if self.mlp else None}


@dataclass(frozen=True)
class GumodraConfig(ModelConfig):
    vocab: int = 0
    width: int = 0
    eps: float = 1e-6
    embedding_scale: float = 1.0
    layers: Tuple[LayerConfig, ...] = ()

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "GumodraConfig":
        vocab, width = field_from(raw, "vocab", int), field_from(raw, "width", int)
        require(vocab > 0 and width > 0, "config.json: vocab and width must be positive")
        norm = raw.get("norm")
        require(isinstance(norm, dict), "config.json: 'norm' must be an object with 'eps'")
        eps = field_from(norm, "eps", float, where="config.json norm")
        require(eps >= 0, "config.json norm: eps must not be negative")
        emb = raw.get("embedding")
        require(emb is None or isinstance(emb, dict), "config.json: 'embedding' must be an object")
        scale = field_from(emb, "scale", float, 1.0, where="config.json embedding") if emb is not None else 1.0
        layers = raw.get("layers")
        require(isinstance(layers, list) and len(layers) > 0, "config.json: 'layers' must be a non-empty list")
        return cls(ARCHITECTURE, vocab, width, eps, scale, tuple(LayerConfig.from_dict(l, i) for i, l in enumerate(layers)))

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "embedding": {"scale": self.embedding_scale}, "layers": [l.to_dict() for l in self.layers]}

    @property
    def vocabulary_size(self) -> int:
        return self.vocab
