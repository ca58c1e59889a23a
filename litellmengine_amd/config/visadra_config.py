"""Visadra: a decoder whose layers are listed one by one in config.json, each with a mixer
(a gated recurrence or latent attention) and a feed-forward (dense, routed, or none).

config.json keys: `architecture` (a string), `vocab`, `width`, `embedding.scale`,
`logit_scale`, `norm.eps`, and `layers`: a list of `{type, mixer: {...}, mlp: {...} | null}`.
Every size and every constant that may differ between models is read from there; nothing of
it stands in code.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError, _optional, _required

MINGRU_TYPES = ("mingru", "mingru_2")  # two names of the same gated recurrence
LATENT_ATTENTION = "latent_attention"
MIXER_TYPES = MINGRU_TYPES + (LATENT_ATTENTION,)
DENSE, MOE = "dense", "moe"


def _section(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where} needs an object `{key}`")
    return v


@dataclasses.dataclass(frozen=True)
class MinGRUSizes:
    width: int


@dataclasses.dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int  # plain (unrotated) query/key elements per head
    rot_dim: int  # rotated query/key elements per head; the key's are shared by all heads
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int  # how many of the rot_dim elements are rotated (the rest pass unchanged)
    window: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class FeedForwardSizes:
    kind: str
    ff: int = 0  # dense: inner width; moe: inner width of one routed expert
    experts: int = 0
    top: int = 0
    shared_ff: int = 0  # moe: inner width of the expert that every token uses (0: none)


@dataclasses.dataclass(frozen=True)
class VisadraLayer:
    type: str
    mixer: Any  # MinGRUSizes or LatentAttentionSizes
    mlp: Optional[FeedForwardSizes]


def _positive(value: int, what: str) -> int:
    if value <= 0:
        raise ConfigError(f"Visadra config {what} must be positive")
    return value


def _mixer_from(kind: str, m: Dict[str, Any], where: str):
    if kind in MINGRU_TYPES:
        return MinGRUSizes(_positive(_required(m, "width", int), f"{where}.mixer.width"))
    rot = m.get("rot") if isinstance(m.get("rot"), dict) else {}
    rot_dim = _positive(_required(m, "rot_dim", int), f"{where}.mixer.rot_dim")
    rot_dims = _optional(rot, "dims", int, rot_dim)
    if rot_dims % 2 or not 0 <= rot_dims <= rot_dim:
        raise ConfigError(f"{where}.mixer.rot.dims must be even and at most rot_dim")
    window = _optional(m, "window", int, None)
    if window is not None and window <= 0:
        raise ConfigError(f"{where}.mixer.window must be positive")
    sizes = LatentAttentionSizes(
        heads=_positive(_required(m, "heads", int), f"{where}.mixer.heads"),
        dim=_positive(_required(m, "dim", int), f"{where}.mixer.dim"),
        rot_dim=rot_dim,
        vdim=_positive(_required(m, "vdim", int), f"{where}.mixer.vdim"),
        kv_rank=_positive(_required(m, "kv_rank", int), f"{where}.mixer.kv_rank"),
        scale=_optional(m, "scale", float, 0.0),
        rot_base=_optional(rot, "base", float, 10000.0),
        rot_dims=rot_dims,
        window=window,
    )
    if not sizes.rot_base > 0.0:
        raise ConfigError(f"{where}.mixer.rot.base must be positive")
    if "scale" not in m or m["scale"] is None:  # the usual one: over all query/key elements of a head
        sizes = dataclasses.replace(sizes, scale=float(sizes.dim + sizes.rot_dim) ** -0.5)
    return sizes


def _mlp_from(m: Optional[Dict[str, Any]], where: str) -> Optional[FeedForwardSizes]:
    if m is None:
        return None
    if not isinstance(m, dict):
        raise ConfigError(f"{where}.mlp must be an object or null")
    kind = m.get("kind")
    act = m.get("act", "silu")
    if act != "silu":
        raise ConfigError(f"{where}.mlp.act={act!r} is not supported (the gate's activation is silu)")
    if kind == DENSE:
        return FeedForwardSizes(DENSE, ff=_positive(_required(m, "ff", int), f"{where}.mlp.ff"))
    if kind == MOE:
        router = _section(m, "router", f"{where}.mlp")
        expert = _section(m, "expert", f"{where}.mlp")
        shared = m.get("shared")
        experts = _positive(_required(router, "experts", int), f"{where}.mlp.router.experts")
        top = _positive(_required(router, "top", int), f"{where}.mlp.router.top")
        if top > experts:
            raise ConfigError(f"{where}.mlp.router.top is larger than the number of experts")
        return FeedForwardSizes(
            MOE, ff=_positive(_required(expert, "ff", int), f"{where}.mlp.expert.ff"), experts=experts, top=top,
            shared_ff=_positive(_required(shared, "ff", int), f"{where}.mlp.shared.ff") if shared else 0,
        )
    raise ConfigError(f"{where}.mlp.kind={kind!r} is unknown (dense, moe)")


@dataclasses.dataclass(frozen=True)
class VisadraConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    layers: Tuple[VisadraLayer, ...]

    ARCHITECTURE = "Visadra"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VisadraConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("Missing required config field: layers")
        out = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                kind = layer.get("type") if isinstance(layer, dict) else layer
                raise ConfigError(f"{where}.type={kind!r} is unknown ({', '.join(MIXER_TYPES)})")
            out.append(VisadraLayer(layer["type"], _mixer_from(layer["type"], _section(layer, "mixer", where), where),
                                    _mlp_from(layer.get("mlp"), where)))
        cfg = cls(
            architecture=str(d.get("architecture") or (d.get("architectures") or [cls.ARCHITECTURE])[0]),
            vocab=_positive(_required(d, "vocab", int), "vocab"),
            width=_positive(_required(d, "width", int), "width"),
            embedding_scale=_optional(d.get("embedding") or {}, "scale", float, 1.0),
            logit_scale=_optional(d, "logit_scale", float, 1.0),
            norm_eps=_required(_section(d, "norm", "Visadra config"), "eps", float),
            layers=tuple(out),
        )
        if not cfg.norm_eps > 0.0:
            raise ConfigError("Visadra config norm.eps must be positive")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, MinGRUSizes):
                mixer: Dict[str, Any] = {"width": m.width}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                         "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.window is not None:
                    mixer["window"] = m.window
            f = layer.mlp
            if f is None:
                mlp = None
            elif f.kind == DENSE:
                mlp = {"kind": DENSE, "ff": f.ff}
            else:
                mlp = {"kind": MOE, "router": {"experts": f.experts, "top": f.top}, "expert": {"ff": f.ff}}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                "norm": {"eps": self.norm_eps}, "layers": layers}
