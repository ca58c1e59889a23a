"""Kezasun: a decoder whose layers are listed one by one in config.json.  Every layer is
`x <- x + residual_mult * (mixer(h) + ff(h))` with one norm `h = norm1(x)` for both sublayers;
the mixer is a `wkv` recurrence (a matrix state per head with data-dependent decay) or
windowed grouped-query `attention` with a sink, the feed-forward a routed one or none.

config.json keys: `architecture` (a string), `vocab`, `width`, `residual_mult`, `norm.eps`, and
`layers`: a list of `{type, mixer: {...}, mlp: {...} | null}`:

  wkv        mixer: heads, dim                 (the decay's inner rank is the shape of `mix.w1`;
                                                a config may also say it as `decay_rank`)
  attention  mixer: heads, kv_heads, dim, vdim, scale, mask.size (absent: every earlier token
             is seen), rot.{base, dims, scaling.{factor, low, high, original}}, kv_from (the
             layer whose keys and values this one reads instead of making its own)
  mlp        kind "moe": router.{experts, top, identity, groups.{count, keep}}, expert.ff

Every size and every constant that may differ between models is read from there (or from a
tensor's shape); nothing of it stands in code.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Mapping, Optional, Tuple

from .model_config import ConfigError, _optional, _required

WKV, ATTENTION = "wkv", "attention"
MIXER_TYPES = (WKV, ATTENTION)
MOE = "moe"


def _section(d: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where} needs an object `{key}`")
    return v


def _positive(value: int, what: str) -> int:
    if value <= 0:
        raise ConfigError(f"Kezasun config {what} must be positive")
    return value


@dataclasses.dataclass(frozen=True)
class WKVSizes:
    heads: int
    dim: int
    decay_rank: Optional[int] = None  # None until a checkpoint's shapes have said it


@dataclasses.dataclass(frozen=True)
class FrequencyScaling:
    """Long wavelengths of a rotation are stretched by `factor`; `low` and `high` bound the band
    (in turns per `original` positions) in which the stretch fades out."""

    factor: float
    low: float
    high: float
    original: float


@dataclasses.dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    rot_scaling: Optional[FrequencyScaling] = None
    window: Optional[int] = None
    kv_from: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class RoutedSizes:
    experts: int  # experts with weights
    identity: int  # experts after them that hand their input on
    top: int
    ff: int
    groups: int = 1
    groups_kept: int = 1


@dataclasses.dataclass(frozen=True)
class KezasunLayer:
    type: str
    mixer: Any  # WKVSizes or AttentionSizes
    mlp: Optional[RoutedSizes]


def _mixer_from(kind: str, m: Dict[str, Any], where: str):
    heads = _positive(_required(m, "heads", int), f"{where}.mixer.heads")
    dim = _positive(_required(m, "dim", int), f"{where}.mixer.dim")
    if kind == WKV:
        rank = _optional(m, "decay_rank", int, None)
        if rank is not None:
            _positive(rank, f"{where}.mixer.decay_rank")
        return WKVSizes(heads, dim, rank)
    kv_heads = _positive(_optional(m, "kv_heads", int, heads), f"{where}.mixer.kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}.mixer.heads must be a multiple of kv_heads")
    rot = m.get("rot") if isinstance(m.get("rot"), dict) else {}
    rot_dims = _optional(rot, "dims", int, 0)
    if rot_dims % 2 or not 0 <= rot_dims <= dim:
        raise ConfigError(f"{where}.mixer.rot.dims must be even and at most dim")
    scaling = None
    if isinstance(rot.get("scaling"), dict):
        s = rot["scaling"]
        scaling = FrequencyScaling(_required(s, "factor", float), _required(s, "low", float), _required(s, "high", float),
                                   _required(s, "original", float))
        if not (scaling.factor > 0 and scaling.high > scaling.low and scaling.original > 0):
            raise ConfigError(f"{where}.mixer.rot.scaling needs factor > 0, high > low and original > 0")
    mask = m.get("mask") if isinstance(m.get("mask"), dict) else {}
    window = _optional(mask, "size", int, None)
    if window is not None:
        _positive(window, f"{where}.mixer.mask.size")
    kv_from = _optional(m, "kv_from", int, None)
    sizes = AttentionSizes(
        heads=heads, kv_heads=kv_heads, dim=dim,
        vdim=_positive(_optional(m, "vdim", int, dim), f"{where}.mixer.vdim"),
        scale=_optional(m, "scale", float, float(dim) ** -0.5),
        rot_base=_optional(rot, "base", float, 10000.0), rot_dims=rot_dims, rot_scaling=scaling, window=window,
        kv_from=kv_from,
    )
    if not sizes.rot_base > 0.0:
        raise ConfigError(f"{where}.mixer.rot.base must be positive")
    return sizes


def _mlp_from(m: Optional[Dict[str, Any]], where: str) -> Optional[RoutedSizes]:
    if m is None:
        return None
    if not isinstance(m, dict):
        raise ConfigError(f"{where}.mlp must be an object or null")
    if m.get("kind", MOE) != MOE:
        raise ConfigError(f"{where}.mlp.kind={m.get('kind')!r} is unknown (moe)")
    router = _section(m, "router", f"{where}.mlp")
    experts = _positive(_required(router, "experts", int), f"{where}.mlp.router.experts")
    identity = _optional(router, "identity", int, 0)
    top = _positive(_required(router, "top", int), f"{where}.mlp.router.top")
    groups = router.get("groups") if isinstance(router.get("groups"), dict) else {}
    count = _positive(_optional(groups, "count", int, 1), f"{where}.mlp.router.groups.count")
    keep = _positive(_optional(groups, "keep", int, count), f"{where}.mlp.router.groups.keep")
    total = experts + identity
    if identity < 0 or total % count or keep > count:
        raise ConfigError(f"{where}.mlp.router: experts and identity experts together form `groups.count` equal groups, "
                          f"of which at most all are kept")
    if top > keep * (total // count):
        raise ConfigError(f"{where}.mlp.router.top is larger than the number of experts in the kept groups")
    return RoutedSizes(experts, identity, top, _positive(_required(_section(m, "expert", f"{where}.mlp"), "ff", int),
                                                         f"{where}.mlp.expert.ff"), count, keep)


@dataclasses.dataclass(frozen=True)
class KezasunConfig:
    architecture: str
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    layers: Tuple[KezasunLayer, ...]

    ARCHITECTURE = "Kezasun"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "KezasunConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("Missing required config field: layers")
        out = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                kind = layer.get("type") if isinstance(layer, dict) else layer
                raise ConfigError(f"{where}.type={kind!r} is unknown ({', '.join(MIXER_TYPES)})")
            mixer = _section(layer, "mixer", where)
            src = mixer.get("kv_from")
            if (layer["type"] == ATTENTION and isinstance(src, int) and not isinstance(src, bool) and 0 <= src < i
                    and isinstance(layers[src], dict) and isinstance(layers[src].get("mixer"), dict)):
                # what a reading layer shares with the layer it reads may be left out of its own entry
                shared = {k: layers[src]["mixer"][k] for k in ("kv_heads", "dim", "vdim", "rot") if k in layers[src]["mixer"]}
                mixer = {**shared, **mixer}
            out.append(KezasunLayer(layer["type"], _mixer_from(layer["type"], mixer, where), _mlp_from(layer.get("mlp"), where)))
        for i, layer in enumerate(out):
            src = layer.mixer.kv_from if layer.type == ATTENTION else None
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if not 0 <= src < i or out[src].type != ATTENTION or out[src].mixer.kv_from is not None:
                raise ConfigError(f"{where} must name an earlier attention layer that makes keys and values of its own")
            a, b = layer.mixer, out[src].mixer
            same = ("kv_heads", "dim", "vdim", "rot_base", "rot_dims", "rot_scaling")
            if any(getattr(a, k) != getattr(b, k) for k in same):
                raise ConfigError(f"{where}: the two layers' key/value heads, sizes and rotation must be equal")
        cfg = cls(
            architecture=str(d.get("architecture") or (d.get("architectures") or [cls.ARCHITECTURE])[0]),
            vocab=_positive(_required(d, "vocab", int), "vocab"),
            width=_positive(_required(d, "width", int), "width"),
            residual_mult=_optional(d, "residual_mult", float, 1.0),
            norm_eps=_required(_section(d, "norm", "Kezasun config"), "eps", float),
            layers=tuple(out),
        )
        if not cfg.norm_eps > 0.0:
            raise ConfigError("Kezasun config norm.eps must be positive")
        return cfg

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "KezasunConfig":
        """The sizes that config.json leaves to the checkpoint, read from its tensors' shapes: the
        inner rank of every wkv layer's decay (rows of `l<i>.mix.w1`)."""
        layers = []
        for i, layer in enumerate(self.layers):
            if layer.type == WKV and layer.mixer.decay_rank is None:
                shape = shapes.get(f"l{i}.mix.w1")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"layers[{i}]: the checkpoint has no matrix l{i}.mix.w1 to read the decay's rank from")
                layer = dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, decay_rank=int(shape[0])))
            layers.append(layer)
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, WKVSizes):
                mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim}
                if m.decay_rank is not None:
                    mixer["decay_rank"] = m.decay_rank
            else:
                rot: Dict[str, Any] = {"base": m.rot_base, "dims": m.rot_dims}
                if m.rot_scaling is not None:
                    s = m.rot_scaling
                    rot["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "rot": rot}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            f = layer.mlp
            mlp = None if f is None else {
                "kind": MOE, "expert": {"ff": f.ff},
                "router": {"experts": f.experts, "identity": f.identity, "top": f.top,
                           "groups": {"count": f.groups, "keep": f.groups_kept}},
            }
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps}, "layers": layers}
