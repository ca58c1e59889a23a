"""Visadra: how its configuration becomes parts.

The layers are listed one by one in the configuration; layer i's tensors start with `l<i>.`,
its mixer's with `l<i>.mix.`, its feed-forward's with `l<i>.mlp.`.  Every layer is a block
whose norms (one gain for all coordinates) sit on the sublayers' outputs; the mixer is a
minGRU recurrence or latent attention, the feed-forward a dense gated one, a routed one with a
shared expert, or none.  The embedding's rows are scaled on their way into the residual
stream and the logits on their way out.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.visadra_config import (DENSE, LATENT_ATTENTION, MINGRU_TYPES, FeedForwardSizes, VisadraConfig,
                                     VisadraLayer)
from ..parts import (Embedding, GatedMLP, LatentAttention, Linear, MinGRU, PostNormBlock, RMSNorm, RotaryInterleaved,
                     RoutedMLP)
from .decoder import DecoderLM, PlanEntry

_FF_NAMES = ("gate", "up", "down")


def _mixer(c: VisadraConfig, layer: VisadraLayer, prefix: str):
    m = layer.mixer
    if layer.type in MINGRU_TYPES:
        return MinGRU(prefix, c.width, m.width)
    if layer.type == LATENT_ATTENTION:
        return LatentAttention(prefix, c.width, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, c.norm_eps,
                               RotaryInterleaved(m.rot_dims, m.rot_base), m.window)
    raise ValueError(layer.type)


def _feed_forward(c: VisadraConfig, f: FeedForwardSizes, prefix: str):
    if f.kind == DENSE:
        return GatedMLP(prefix, c.width, f.ff, names=_FF_NAMES, to_residual=False)
    shared = GatedMLP(prefix + "shared.", c.width, f.shared_ff, names=_FF_NAMES, to_residual=False) if f.shared_ff else None
    return RoutedMLP(prefix, c.width, f.ff, f.experts, f.top, shared)


def build_visadra(config: VisadraConfig) -> DecoderLM:
    c = config
    scalar_norm = lambda name: RMSNorm(name, c.width, c.norm_eps, scalar=True)
    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        ff = _feed_forward(c, layer.mlp, p + "mlp.") if layer.mlp is not None else None
        blocks.append(PostNormBlock(scalar_norm(p + "norm1"), _mixer(c, layer, p + "mix."),
                                    scalar_norm(p + "norm2") if ff is not None else None, ff))
    return DecoderLM(
        config=c,
        embedding=Embedding("embed", c.vocab, c.width, scale=c.embedding_scale),
        blocks=blocks,
        plan=[PlanEntry(i) for i in range(len(blocks))],
        final_norm=scalar_norm("final.norm"),
        head=Linear(["head"], c.width, [c.vocab]),
        tied_head=False,
        logit_scale=c.logit_scale,
    )


register_architecture(VisadraConfig.ARCHITECTURE, VisadraConfig, build_visadra)
