"""Kezasun: how its configuration becomes parts.

The layers are listed one by one in the configuration; layer i's tensors start with `l<i>.`,
its mixer's with `l<i>.mix.`, its feed-forward's with `l<i>.mlp.`.  Every layer is a block whose
two sublayers read the same norm (gain 1 + weight) and whose sum enters the residual stream
times `residual_mult`; the mixer is a `wkv` recurrence or windowed attention with a sink, a gate
per head and, for some layers, the keys and values of an earlier layer (that layer's plan
entry then reads the other's cache and writes none); the feed-forward is routed with a
group-limited choice and identity experts, or absent.
"""
from __future__ import annotations

from ..config.kezasun_config import ATTENTION, WKV, KezasunConfig, KezasunLayer, RoutedSizes
from ..config.registry import register_architecture
from ..parts import (Embedding, GroupLimitedMLP, Linear, NoPositionEncoding, ParallelBlock, RMSNorm, RotaryHalfSplit,
                     SinkAttention, WKVMixer)
from .decoder import DecoderLM, PlanEntry


def _cache_windows(c: KezasunConfig):
    """For every attention layer that makes keys and values: what its cache has to keep, the
    largest window of the layers that read it (SinkAttention.UNBOUNDED if one sees everything)."""
    out = {}
    for i, layer in enumerate(c.layers):
        if layer.type != ATTENTION:
            continue
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        w = layer.mixer.window
        if owner in out and out[owner] is SinkAttention.UNBOUNDED:
            continue
        if w is None:
            out[owner] = SinkAttention.UNBOUNDED
        else:
            out[owner] = max(w, out.get(owner, 0))
    return out


def _mixer(c: KezasunConfig, layer: KezasunLayer, prefix: str, cache_window):
    m = layer.mixer
    if layer.type == WKV:
        if m.decay_rank is None:
            raise ValueError("the decay's inner rank is not known yet: it is read from the checkpoint's shapes "
                             "(KezasunConfig.with_tensor_shapes) or given as `decay_rank`")
        return WKVMixer(prefix, c.width, m.heads, m.dim, m.decay_rank, c.norm_eps)
    position = (RotaryHalfSplit(m.dim, m.rot_base, m.rot_dims, scaling=m.rot_scaling) if m.rot_dims
                else NoPositionEncoding())
    return SinkAttention(prefix, c.width, m.heads, m.kv_heads, m.dim, m.vdim, position, c.norm_eps, m.scale,
                         window=m.window, sink=0.0, own_kv=m.kv_from is None, cache_window=cache_window)


def _feed_forward(c: KezasunConfig, f: RoutedSizes, prefix: str):
    return GroupLimitedMLP(prefix, c.width, f.ff, f.experts, f.top, f.identity, f.groups, f.groups_kept)


def build_kezasun(config: KezasunConfig) -> DecoderLM:
    c = config
    norm = lambda name: RMSNorm(name, c.width, c.norm_eps, one_plus=True)
    windows = _cache_windows(c)
    blocks, plan = [], []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        ff = _feed_forward(c, layer.mlp, p + "mlp.") if layer.mlp is not None else None
        blocks.append(ParallelBlock(norm(p + "norm1"), _mixer(c, layer, p + "mix.", windows.get(i)), ff, c.residual_mult))
        src = layer.mixer.kv_from if layer.type == ATTENTION else None
        plan.append(PlanEntry(i) if src is None else PlanEntry(i, cache=src, writes=False))
    return DecoderLM(
        config=c,
        embedding=Embedding("embed", c.vocab, c.width),
        blocks=blocks,
        plan=plan,
        final_norm=norm("final.norm"),
        head=Linear(["head"], c.width, [c.vocab]),
        tied_head=False,
    )


register_architecture(KezasunConfig.ARCHITECTURE, KezasunConfig, build_kezasun)
